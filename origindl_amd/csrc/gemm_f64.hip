// Float64 GEMM on v_mfma_f64_16x16x4_f64 (peak 78.6 TFLOP/s): C[M,N] = op(A)[M,K] . op(B)[K,N], row-major, any of
// NN / NT / TN / TT, optionally a batch of independent products. The reference's device matmul is a template over
// the element type and serves double through the same kernels as float (src/mat/origin/cuda/math/mat_mul.cu:1911-1954;
// CPU form src/mat/origin/cpu/math/matmul.cpp:27-41, one `sum += a * b` chain per output in K order).
//
// A workgroup of eight waves owns a 128x128 tile; a wave 32x64 of it as 2x4 blocks of 16x16 (eight accumulators of
// four doubles a lane). K goes by in slabs of 16 through two LDS buffers, both operands stored K-major ([k][m], [k][n])
// whatever their layout in memory, so every fragment is one 8-byte LDS read of 16 consecutive doubles per K row: the
// slab after the current one travels global memory -> registers while the current one is multiplied, and is written to
// the other buffer before the barrier. Rows, columns and K positions outside the matrices are staged as zeros.
#include "odl_common.h"

typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));

namespace
{
constexpr int kBM = 128, kBN = 128, kBK = 16, kThreads = 512;

struct DArgs
{
    const double *A, *B;
    double *C;
    int64_t lda, ldb, ldc, sa, sb, sc;  // leading dimensions; distances between the products of a batch
    int M, N, K;
    int tiles_n;
};

// One operand's 128 x 16 slab: four doubles a thread. KC: the operand is K-contiguous in memory (A as [M,K], B as
// [N,K]): a thread takes four consecutive K positions of one row; otherwise ([K,M], [K,N]) four consecutive rows of one K.
template <bool KC>
struct Stage
{
    double v[4];
    __device__ inline void load(const double *p, int64_t ld, int r0, int rows, int k0, int K)
    {
        const int t = threadIdx.x;
        if (KC)
        {
            const int r = r0 + (t >> 2), k = k0 + 4 * (t & 3);
            const double *q = p + (int64_t)r * ld + k;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                v[j] = (r < rows && k + j < K) ? q[j] : 0.0;
        }
        else
        {
            const int k = k0 + (t >> 5), r = r0 + 4 * (t & 31);
            const double *q = p + (int64_t)k * ld + r;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                v[j] = (k < K && r + j < rows) ? q[j] : 0.0;
        }
    }
    __device__ inline void store(double *s) const  // s: [kBK][128]
    {
        const int t = threadIdx.x;
        if (KC)
        {
            const int r = t >> 2, k = 4 * (t & 3);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                s[(k + j) * 128 + r] = v[j];
        }
        else
        {
            const int k = t >> 5, r = 4 * (t & 31);
            *reinterpret_cast<f64x2 *>(s + k * 128 + r) = f64x2{v[0], v[1]};
            *reinterpret_cast<f64x2 *>(s + k * 128 + r + 2) = f64x2{v[2], v[3]};
        }
    }
};

template <bool TA, bool TB>
__global__ __launch_bounds__(kThreads) void dgemm_kernel(DArgs g)
{
    __shared__ double As[2][kBK * kBM], Bs[2][kBK * kBN];
    const int tile = blockIdx.x;
    const int tm = tile / g.tiles_n, tn = tile - tm * g.tiles_n;
    const int m0 = tm * kBM, n0 = tn * kBN;
    const double *A = g.A + (int64_t)blockIdx.y * g.sa, *B = g.B + (int64_t)blockIdx.y * g.sb;
    double *C = g.C + (int64_t)blockIdx.y * g.sc;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;  // the wave's 32 rows and 64 columns of the tile
    const int l16 = lane & 15, lk = lane >> 4;

    Stage<!TA> sa;  // A as stored [M,K] is K-contiguous
    Stage<TB> sb;   // B as stored [N,K] (transposed) is K-contiguous
    f64x4 acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            acc[i][j] = f64x4{0.0, 0.0, 0.0, 0.0};

    const int slabs = (g.K + kBK - 1) / kBK;
    sa.load(A, g.lda, m0, g.M, 0, g.K);
    sb.load(B, g.ldb, n0, g.N, 0, g.K);
    sa.store(As[0]);
    sb.store(Bs[0]);
    __syncthreads();
    for (int s = 0; s < slabs; ++s)
    {
        const int cur = s & 1;
        if (s + 1 < slabs)
        {
            sa.load(A, g.lda, m0, g.M, (s + 1) * kBK, g.K);
            sb.load(B, g.ldb, n0, g.N, (s + 1) * kBK, g.K);
        }
        const double *as = As[cur] + wm * 32 + l16, *bs = Bs[cur] + wn * 64 + l16;
#pragma unroll
        for (int kk = 0; kk < kBK; kk += 4)
        {
            double a[2], b[4];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                a[i] = as[(kk + lk) * 128 + i * 16];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                b[j] = bs[(kk + lk) * 128 + j * 16];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (s + 1 < slabs)
        {
            sa.store(As[cur ^ 1]);
            sb.store(Bs[cur ^ 1]);
        }
        __syncthreads();
    }
    // accumulator element q of a lane: row 4 * q + lane / 16, column lane % 16 of the block
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            const int col = n0 + wn * 64 + j * 16 + l16;
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const int row = m0 + wm * 32 + i * 16 + 4 * q + lk;
                if (row < g.M && col < g.N)
                    C[(int64_t)row * g.ldc + col] = acc[i][j][q];
            }
        }
}
}  // namespace

extern "C" int odl_hip_dgemm(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const double *A, int64_t lda,
                             const double *B, int64_t ldb, double *C, int64_t ldc, int64_t batch, int64_t stride_a,
                             int64_t stride_b, int64_t stride_c, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(M >= 0 && N >= 0 && K >= 0 && batch >= 0, "dgemm: negative extent");
    if (M == 0 || N == 0 || batch == 0)
        return ODL_OK;
    ODL_REQUIRE(C && (K == 0 || (A && B)), "dgemm: null operand");
    ODL_REQUIRE(lda >= (trans_a ? M : K) && ldb >= (trans_b ? K : N) && ldc >= N, "dgemm: a leading dimension is shorter than its row");
    ODL_REQUIRE(M < (1ll << 30) && N < (1ll << 30) && K < (1ll << 30) && batch < 65536, "dgemm: extent too large");
    const int64_t tm = odl::ceil_div(M, kBM), tn = odl::ceil_div(N, kBN);
    ODL_REQUIRE(tm * tn < (1ll << 31), "dgemm: too many tiles");
    DArgs g{A, B, C, lda, ldb, ldc, stride_a, stride_b, stride_c, (int)M, (int)N, (int)K, (int)tn};
    const dim3 grid((unsigned)(tm * tn), (unsigned)batch), block(kThreads);
    hipStream_t st = odl::as_stream(stream);
    if (!trans_a && !trans_b)
        hipLaunchKernelGGL((dgemm_kernel<false, false>), grid, block, 0, st, g);
    else if (!trans_a)
        hipLaunchKernelGGL((dgemm_kernel<false, true>), grid, block, 0, st, g);
    else if (!trans_b)
        hipLaunchKernelGGL((dgemm_kernel<true, false>), grid, block, 0, st, g);
    else
        hipLaunchKernelGGL((dgemm_kernel<true, true>), grid, block, 0, st, g);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}
