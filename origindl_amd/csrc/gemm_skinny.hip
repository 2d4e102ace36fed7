// Products with a very narrow output side — a classifier layer, x[M,K] . w[K,N] with N <= 16 (the MLP's 1000 -> 10
// layer: src/nn/layers/linear.cpp:80-106 forward, src/operators/math/mat_mul.cpp:123-182 backward). A 64-wide MFMA tile
// would multiply 54 columns of padding and the product would need K slices plus a launch that adds them; here each of the
// three products is a handful of fused multiply-adds per loaded value on the vector ALUs, one launch forward and one
// launch for both gradients, no workspace.
//   forward   y[m][n]  = act(sum_k x[m][k] w[k][n] + b[n])    a workgroup per four rows, threads strided over k
//   gx[m][k]  = sum_n gy[m][n] w[k][n]                        a thread per k keeps w[k][:] in registers, walks rows
//   gw[k][n]  = sum_m x[m][k] gy[m][n]                        sixteen k a workgroup, its waves share the rows, summed in wave order
// Sums are formed in a fixed order (strided partials, then fixed-order passes through LDS): deterministic.
#include "odl_common.h"
#include "reduce_small.h"

namespace
{
constexpr int kNMax = 16;

constexpr int kFwdRows = 4;

// grid: ceil(M / 4) workgroups of 256 threads. A workgroup owns four rows; its threads stride over k together (thread t
// takes k = t, t + 256, ...), so a K of 1000 is four rounds of loads, all of them in flight at once; the partial sums
// meet in LDS and are added in two fixed-order passes.
template <int N>
__global__ __launch_bounds__(256) void skinny_fwd_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                          const float *__restrict__ bias, float *__restrict__ y, int M, int K,
                                                          int64_t ldx, int64_t ldw, int64_t ldy, int act)
{
    __shared__ float part[kFwdRows * N * 257];
    const int r0 = blockIdx.x * kFwdRows;
    const float *xr[kFwdRows];
#pragma unroll
    for (int r = 0; r < kFwdRows; ++r)
        xr[r] = x + (int64_t)(r0 + r < M ? r0 + r : M - 1) * ldx;  // (rows past the end repeat the last one, unused)
    float acc[kFwdRows][N];
#pragma unroll
    for (int r = 0; r < kFwdRows; ++r)
#pragma unroll
        for (int n = 0; n < N; ++n)
            acc[r][n] = 0.f;
#pragma unroll 4
    for (int k = threadIdx.x; k < K; k += 256)
    {
        float xv[kFwdRows], wv[N];
#pragma unroll
        for (int r = 0; r < kFwdRows; ++r)
            xv[r] = xr[r][k];
        const float *wr = w + (int64_t)k * ldw;
#pragma unroll
        for (int n = 0; n < N; ++n)
            wv[n] = wr[n];
#pragma unroll
        for (int r = 0; r < kFwdRows; ++r)
#pragma unroll
            for (int n = 0; n < N; ++n)
                acc[r][n] += xv[r] * wv[n];
    }
    // the 256 threads' partial sums of the 4 x N outputs meet in LDS: thread (output o, part q) adds the partials of
    // threads q*16 .. q*16+15 in order, then the sixteen parts of an output are added in order
#pragma unroll
    for (int r = 0; r < kFwdRows; ++r)
#pragma unroll
        for (int n = 0; n < N; ++n)
            part[(r * N + n) * 257 + threadIdx.x] = acc[r][n];
    __syncthreads();
    constexpr int kOut = kFwdRows * N;
    float s = 0.f;
    const int o = threadIdx.x >> 4, q = threadIdx.x & 15;
    if (o < kOut)
    {
        const float *p = part + o * 257 + q * 16;
#pragma unroll
        for (int i = 0; i < 16; ++i)
            s += p[i];
    }
    // (outputs 16 .. kOut-1 of a wide N: a second pass of the same threads)
    float s2 = 0.f;
    if (kOut > 16 && o + 16 < kOut)
    {
        const float *p = part + (o + 16) * 257 + q * 16;
#pragma unroll
        for (int i = 0; i < 16; ++i)
            s2 += p[i];
    }
    float s3 = 0.f, s4 = 0.f;
    if (kOut > 32 && o + 32 < kOut)
    {
        const float *p = part + (o + 32) * 257 + q * 16;
#pragma unroll
        for (int i = 0; i < 16; ++i)
            s3 += p[i];
    }
    if (kOut > 48 && o + 48 < kOut)
    {
        const float *p = part + (o + 48) * 257 + q * 16;
#pragma unroll
        for (int i = 0; i < 16; ++i)
            s4 += p[i];
    }
    __syncthreads();
    part[threadIdx.x] = s, part[256 + threadIdx.x] = s2, part[512 + threadIdx.x] = s3, part[768 + threadIdx.x] = s4;
    __syncthreads();
    if (threadIdx.x < kOut)
    {
        const int oo = threadIdx.x;
        const float *p = part + (oo >> 4) * 256 + (oo & 15) * 16;
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i)
            t += p[i];
        const int r = oo / N, n = oo - r * N;
        if (r0 + r < M)
            y[(int64_t)(r0 + r) * ldy + n] = odl::apply_act(t + (bias ? bias[n] : 0.f), act);
    }
}

struct SkinnyBwd
{
    const float *x, *w, *gy;
    float *gx, *gw, *gb;
    int M, K;
    int gb_quads;     // the bias gradient's column sums take four columns a lane (N % 4 == 0 and gy 16-byte aligned)
    int gw_blocks;    // workgroups [gx_blocks, gx_blocks + gw_blocks) form gw; one more, if gb is wanted, the bias gradient
    int gx_blocks;    // workgroups [0, gx_blocks) form gx
    int gx_ktiles;    // tiles of 1024 k per row group
    int rows_per;     // rows of gx a workgroup walks
};

constexpr int kGyRows = 512;  // rows of gy a gw workgroup keeps in LDS at a time

// Both gradients in one launch of 1024-thread workgroups. gx part: workgroup (row group, k tile), a thread per k keeps
// w[k][:] in registers and walks the group's rows (gy through LDS). gw part: workgroup per 16 k, gy through LDS in blocks
// of 512 rows (below).
template <int N>
__global__ __launch_bounds__(1024) void skinny_bwd_kernel(SkinnyBwd g)
{
    __shared__ float buf[16 * 64 * N];  // gy rows while summing, the sixteen waves' partial sums afterwards
    float *gys = buf;
    float(*part)[64][N] = reinterpret_cast<float(*)[64][N]>(buf);
    static_assert(kGyRows <= 16 * 64, "a block of gy rows must fit the buffer");
    const int bid = blockIdx.x;
    if (bid >= g.gx_blocks + g.gw_blocks)
    {
        // the bias gradient of the layer, gb[n] = sum over the rows of gy[:, n]: the column sum Mat::sum_to would run as a
        // launch of its own (reduce_small.h), here by this workgroup's first 256 threads — the same additions in the same
        // order
        static_assert(sizeof(buf) >= sizeof(odl::ColSumSmall<1, 16>::Sums), "the group sums must fit the buffer");
        static_assert(N % 4 != 0 || sizeof(buf) >= sizeof(odl::ColSumSmall<4, 8>::Sums), "the group sums must fit the buffer");
        const unsigned tid = threadIdx.x;
        if (N % 4 == 0 && g.gb_quads)
        {
            auto &sh = *reinterpret_cast<typename odl::ColSumSmall<4, 8>::Sums *>(buf);
            if (tid < 256)
                odl::ColSumSmall<4, 8>::accumulate(g.gy, g.M, N, 0, 0, tid, sh);
            __syncthreads();
            if (tid < 256)
                odl::ColSumSmall<4, 8>::finish(g.gb, N, 0, 0, tid, sh);
        }
        else
        {
            auto &sh = *reinterpret_cast<typename odl::ColSumSmall<1, 16>::Sums *>(buf);
            if (tid < 256)
                odl::ColSumSmall<1, 16>::accumulate(g.gy, g.M, N, 0, 0, tid, sh);
            __syncthreads();
            if (tid < 256)
                odl::ColSumSmall<1, 16>::finish(g.gb, N, 0, 0, tid, sh);
        }
        return;
    }
    if (bid < g.gx_blocks)
    {
        const int kt = bid % g.gx_ktiles, rg = bid / g.gx_ktiles;
        const int k = kt * 1024 + (int)threadIdx.x;
        const bool kok = k < g.K;
        float wr[N];
#pragma unroll
        for (int n = 0; n < N; ++n)
            wr[n] = kok ? g.w[(int64_t)k * N + n] : 0.f;
        const int m0 = rg * g.rows_per, m1 = m0 + g.rows_per < g.M ? m0 + g.rows_per : g.M;
        // the group's rows of gy through LDS: every lane of a wave wants the same N values per row, which LDS hands out
        // in one pass (as global loads they would hold the address unit as long as loads of 64 different addresses)
        for (int mb = m0; mb < m1; mb += kGyRows)
        {
            const int rows = m1 - mb < kGyRows ? m1 - mb : kGyRows;
            __syncthreads();
            for (int e = threadIdx.x; e < rows * N; e += 1024)
                gys[e] = g.gy[(int64_t)mb * N + e];
            __syncthreads();
            if (kok)
            {
#pragma unroll 4
                for (int m = 0; m < rows; ++m)
                {
                    const float *gr = gys + m * N;
                    float s = 0.f;
#pragma unroll
                    for (int n = 0; n < N; ++n)
                        s += gr[n] * wr[n];
                    g.gx[(int64_t)(mb + m) * g.K + k] = s;
                }
            }
        }
        return;
    }
    // gw: sixteen k per workgroup. A wave's load covers four rows of x (lane = row j of the four, k of the sixteen): 64
    // bytes per row, and enough workgroups (K / 16) that no compute unit's address unit is the limit. Wave v takes the
    // row quads v, v + 16, ...; the four row lanes meet by two exchanges, the sixteen waves through LDS in wave order.
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int kk = lane & 15, j = lane >> 4;
    const int k = (bid - g.gx_blocks) * 16 + kk;
    const bool ok = k < g.K;
    const float *xk = g.x + (ok ? k : 0);
    float acc[N];
#pragma unroll
    for (int n = 0; n < N; ++n)
        acc[n] = 0.f;
    for (int mb = 0; mb < g.M; mb += kGyRows)
    {
        const int rows = g.M - mb < kGyRows ? g.M - mb : kGyRows;
        // this wave's eight row quads of the block (512 rows = 128 quads over 16 waves), asked for before gy is staged
        float xv[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
        {
            const int m = 4 * (wave + 16 * i) + j;
            xv[i] = (ok && m < rows) ? xk[(int64_t)(mb + m) * g.K] : 0.f;
        }
        __syncthreads();  // the previous block of gy has been read
        for (int e = threadIdx.x; e < rows * N; e += 1024)
            gys[e] = g.gy[(int64_t)mb * N + e];
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 8; ++i)
        {
            const int m = 4 * (wave + 16 * i) + j;
            if (m < rows)
            {
                const float *gr = gys + m * N;
#pragma unroll
                for (int n = 0; n < N; ++n)
                    acc[n] += xv[i] * gr[n];
            }
        }
    }
#pragma unroll
    for (int n = 0; n < N; ++n)
    {
        acc[n] += __shfl_xor(acc[n], 16, 64);
        acc[n] += __shfl_xor(acc[n], 32, 64);
    }
    __syncthreads();  // every wave is done with the gy rows
    if (j == 0)
    {
#pragma unroll
        for (int n = 0; n < N; ++n)
            part[wave][kk][n] = acc[n];
    }
    __syncthreads();
    if (threadIdx.x < 16 * N)
    {
        const int kl = threadIdx.x / N, n = threadIdx.x - kl * N;
        float s = part[0][kl][n];
#pragma unroll
        for (int v = 1; v < 16; ++v)
            s += part[v][kl][n];
        const int ko = (bid - g.gx_blocks) * 16 + kl;
        if (ko < g.K)
            g.gw[(int64_t)ko * N + n] = s;
    }
}

template <int N>
void launch_fwd(const float *x, const float *w, const float *b, float *y, int64_t M, int64_t K, int64_t ldx, int64_t ldw,
                int64_t ldy, int act, hipStream_t st)
{
    hipLaunchKernelGGL(skinny_fwd_kernel<N>, dim3((unsigned)odl::ceil_div(M, kFwdRows)), dim3(256), 0, st, x, w, b, y, (int)M, (int)K, ldx,
                       ldw, ldy, act);
}

template <int N>
void launch_bwd(const SkinnyBwd &g, hipStream_t st)
{
    hipLaunchKernelGGL(skinny_bwd_kernel<N>, dim3((unsigned)(g.gx_blocks + g.gw_blocks + (g.gb ? 1 : 0))), dim3(1024), 0, st, g);
}
}  // namespace

namespace odl
{
// x[M,K] . w[K,N] with N <= 16 and a K long enough to be worth a wave per row pair
bool skinny_ok(int64_t M, int64_t N, int64_t K)
{
    return N >= 1 && N <= kNMax && K >= 128 && M >= 1 && M < (1ll << 28) && K < (1ll << 28);
}

#define ODL_SKINNY_N(CALL)                                                  \
    switch (N)                                                              \
    {                                                                       \
        case 1: CALL(1); break;                                             \
        case 2: CALL(2); break;                                             \
        case 3: CALL(3); break;                                             \
        case 4: CALL(4); break;                                             \
        case 5: CALL(5); break;                                             \
        case 6: CALL(6); break;                                             \
        case 7: CALL(7); break;                                             \
        case 8: CALL(8); break;                                             \
        case 9: CALL(9); break;                                             \
        case 10: CALL(10); break;                                           \
        case 11: CALL(11); break;                                           \
        case 12: CALL(12); break;                                           \
        case 13: CALL(13); break;                                           \
        case 14: CALL(14); break;                                           \
        case 15: CALL(15); break;                                           \
        default: CALL(16); break;                                           \
    }

// y = act(x . w + bias); rows of x, w, y are ldx, ldw, ldy floats apart
int skinny_forward(const float *x, const float *w, const float *bias, float *y, int64_t M, int64_t N, int64_t K, int64_t ldx,
                   int64_t ldw, int64_t ldy, int act, hipStream_t st)
{
#define ODL_CALL(NV) launch_fwd<NV>(x, w, bias, y, M, K, ldx, ldw, ldy, act, st)
    ODL_SKINNY_N(ODL_CALL)
#undef ODL_CALL
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

// gx[M,K] = gy[M,N] . w[K,N]^T and gw[K,N] = x[M,K]^T . gy[M,N] (dense operands), either output may be null
// gb (may be null): the bias gradient gy summed over its rows, as one more workgroup of the launch; only for sizes that
// Mat::sum_to would sum in one small launch (skinny_bias_ok), whose bits it then gives
bool skinny_bias_ok(int64_t M, int64_t N)
{
    return N <= 16 && small_cols(1, M, N);
}

int skinny_backward(const float *x, const float *w, const float *gy, float *gx, float *gw, float *gb, int64_t M, int64_t K,
                    int64_t N, hipStream_t st)
{
    if (gb && !skinny_bias_ok(M, N))
        return fail(ODL_ERR_RUNTIME, "linear_backward: the bias gradient of this size does not ride in the classifier launch");
    SkinnyBwd g{};
    g.x = x, g.w = w, g.gy = gy, g.gx = gx, g.gw = gw, g.gb = gb, g.M = (int)M, g.K = (int)K;
    g.gb_quads = (N % 4 == 0 && reinterpret_cast<uintptr_t>(gy) % 16 == 0) ? 1 : 0;
    g.gw_blocks = gw ? (int)ceil_div(K, 16) : 0;
    g.gx_blocks = 0, g.gx_ktiles = (int)ceil_div(K, 1024), g.rows_per = 2;
    if (gx)
    {
        // a workgroup re-reads w once per group of rows: eight rows or more, and no more workgroups than two per compute unit
        int64_t rows = ceil_div(M * g.gx_ktiles, 2 * (int64_t)device_cus());
        rows = rows < 8 ? 8 : rows;
        g.rows_per = (int)rows;
        g.gx_blocks = (int)(ceil_div(M, rows) * g.gx_ktiles);
    }
#define ODL_CALL(NV) launch_bwd<NV>(g, st)
    ODL_SKINNY_N(ODL_CALL)
#undef ODL_CALL
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}
}  // namespace odl
