// Convolution path of the backend: im2col / col2im in both of the reference's layouts, and conv2d forward /
// backward composed from them and the MFMA GEMM (src/mat/origin/cpu/conv/conv2d.cpp:39-599 is the behaviour
// being matched; nothing of the reference's CUDA design is kept).
//
//   forward : col = im2col(x); y^T[OC, N*OH*OW] = W2d[OC,K] . col^T  — computed as an "NT" GEMM whose epilogue
//             adds the bias per row and stores straight into NCHW, so neither the W transpose, nor the
//             broadcast bias matrix, nor the NHWC->NCHW pass of the reference exist here.
//   backward: gW[OC,K] = gy2d^T . col as a "TN" GEMM with split-K (the reduction runs over N*OH*OW rows);
//             gx = col2im(gy2d . W2d); gb = per-channel sum of gy. gy2d is gy's buffer read as a row-major
//             [N*OH*OW, OC] matrix exactly as it lies (conv2d.cpp:548) — free on the GPU: it is the same pointer.
//   col2im is a gather: one thread owns one image pixel and adds its taps in ascending (kh, kw) order, which
//   is the order in which the reference's scatter loop reaches that pixel — bit-identical sums, no atomics.
#include "odl_common.h"

namespace odl
{
int sgemm_launch(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                 const float *B, int64_t ldb, float *C, int64_t ldc, const float *bias, int epi, int64_t P,
                 int split_k, void *workspace, size_t workspace_bytes, hipStream_t st);
size_t sgemm_workspace(int64_t M, int64_t N, int64_t K, int split_k);
bool conv_implicit_forward_ok(const float *w, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                              int64_t OH, int64_t OW);
bool conv_implicit_wgrad_ok(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                            int64_t OH, int64_t OW);
bool conv_implicit_dgrad_ok(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                            int SH, int SW);
size_t conv_implicit_wgrad_workspace(int64_t N, int64_t C, int64_t OC, int KH, int KW, int64_t OH, int64_t OW);
size_t conv_implicit_dgrad_workspace(int64_t C, int64_t OC, int KH, int KW);
int conv_implicit_forward(const float *x, const float *w, const float *b, float *y, int64_t N, int64_t C, int64_t H,
                          int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, int64_t OH, int64_t OW,
                          hipStream_t st);
int conv_implicit_wgrad(const float *gy, const float *x, float *gw, int64_t N, int64_t C, int64_t H, int64_t W,
                        int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, int64_t OH, int64_t OW,
                        void *workspace, size_t workspace_bytes, hipStream_t st);
int conv_implicit_dgrad(const float *gy, const float *w, float *gx, int64_t N, int64_t C, int64_t H, int64_t W,
                        int64_t OC, int KH, int KW, int PH, int PW, int64_t OH, int64_t OW, void *workspace,
                        size_t workspace_bytes, hipStream_t st);
int sum_nchw_channels_launch(const float *gy, int64_t N, int64_t OC, int64_t P, float *gb, void *workspace,
                             size_t workspace_bytes, hipStream_t st);
size_t sum_nchw_channels_workspace(int64_t N, int64_t OC, int64_t P);
}  // namespace odl

typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace
{
struct ConvGeom
{
    int64_t N, C, H, W;
    int KH, KW, SH, SW, PH, PW;
    int64_t OH, OW;
};

inline int64_t outsize(int64_t in, int k, int s, int p)
{
    return (in + 2 * (int64_t)p - k) / s + 1;  // include/origin/utils/conv_utils.h
}

inline size_t align256(size_t b)
{
    return (b + 255) & ~(size_t)255;
}

// Workgroups are dealt round-robin over the 8 XCDs (one L2 each); unfolding the id this way gives every XCD
// a contiguous band of virtual blocks, so neighbouring tiles — which read the same image lines — share an L2.
__device__ inline int64_t xcd_contiguous_block(int64_t bid, int64_t nb)
{
    const int64_t xcd = bid % 8, loc = bid / 8;
    const int64_t full = nb / 8, rem = nb % 8;
    return xcd * full + (xcd < rem ? xcd : rem) + loc;
}

constexpr int kImPix = 64;   // pixels (col rows) per tile
constexpr int kImCk  = 144;  // col columns per tile at most

// col[m][ck] (m = (n,oh,ow), ck = (c,kh,kw)), tile = 64 consecutive rows x up to 144 columns.
// Read phase: for one ck at a time the 64 lanes of a wave read 64 consecutive pixels — contiguous image addresses
// (stride SW) — into an LDS tile; write phase: the tile leaves row by row with 16-byte stores. The image is read
// through coalesced loads and the 9x larger col matrix is written through full-width stores.
constexpr int kImThreads = 512;
__global__ __launch_bounds__(kImThreads) void im2col_matrix_kernel(const float *__restrict__ img,
                                                                    float *__restrict__ col, ConvGeom g, int tk,
                                                                    int ktiles, int64_t mtiles)
{
    __shared__ float sh[kImPix][kImCk + 1];
    const int64_t vb = xcd_contiguous_block(blockIdx.x, mtiles * ktiles);
    const int64_t mt = vb / ktiles;
    const int kt = (int)(vb % ktiles);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t M = g.N * g.OH * g.OW;
    const int K = (int)(g.C * g.KH * g.KW);
    const int64_t m = mt * kImPix + lane;
    const bool live = m < M;
    const int64_t mm = live ? m : 0;
    const int ow = (int)(mm % g.OW), oh = (int)((mm / g.OW) % g.OH);
    const int64_t n = mm / (g.OW * g.OH);
    const int h0 = oh * g.SH - g.PH, w0 = ow * g.SW - g.PW;
    const float *base = img + n * g.C * g.H * g.W;
    const int ck0 = kt * tk;
    const int ckn = (K - ck0 < tk) ? K - ck0 : tk;
    const int H = (int)g.H, W = (int)g.W;
    constexpr int U = 9;  // independent loads in flight per lane
    constexpr int NW = kImThreads / 64;
    for (int j = wave; j < ckn; j += NW * U)
    {
        float v[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
        {
            const int ck = ck0 + j + NW * u;  // wave-uniform
            const int kw = ck % g.KW, t2 = ck / g.KW;
            const int kh = t2 % g.KH, c = t2 / g.KH;
            const int h = h0 + kh, w = w0 + kw;
            v[u] = 0.f;
            if (j + NW * u < ckn && live && h >= 0 && h < H && w >= 0 && w < W)
                v[u] = base[((int64_t)c * H + h) * W + w];
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (j + NW * u < ckn)
                sh[lane][j + NW * u] = v[u];
    }
    __syncthreads();
    const int64_t row0 = mt * kImPix;
    if ((ckn & 3) == 0 && (K & 3) == 0 && (ck0 & 3) == 0 && (reinterpret_cast<uintptr_t>(col) & 15) == 0)
    {
        const int q4 = ckn >> 2;
        for (int e = threadIdx.x; e < kImPix * q4; e += kImThreads)
        {
            const int row = e / q4, q = e % q4;
            if (row0 + row < M)
            {
                f32x4 o = {sh[row][4 * q], sh[row][4 * q + 1], sh[row][4 * q + 2], sh[row][4 * q + 3]};
                *reinterpret_cast<f32x4 *>(col + (row0 + row) * K + ck0 + 4 * q) = o;
            }
        }
    }
    else
    {
        for (int e = threadIdx.x; e < kImPix * ckn; e += kImThreads)
        {
            const int row = e / ckn, j = e % ckn;
            if (row0 + row < M)
                col[(row0 + row) * K + ck0 + j] = sh[row][j];
        }
    }
}

// col[n][c][kh][kw][oh][ow]; one thread per element, consecutive threads along ow.
__global__ void im2col_6d_kernel(const float *__restrict__ img, float *__restrict__ col, ConvGeom g)
{
    const int64_t total = g.N * g.C * g.KH * g.KW * g.OH * g.OW;
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total)
        return;
    int64_t r = t;
    const int64_t ow = r % g.OW;
    r /= g.OW;
    const int64_t oh = r % g.OH;
    r /= g.OH;
    const int kw = (int)(r % g.KW);
    r /= g.KW;
    const int kh = (int)(r % g.KH);
    r /= g.KH;  // r = n*C + c
    const int64_t h = oh * g.SH + kh - g.PH, w = ow * g.SW + kw - g.PW;
    col[t] = (h >= 0 && h < g.H && w >= 0 && w < g.W) ? img[(r * g.H + h) * g.W + w] : 0.f;
}

// Taps of one image pixel are added in ascending (kh, kw), starting from +0.0f like the reference's zero-filled
// padded image (conv2d.cpp:316-349): bit-identical sums, no atomics.
//
// 6-D layout [N,C,KH,KW,OH,OW]: one thread per pixel, lanes along w — reads and writes are contiguous.
__global__ void col2im_6d_kernel(const float *__restrict__ col, float *__restrict__ img, ConvGeom g)
{
    const int64_t total = g.N * g.C * g.H * g.W;
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total)
        return;
    const int64_t w = t % g.W, h = (t / g.W) % g.H;
    const int64_t nc = t / (g.W * g.H);
    float acc = 0.f;
    for (int kh = 0; kh < g.KH; ++kh)
    {
        const int64_t hp = h + g.PH - kh;
        if (hp < 0 || hp % g.SH != 0)
            continue;
        const int64_t oh = hp / g.SH;
        if (oh >= g.OH)
            continue;
        for (int kw = 0; kw < g.KW; ++kw)
        {
            const int64_t wp = w + g.PW - kw;
            if (wp < 0 || wp % g.SW != 0)
                continue;
            const int64_t ow = wp / g.SW;
            if (ow >= g.OW)
                continue;
            acc += col[(((nc * g.KH + kh) * g.KW + kw) * g.OH + oh) * g.OW + ow];
        }
    }
    img[t] = acc;
}

// Matrix layout [N*OH*OW, C*KH*KW]: a workgroup owns 64 channels x 16 consecutive w of one image row. Lanes run
// along the channel, where a col row is nearly contiguous (KH*KW floats apart), each thread sums 4 pixels, and the
// 64x16 result tile is turned through LDS so that the image is written in 64-byte runs along w.
template <int CKH, int CKW>
__global__ __launch_bounds__(256) void col2im_matrix_kernel(const float *__restrict__ col, float *__restrict__ img,
                                                             ConvGeom g, int wtiles, int ctiles)
{
    __shared__ float sh[64][17];
    const int KH = CKH > 0 ? CKH : g.KH, KW = CKW > 0 ? CKW : g.KW;
    const int64_t nb = g.N * g.H * wtiles * ctiles;
    int64_t vb = xcd_contiguous_block(blockIdx.x, nb);
    const int ct = (int)(vb % ctiles);
    vb /= ctiles;
    const int wt = (int)(vb % wtiles);
    vb /= wtiles;
    const int h = (int)(vb % g.H);
    const int64_t n = vb / g.H;
    const int cl = threadIdx.x & 63, wq = threadIdx.x >> 6;
    const int c = ct * 64 + cl;
    const int K = (int)(g.C * KH * KW);
    const int W = (int)g.W, OH = (int)g.OH, OW = (int)g.OW;
    if (c < g.C)
    {
        const float *cbase = col + (int64_t)c * KH * KW;
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            const int w = wt * 16 + wq * 4 + i;
            float acc = 0.f;
            if (w < W)
            {
                if (CKH > 0)
                {
                    // all taps are loaded (or zeroed) first, then added in ascending (kh, kw)
                    float v[(CKH > 0 ? CKH : 1) * (CKW > 0 ? CKW : 1)];
#pragma unroll
                    for (int kh = 0; kh < CKH; ++kh)
                    {
                        const int hp = h + g.PH - kh;
                        const int oh = hp / g.SH;
                        const bool hok = hp >= 0 && hp % g.SH == 0 && oh < OH;
#pragma unroll
                        for (int kw = 0; kw < CKW; ++kw)
                        {
                            const int wp = w + g.PW - kw;
                            const int ow = wp / g.SW;
                            const bool ok = hok && wp >= 0 && wp % g.SW == 0 && ow < OW;
                            v[kh * CKW + kw] = ok ? cbase[((n * OH + oh) * OW + ow) * K + kh * CKW + kw] : 0.f;
                        }
                    }
                    // a skipped tap contributes nothing in the reference; adding +0.0f instead leaves every
                    // partial sum unchanged because the accumulator starts at +0.0f and never becomes -0.0f
#pragma unroll
                    for (int q = 0; q < CKH * CKW; ++q)
                        acc += v[q];
                }
                else
                {
                    for (int kh = 0; kh < KH; ++kh)
                    {
                        const int hp = h + g.PH - kh;
                        if (hp < 0 || hp % g.SH != 0)
                            continue;
                        const int oh = hp / g.SH;
                        if (oh >= OH)
                            continue;
                        for (int kw = 0; kw < KW; ++kw)
                        {
                            const int wp = w + g.PW - kw;
                            if (wp < 0 || wp % g.SW != 0)
                                continue;
                            const int ow = wp / g.SW;
                            if (ow >= OW)
                                continue;
                            acc += cbase[((n * OH + oh) * OW + ow) * K + kh * KW + kw];
                        }
                    }
                }
            }
            sh[cl][wq * 4 + i] = acc;
        }
    }
    __syncthreads();
    const int row = threadIdx.x >> 2, part = threadIdx.x & 3;
    const int cc = ct * 64 + row;
    const int wbase = wt * 16 + part * 4;
    if (cc < g.C && wbase < W)
    {
        float *dst = img + ((n * g.C + cc) * g.H + h) * W + wbase;
        if ((W & 3) == 0 && (reinterpret_cast<uintptr_t>(img) & 15) == 0)
        {
            f32x4 o = {sh[row][part * 4], sh[row][part * 4 + 1], sh[row][part * 4 + 2], sh[row][part * 4 + 3]};
            *reinterpret_cast<f32x4 *>(dst) = o;
        }
        else
            for (int i = 0; i < 4 && wbase + i < W; ++i)
                dst[i] = sh[row][part * 4 + i];
    }
}

int make_geom(ConvGeom &g, const char *who, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW,
              int PH, int PW)
{
    ODL_REQUIRE(N >= 0 && C >= 0 && H > 0 && W > 0, "%s: bad image shape (%lld,%lld,%lld,%lld)", who, (long long)N,
                (long long)C, (long long)H, (long long)W);
    ODL_REQUIRE(KH > 0 && KW > 0 && SH > 0 && SW > 0 && PH >= 0 && PW >= 0, "%s: bad kernel/stride/pad", who);
    g = ConvGeom{N, C, H, W, KH, KW, SH, SW, PH, PW, outsize(H, KH, SH, PH), outsize(W, KW, SW, PW)};
    ODL_REQUIRE(g.OH > 0 && g.OW > 0,
                "%s: invalid output size OH=%lld, OW=%lld for input H=%lld, W=%lld, kernel=(%d,%d), stride=(%d,%d), "
                "pad=(%d,%d)",
                who, (long long)g.OH, (long long)g.OW, (long long)H, (long long)W, KH, KW, SH, SW, PH, PW);
    return ODL_OK;
}

int im2col_launch(const float *img, float *col, const ConvGeom &g, int to_matrix, hipStream_t st)
{
    const int64_t K = g.C * g.KH * g.KW;
    const int64_t total = g.N * g.OH * g.OW * K;
    if (total == 0)
        return ODL_OK;
    if (to_matrix)
    {
        const int tk = K < kImCk ? (int)K : kImCk;
        const int ktiles = (int)odl::ceil_div(K, tk);
        const int64_t mtiles = odl::ceil_div(g.N * g.OH * g.OW, kImPix);
        ODL_REQUIRE(mtiles * ktiles < (1ll << 31) && K < (1ll << 31), "im2col: too many tiles");
        hipLaunchKernelGGL(im2col_matrix_kernel, dim3((unsigned)(mtiles * ktiles)), dim3(kImThreads), 0, st, img, col, g,
                           tk, ktiles, mtiles);
    }
    else
    {
        hipLaunchKernelGGL(im2col_6d_kernel, dim3((unsigned)odl::ceil_div(total, 256)), dim3(256), 0, st, img, col, g);
    }
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int col2im_launch(const float *col, float *img, const ConvGeom &g, int to_matrix, hipStream_t st)
{
    const int64_t total = g.N * g.C * g.H * g.W;
    if (total == 0)
        return ODL_OK;
    if (to_matrix)
    {
        const int wtiles = (int)odl::ceil_div(g.W, 16), ctiles = (int)odl::ceil_div(g.C, 64);
        const int64_t nb = g.N * g.H * wtiles * ctiles;
        ODL_REQUIRE(nb < (1ll << 31) && g.N * g.OH * g.OW * g.C * g.KH * g.KW < (1ll << 40), "col2im: too large");
        if (g.KH == 3 && g.KW == 3)
            hipLaunchKernelGGL((col2im_matrix_kernel<3, 3>), dim3((unsigned)nb), dim3(256), 0, st, col, img, g, wtiles,
                               ctiles);
        else
            hipLaunchKernelGGL((col2im_matrix_kernel<0, 0>), dim3((unsigned)nb), dim3(256), 0, st, col, img, g, wtiles,
                               ctiles);
    }
    else
        hipLaunchKernelGGL(col2im_6d_kernel, dim3((unsigned)odl::ceil_div(total, 256)), dim3(256), 0, st, col, img, g);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}
}  // namespace

extern "C" {

int odl_hip_im2col(const float *img, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH,
                   int PW, int to_matrix, float *col, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ConvGeom g;
    int rc = make_geom(g, "im2col", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    ODL_REQUIRE(g.N * g.OH * g.OW * g.C * g.KH * g.KW < (1ll << 40), "im2col: column matrix too large");
    return im2col_launch(img, col, g, to_matrix, odl::as_stream(stream));
}

int odl_hip_col2im(const float *col, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH,
                   int PW, int to_matrix, float *img, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ConvGeom g;
    int rc = make_geom(g, "col2im", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    return col2im_launch(col, img, g, to_matrix, odl::as_stream(stream));
}

// 16-byte aligned stand-in used by the workspace queries, which see shapes only
static const float *const kAlignedProbe = reinterpret_cast<const float *>(uintptr_t(256));

size_t odl_hip_conv2d_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH,
                                      int SW, int PH, int PW)
{
    if (KH <= 0 || KW <= 0 || SH <= 0 || SW <= 0)
        return 0;
    const int64_t OH = outsize(H, KH, SH, PH), OW = outsize(W, KW, SW, PW);
    if (OH <= 0 || OW <= 0)
        return 0;
    if (odl::conv_implicit_forward_ok(kAlignedProbe, N, C, H, W, OC, KH, KW, OH, OW))
        return 0;  // the im2col matrix is never materialised
    return align256((size_t)(N * OH * OW * C * KH * KW) * sizeof(float));
}

int odl_hip_conv2d(const float *x, const float *w, const float *b, int64_t N, int64_t C, int64_t H, int64_t W,
                   int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, float *y, void *workspace,
                   size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ConvGeom g;
    int rc = make_geom(g, "conv2d", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    ODL_REQUIRE(OC > 0, "conv2d: OC must be positive");
    const int64_t M = N * g.OH * g.OW, K = C * KH * KW;
    if (M == 0)
        return ODL_OK;
    hipStream_t st = odl::as_stream(stream);
    if (odl::conv_implicit_forward_ok(w, N, C, H, W, OC, KH, KW, g.OH, g.OW))
        return odl::conv_implicit_forward(x, w, b, y, N, C, H, W, OC, KH, KW, SH, SW, PH, PW, g.OH, g.OW, st);
    // explicit path: col = im2col(x), then y^T[OC, M] = W2d[OC,K] . col[M,K]^T stored as y[n][oc][p] (+ bias per channel)
    const size_t need = align256((size_t)(M * K) * sizeof(float));
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= need,
                "conv2d: this shape/alignment needs a workspace of %zu bytes, got %zu", need, workspace_bytes);
    float *col = static_cast<float *>(workspace);
    rc = im2col_launch(x, col, g, 1, st);
    if (rc != ODL_OK)
        return rc;
    return odl::sgemm_launch(0, 1, OC, M, K, w, K, col, K, y, 0, b, /*EPI_NCHW_ROWB*/ 2, g.OH * g.OW, 1, nullptr, 0,
                             st);
}

namespace
{
// workspace regions of conv2d_backward, in order: [col][split-K partials][permuted weights][bias partials]
struct BwdPlan
{
    bool wgrad_implicit, dgrad_implicit;
    size_t col_bytes, splitk_bytes, wp_bytes, red_bytes;
    size_t total() const { return col_bytes + splitk_bytes + wp_bytes + red_bytes; }
};

BwdPlan plan_backward(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH,
                      int SW, int64_t OH, int64_t OW)
{
    BwdPlan p{};
    const int64_t M = N * OH * OW, K = C * KH * KW;
    p.wgrad_implicit = odl::conv_implicit_wgrad_ok(gy, N, C, H, W, OC, KH, KW, OH, OW);
    p.dgrad_implicit = odl::conv_implicit_dgrad_ok(gy, N, C, H, W, OC, KH, KW, SH, SW);
    p.col_bytes = (p.wgrad_implicit && p.dgrad_implicit) ? 0 : align256((size_t)(M * K) * sizeof(float));
    p.splitk_bytes = align256(p.wgrad_implicit ? odl::conv_implicit_wgrad_workspace(N, C, OC, KH, KW, OH, OW)
                                               : odl::sgemm_workspace(OC, K, M, 0));
    p.wp_bytes = p.dgrad_implicit ? align256(odl::conv_implicit_dgrad_workspace(C, OC, KH, KW)) : 0;
    p.red_bytes = align256(odl::sum_nchw_channels_workspace(N, OC, OH * OW));
    return p;
}
}  // namespace

size_t odl_hip_conv2d_backward_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                                               int SH, int SW, int PH, int PW)
{
    if (KH <= 0 || KW <= 0 || SH <= 0 || SW <= 0)
        return 0;
    const int64_t OH = outsize(H, KH, SH, PH), OW = outsize(W, KW, SW, PW);
    if (OH <= 0 || OW <= 0)
        return 0;
    return plan_backward(kAlignedProbe, N, C, H, W, OC, KH, KW, SH, SW, OH, OW).total();
}

int odl_hip_conv2d_backward(const float *gy, const float *x, const float *w, int64_t N, int64_t C, int64_t H, int64_t W,
                            int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, float *gx, float *gw, float *gb,
                            void *workspace, size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ConvGeom g;
    int rc = make_geom(g, "conv2d_backward", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    ODL_REQUIRE(OC > 0, "conv2d_backward: OC must be positive");
    const int64_t M = N * g.OH * g.OW, K = C * KH * KW;
    if (M == 0)
        return ODL_OK;
    const BwdPlan p = plan_backward(gy, N, C, H, W, OC, KH, KW, SH, SW, g.OH, g.OW);
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= p.total(),
                "conv2d_backward: this shape/alignment needs a workspace of %zu bytes, got %zu", p.total(),
                workspace_bytes);
    hipStream_t st = odl::as_stream(stream);
    char *ws = static_cast<char *>(workspace);
    float *col = reinterpret_cast<float *>(ws);
    void *splitk_ws = ws + p.col_bytes;
    void *wp_ws = ws + p.col_bytes + p.splitk_bytes;
    void *red_ws = ws + p.col_bytes + p.splitk_bytes + p.wp_bytes;

    // gy2d: gy's NCHW buffer read as a row-major [M, OC] matrix exactly as it lies (conv2d.cpp:548)
    if (gw)
    {
        if (p.wgrad_implicit)
            rc = odl::conv_implicit_wgrad(gy, x, gw, N, C, H, W, OC, KH, KW, SH, SW, PH, PW, g.OH, g.OW, splitk_ws,
                                          p.splitk_bytes, st);
        else
        {
            rc = im2col_launch(x, col, g, 1, st);
            if (rc == ODL_OK)  // gW[OC,K] = gy2d[M,OC]^T . col[M,K]
                rc = odl::sgemm_launch(1, 0, OC, K, M, gy, OC, col, K, gw, K, nullptr, 0, 0, 0, splitk_ws,
                                       p.splitk_bytes, st);
        }
        if (rc != ODL_OK)
            return rc;
    }
    if (gb)
    {
        rc = odl::sum_nchw_channels_launch(gy, N, OC, g.OH * g.OW, gb, red_ws, p.red_bytes, st);
        if (rc != ODL_OK)
            return rc;
    }
    if (gx)
    {
        if (p.dgrad_implicit)
            rc = odl::conv_implicit_dgrad(gy, w, gx, N, C, H, W, OC, KH, KW, PH, PW, g.OH, g.OW, wp_ws, p.wp_bytes, st);
        else
        {
            // gx_col[M,K] = gy2d[M,OC] . W2d[OC,K], then the gather back to the image
            rc = odl::sgemm_launch(0, 0, M, K, OC, gy, OC, w, K, col, K, nullptr, 0, 0, 1, nullptr, 0, st);
            if (rc == ODL_OK)
                rc = col2im_launch(col, gx, g, 1, st);
        }
        if (rc != ODL_OK)
            return rc;
    }
    return ODL_OK;
}

}  // extern "C"
