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
#include "conv_side.h"
#include "gemm_dma.h"
#include "odl_common.h"

#include <algorithm>
#include <atomic>

namespace odl
{
int sgemm_launch(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                 const float *B, int64_t ldb, float *C, int64_t ldc, const float *bias, int epi, int64_t P,
                 int split_k, void *workspace, size_t workspace_bytes, hipStream_t st, int act = 0);
size_t sgemm_workspace(int64_t M, int64_t N, int64_t K, int split_k);
bool conv_implicit_forward_ok(const float *w, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                              int64_t OH, int64_t OW);
bool conv_implicit_wgrad_ok(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                            int64_t OH, int64_t OW);
bool conv_implicit_dgrad_ok(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                            int SH, int SW);
size_t conv_implicit_wgrad_workspace(int64_t N, int64_t C, int64_t OC, int KH, int KW, int64_t OH, int64_t OW);
size_t conv_implicit_dgrad_workspace(int64_t C, int64_t OC, int KH, int KW, int64_t pixels);
int conv_implicit_forward(const float *x, const float *w, const float *b, float *y, int64_t N, int64_t C, int64_t H,
                          int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, int64_t OH, int64_t OW,
                          int act, void *workspace, size_t workspace_bytes, hipStream_t st, const float *packed = nullptr);
size_t conv_implicit_forward_packed_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW);
int conv_implicit_forward_pack(const float *w, int64_t C, int64_t OC, int KH, int KW, float *packed, hipStream_t st);
int conv_implicit_forward_splits(int64_t OC, int64_t M, int64_t K);
size_t conv_implicit_forward_workspace(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                                       int64_t OH, int64_t OW);
int conv_implicit_wgrad(const float *gy, const float *x, float *gw, int64_t N, int64_t C, int64_t H, int64_t W,
                        int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, int64_t OH, int64_t OW,
                        void *workspace, size_t workspace_bytes, hipStream_t st);
int conv_implicit_dgrad(const float *gy, const float *w, float *gx, int64_t N, int64_t C, int64_t H, int64_t W,
                        int64_t OC, int KH, int KW, int PH, int PW, int64_t OH, int64_t OW, void *workspace,
                        size_t workspace_bytes, hipStream_t st);
// the first layer of an image network (1 or 3 input channels): direct kernels, one thread per pixel (conv_small.hip)
bool conv_small_forward_ok(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int64_t OH, int64_t OW);
int conv_small_forward(const float *x, const float *w, const float *b, float *y, int64_t N, int64_t C, int64_t H, int64_t W,
                       int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, int64_t OH, int64_t OW, int act,
                       hipStream_t st);
// 3x3, stride 1, padding 1 with the input channels a multiple of 16: the input patch stays in LDS (conv_patch.hip)
bool conv_patch_forward_ok(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH,
                           int SW, int PH, int PW);
size_t conv_patch_forward_workspace(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC);
int conv_patch_forward(const float *x, const float *w, const float *b, float *y, int64_t N, int64_t C, int64_t H,
                       int64_t W, int64_t OC, int act, void *workspace, size_t workspace_bytes, hipStream_t st);
bool conv_patch_dgrad_ok(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH,
                         int SW, int PH, int PW);
size_t conv_patch_dgrad_workspace(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC);

int conv_patch_dgrad(const float *gy, const float *w, float *gx, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
                     void *workspace, size_t workspace_bytes, hipStream_t st, bool packed);
SidePack conv_patch_dgrad_pack(const float *w, int64_t C, int64_t OC, void *workspace);
int conv_small_forward_pool(const float *x, const float *w, const float *b, float *y, uint64_t *idx, uint8_t *idx8, int64_t N,
                            int64_t C, int64_t H, int64_t W, int64_t OC, int act, hipStream_t st);
bool conv_small_wgrad_ok(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int64_t OH,
                         int64_t OW);
size_t conv_small_wgrad_workspace(int64_t N, int64_t C, int64_t OC, int KH, int KW, int64_t OH, int64_t OW);
int conv_small_wgrad(const float *gy, const float *x, float *gw, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
                     int KH, int KW, int SH, int SW, int PH, int PW, int64_t OH, int64_t OW, void *workspace,
                     size_t workspace_bytes, hipStream_t st);
bool conv_small_dgrad_ok(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int64_t OH,
                         int64_t OW);
size_t conv_small_dgrad_workspace(int64_t C, int64_t OC, int KH, int KW);
int conv_small_dgrad(const float *gy, const float *w, float *gx, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
                     int KH, int KW, int SH, int SW, int PH, int PW, int64_t OH, int64_t OW, void *workspace,
                     size_t workspace_bytes, hipStream_t st);
// conv_stem.hip: the whole backward pass of a one-channel 3x3 / stride 1 / padding 1 layer in one pass over gy
bool conv_stem_backward_ok(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW,
                           int PH, int PW);
size_t conv_stem_backward_workspace(int64_t N, int64_t OC);
int conv_stem_backward(const float *gy, const float *x, const float *w, float *gx, float *gw, float *gb, int64_t N, int64_t H,
                       int64_t W, int64_t OC, void *workspace, size_t workspace_bytes, hipStream_t st);
// conv_image.hip: 3x3 / stride 1 / padding 1 over small images with few channels, an image at a time resident in LDS;
// the weight and the bias gradient in one pass
bool conv_image_wgrad_ok(const float *gy, const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                         int SH, int SW, int PH, int PW);
size_t conv_image_wgrad_workspace(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC);
int conv_image_wgrad(const float *gy, const float *x, float *gw, float *gb, int64_t N, int64_t C, int64_t H, int64_t W,
                     int64_t OC, void *workspace, size_t workspace_bytes, hipStream_t st, const SidePack *pack, unsigned n_pack);
// conv_wgrad.hip: 3x3 / padding 1 / stride 1 or 2, walking the output rows with the input rows staged in LDS
bool conv_wgrad_rows_ok(const float *gy, const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH,
                        int KW, int SH, int SW, int PH, int PW, int64_t OH, int64_t OW);
size_t conv_wgrad_rows_workspace(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW,
                                 int PH, int PW, int64_t OH, int64_t OW);
int conv_wgrad_rows(const float *gy, const float *x, float *gw, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
                    int S, int64_t OH, int64_t OW, void *workspace, size_t workspace_bytes, hipStream_t st, SideFold *fold);
int sum_nchw_channels_launch(const float *gy, int64_t N, int64_t OC, int64_t P, float *gb, void *workspace,
                             size_t workspace_bytes, hipStream_t st);
size_t sum_nchw_channels_workspace(int64_t N, int64_t OC, int64_t P);
// conv_direct.hip: small problems, operands straight from global memory, K shared between the waves of a workgroup;
// input, output and residual may be channel slices of wider tensors
bool conv_direct_ok(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW,
                    int64_t OH, int64_t OW);
size_t conv_direct_packed_bytes(int64_t C, int64_t OC, int KH, int KW, int P, int64_t W);
int conv_direct_pack(const float *w, int64_t C, int64_t OC, int KH, int KW, int P, int64_t W, float *packed, hipStream_t st);
int conv_direct(const float *x, int64_t x_bs, const float *packed, const float *b, const float *res, int64_t res_bs, float *y,
                int64_t y_bs, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int S, int P, int64_t OH,
                int64_t OW, int act, hipStream_t st, float *y2 = nullptr, int64_t y2_bs = 0, int64_t split = 0);
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

__device__ inline unsigned xcd_contiguous_block32(unsigned bid, unsigned nb, unsigned xcds)
{
    const unsigned loc = bid / xcds, xcd = bid - loc * xcds;
    const unsigned full = nb / xcds, rem = nb - full * xcds;
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

// Matrix layout, the fast path: tile = 64 consecutive col rows (pixels) x CT channels with all their taps.
// Read phase: lanes run along the pixels, each wave takes every fourth channel and issues that channel's taps
// together (a 3x3 window is unrolled and its in-image test is one bit of a per-lane mask computed once);
// the tile is turned through LDS (odd row stride: no bank conflicts) and leaves as 16-byte stores along the
// col rows. All index arithmetic is 32-bit, and the per-store division is a multiply by a precomputed reciprocal:
// on a 64-wide wave integer address arithmetic, not memory, is what this kernel would otherwise wait for.
struct Im2colTile
{
    int CT, ctiles, LS;      // channels per tile, channel tiles, LDS row stride (floats, odd)
    unsigned mtiles;         // pixel tiles
    unsigned q4_magic;       // ceil(2^32 / q4) for q4 = CT*KH*KW/4
    unsigned xcds;           // L2 domains the hardware deals workgroups over
};

template <int CK>
__global__ __launch_bounds__(256) void im2col_tile_kernel(const float *__restrict__ img, float *__restrict__ col,
                                                           ConvGeom g, Im2colTile t)
{
    extern __shared__ float sh_i2c[];
    float *sh = sh_i2c;
    const int KH = CK > 0 ? CK : g.KH, KW = CK > 0 ? CK : g.KW;
    const int KHW = KH * KW;
    const unsigned vb = xcd_contiguous_block32(blockIdx.x, t.mtiles * (unsigned)t.ctiles, t.xcds);
    const unsigned mt = vb / (unsigned)t.ctiles;
    const int ct = (int)(vb - mt * (unsigned)t.ctiles);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int H = (int)g.H, W = (int)g.W, C = (int)g.C, OW = (int)g.OW;
    const unsigned P = (unsigned)(g.OH * g.OW);
    const unsigned M = (unsigned)(g.N * g.OH * g.OW);
    const unsigned m = mt * 64u + (unsigned)lane;
    const bool live = m < M;
    const unsigned mm = live ? m : 0u;
    const unsigned n = mm / P, r = mm - n * P;
    const int oh = (int)(r / (unsigned)OW), ow = (int)(r - (unsigned)oh * (unsigned)OW);
    const int h0 = oh * g.SH - g.PH, w0 = ow * g.SW - g.PW;
    const int c0 = ct * t.CT;
    const int ccn = (C - c0 < t.CT) ? C - c0 : t.CT;
    const int HW = H * W;
    // first tap of this lane's window in channel c0; dereferenced only where the tap lies inside the image
    const float *p = img + ((int64_t)n * C + c0) * HW + (int64_t)h0 * W + w0;
    float *srow = sh + lane * t.LS;
    if constexpr (CK > 0)
    {
        unsigned mask = 0;
#pragma unroll
        for (int kh = 0; kh < CK; ++kh)
#pragma unroll
            for (int kw = 0; kw < CK; ++kw)
                if (live && (unsigned)(h0 + kh) < (unsigned)H && (unsigned)(w0 + kw) < (unsigned)W)
                    mask |= 1u << (kh * CK + kw);
        for (int cl = wave; cl < ccn; cl += 4)
        {
            const float *pc = p + cl * HW;
            float v[CK * CK];
#pragma unroll
            for (int kh = 0; kh < CK; ++kh)
#pragma unroll
                for (int kw = 0; kw < CK; ++kw)
                    v[kh * CK + kw] = ((mask >> (kh * CK + kw)) & 1u) ? pc[kh * W + kw] : 0.f;
#pragma unroll
            for (int q = 0; q < CK * CK; ++q)
                srow[cl * (CK * CK) + q] = v[q];
        }
    }
    else
    {
        for (int cl = wave; cl < ccn; cl += 4)
        {
            const float *pc = p + cl * HW;
            for (int kh = 0; kh < KH; ++kh)
            {
                const bool hok = live && (unsigned)(h0 + kh) < (unsigned)H;
                for (int kw = 0; kw < KW; ++kw)
                {
                    const bool ok = hok && (unsigned)(w0 + kw) < (unsigned)W;
                    srow[cl * KHW + kh * KW + kw] = ok ? pc[kh * W + kw] : 0.f;
                }
            }
        }
    }
    __syncthreads();
    const int K = C * KHW;
    const int run = ccn * KHW;
    const unsigned row0 = mt * 64u;
    const int rows = (M - row0 < 64u) ? (int)(M - row0) : 64;
    float *dst0 = col + (int64_t)row0 * K + c0 * KHW;
    if ((run & 3) == 0 && (K & 3) == 0 && ((c0 * KHW) & 3) == 0 && (reinterpret_cast<uintptr_t>(col) & 15) == 0)
    {
        const int q4 = run >> 2;
        // row = e / q4 through the reciprocal: exact while e < 2^32 / q4, and e < 64 * q4 here. The reciprocal is that
        // of a full tile's q4; a ragged last channel tile (smaller run) divides directly.
        const bool full = ccn == t.CT && t.q4_magic != 0;
        for (int e = threadIdx.x; e < rows * q4; e += 256)
        {
            const int row = full ? (int)__umulhi((unsigned)e, t.q4_magic) : e / q4;
            const int q = e - row * q4;
            const float *sr = sh + row * t.LS + 4 * q;
            const f32x4 o = {sr[0], sr[1], sr[2], sr[3]};
            *reinterpret_cast<f32x4 *>(dst0 + (int64_t)row * K + 4 * q) = o;
        }
    }
    else
    {
        for (int e = threadIdx.x; e < rows * run; e += 256)
        {
            const int row = e / run, j = e - row * run;
            dst0[(int64_t)row * K + j] = sh[row * t.LS + j];
        }
    }
}

// Tile shape for im2col_tile_kernel, or false when the shape needs the general kernel (64-bit indices, huge windows).
bool plan_im2col_tile(const ConvGeom &g, Im2colTile &t)
{
    const int64_t KHW = (int64_t)g.KH * g.KW, M = g.N * g.OH * g.OW;
    if (KHW > 160 || M >= (1ll << 31) - 64 || g.C * g.H * g.W >= (1ll << 31) || g.C * KHW >= (1ll << 31))
        return false;
    int CT = (int)(144 / KHW);
    CT = CT < 1 ? 1 : (CT > 128 ? 128 : CT);
    if (CT > g.C)
        CT = (int)g.C;
    if (CT >= 4)
        CT &= ~3;  // a multiple of four channels keeps every tile's columns 16-byte aligned
    // a small problem gets narrower tiles: more workgroups in flight matter more than longer runs per store
    while (CT >= 8 && odl::ceil_div(M, 64) * odl::ceil_div(g.C, CT) < 1536)
        CT = (CT / 2) & ~3;
    t.CT = CT;
    t.ctiles = (int)odl::ceil_div(g.C, CT);
    t.LS = (int)(CT * KHW) | 1;
    t.mtiles = (unsigned)odl::ceil_div(M, 64);
    if ((int64_t)t.mtiles * t.ctiles >= (1ll << 31))
        return false;
    const unsigned q4 = (unsigned)(CT * KHW / 4);
    t.q4_magic = q4 > 1 ? (unsigned)(((1ull << 32) + q4 - 1) / q4) : 0u;  // 0: the kernel divides directly
    t.xcds = (unsigned)odl::chip().xcds;
    return true;
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
// CS > 0 fixes both strides at compile time (the tap arithmetic divides by them).
template <int CKH, int CKW, int CS>
__global__ __launch_bounds__(256) void col2im_matrix_kernel(const float *__restrict__ col, float *__restrict__ img,
                                                             ConvGeom g, int wtiles, int ctiles)
{
    __shared__ float sh[64][17];
    const int KH = CKH > 0 ? CKH : g.KH, KW = CKW > 0 ? CKW : g.KW;
    const int SH = CS > 0 ? CS : g.SH, SW = CS > 0 ? CS : g.SW;
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
        const float *nbase = cbase + n * OH * OW * K;  // this image's rows; offsets below fit 32 bits (checked by the host)
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
                        const int oh = hp / SH;
                        const bool hok = hp >= 0 && hp % SH == 0 && oh < OH;
                        const int ro = oh * OW;
#pragma unroll
                        for (int kw = 0; kw < CKW; ++kw)
                        {
                            const int wp = w + g.PW - kw;
                            const int ow = wp / SW;
                            const bool ok = hok && wp >= 0 && wp % SW == 0 && ow < OW;
                            v[kh * CKW + kw] = ok ? nbase[(ro + ow) * K + kh * CKW + kw] : 0.f;
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
                        if (hp < 0 || hp % SH != 0)
                            continue;
                        const int oh = hp / SH;
                        if (oh >= OH)
                            continue;
                        for (int kw = 0; kw < KW; ++kw)
                        {
                            const int wp = w + g.PW - kw;
                            if (wp < 0 || wp % SW != 0)
                                continue;
                            const int ow = wp / SW;
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

// Matrix layout, the fast path: a workgroup owns CT channels x TH x TW pixels of one image. It first copies the
// rectangle of col rows those pixels draw from — ohr x owr output positions, CT*KH*KW consecutive floats of each —
// into LDS with coalesced 16-byte loads, then sums each pixel's taps out of LDS in ascending (kh, kw) and writes the
// image along w. Lanes run along w in both the LDS reads (odd row stride: distinct banks) and the image writes.
// Index arithmetic is 32-bit with reciprocal multiplies, and the compute loop is wave-uniform over (channel, row).
struct Col2imTile
{
    int TH, TW, CT;          // pixels and channels per workgroup
    int htiles, wtiles, ctiles;
    int ohr, owr;            // staged rectangle of output positions
    int LS;                  // LDS row stride in floats (odd)
    unsigned q4_magic;       // ceil(2^32 / (CT*KH*KW/4)), 0 = divide directly
    unsigned owr_magic;      // ceil(2^32 / owr)
    unsigned xcds;           // L2 domains the hardware deals workgroups over
};

__device__ inline int ceil_div_signed(int a, int d)  // d > 0
{
    return a >= 0 ? (a + d - 1) / d : -((-a) / d);
}

template <int CK, int CS>
__global__ __launch_bounds__(256) void col2im_tile_kernel(const float *__restrict__ col, float *__restrict__ img,
                                                           ConvGeom g, Col2imTile t)
{
    extern __shared__ float sh_c2i[];
    float *sh = sh_c2i;
    const int KH = CK > 0 ? CK : g.KH, KW = CK > 0 ? CK : g.KW;
    const int SH = CS > 0 ? CS : g.SH, SW = CS > 0 ? CS : g.SW;
    const int KHW = KH * KW;
    const int H = (int)g.H, W = (int)g.W, OH = (int)g.OH, OW = (int)g.OW, C = (int)g.C;
    unsigned vb = xcd_contiguous_block32(blockIdx.x, (unsigned)g.N * t.htiles * t.wtiles * t.ctiles, t.xcds);
    const int ct = (int)(vb % (unsigned)t.ctiles);
    vb /= (unsigned)t.ctiles;
    const int wt = (int)(vb % (unsigned)t.wtiles);
    vb /= (unsigned)t.wtiles;
    const int ht = (int)(vb % (unsigned)t.htiles);
    const int n = (int)(vb / (unsigned)t.htiles);
    const int h0 = ht * t.TH, w0 = wt * t.TW, c0 = ct * t.CT;
    const int th = (H - h0 < t.TH) ? H - h0 : t.TH, tw = (W - w0 < t.TW) ? W - w0 : t.TW;
    const int ccn = (C - c0 < t.CT) ? C - c0 : t.CT;
    // first output position (possibly negative) whose window can reach this tile
    const int oh_lo = ceil_div_signed(h0 + g.PH - (KH - 1), SH), ow_lo = ceil_div_signed(w0 + g.PW - (KW - 1), SW);
    const int K = C * KHW;
    const int run = ccn * KHW;
    const float *src0 = col + (int64_t)n * OH * OW * K + c0 * KHW;  // offsets from here fit 32 bits (checked by the host)
    const int R = t.ohr * t.owr;
    if ((run & 3) == 0 && (K & 3) == 0 && ((c0 * KHW) & 3) == 0 && (reinterpret_cast<uintptr_t>(col) & 15) == 0)
    {
        const int q4 = run >> 2;
        const bool recip = ccn == t.CT && t.q4_magic != 0;
        constexpr int U = 8;  // independent 16-byte loads in flight per thread
        for (int e0 = threadIdx.x; e0 < R * q4; e0 += 256 * U)
        {
            f32x4 v[U];
            int doff[U];
#pragma unroll
            for (int u = 0; u < U; ++u)
            {
                const int e = e0 + 256 * u;
                const int r = recip ? (int)__umulhi((unsigned)e, t.q4_magic) : e / q4;
                const int q = e - r * q4;
                const int ro = t.owr_magic ? (int)__umulhi((unsigned)r, t.owr_magic) : r;  // owr == 1: every row is its own
                const int oh = oh_lo + ro, ow = ow_lo + (r - ro * t.owr);
                const bool ok = e < R * q4 && (unsigned)oh < (unsigned)OH && (unsigned)ow < (unsigned)OW;
                doff[u] = ok ? r * t.LS + 4 * q : -1;
                v[u] = f32x4{0.f, 0.f, 0.f, 0.f};
                if (ok)
                    v[u] = *reinterpret_cast<const f32x4 *>(src0 + (oh * OW + ow) * K + 4 * q);
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (doff[u] >= 0)
                {
                    float *d = sh + doff[u];
                    d[0] = v[u][0], d[1] = v[u][1], d[2] = v[u][2], d[3] = v[u][3];
                }
        }
    }
    else
    {
        for (int e = threadIdx.x; e < R * run; e += 256)
        {
            const int r = e / run, j = e - r * run;
            const int ro = t.owr_magic ? (int)__umulhi((unsigned)r, t.owr_magic) : r;  // owr == 1: every row is its own
            const int oh = oh_lo + ro, ow = ow_lo + (r - ro * t.owr);
            if ((unsigned)oh < (unsigned)OH && (unsigned)ow < (unsigned)OW)
                sh[r * t.LS + j] = src0[(oh * OW + ow) * K + j];
        }
    }
    __syncthreads();
    // lanes: RW image rows of TW pixels per wave; waves walk (channel, row group) pairs
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int RW = 64 / t.TW;  // >= 1 (TW <= 64)
    const int lr = lane / t.TW, lw = lane - lr * t.TW;
    const int hgroups = (th + RW - 1) / RW;
    const int w = w0 + lw;
    const bool lane_ok = lr < RW && lw < tw;
    float *dst0 = img + ((int64_t)n * C + c0) * H * W;
    for (int idx = wave; idx < ccn * hgroups; idx += 4)
    {
        const int cl = idx / hgroups, hg = idx - cl * hgroups;  // wave-uniform
        const int hh = hg * RW + lr;
        if (!lane_ok || hh >= th)
            continue;
        const int h = h0 + hh;
        const float *cs = sh + cl * KHW;
        float acc = 0.f;
        if constexpr (CK > 0)
        {
            // every tap is read (or zeroed) first, then added in ascending (kh, kw): a skipped tap contributes nothing
            // in the reference, and adding +0.0f instead leaves each partial sum unchanged (the accumulator starts at
            // +0.0f and never becomes -0.0f)
            float v[CK * CK];
#pragma unroll
            for (int kh = 0; kh < CK; ++kh)
            {
                const int hp = h + g.PH - kh;
                const int oh = hp / SH;
                const bool hok = hp >= 0 && hp % SH == 0 && oh < OH;
                const int rb = (oh - oh_lo) * t.owr - ow_lo;
#pragma unroll
                for (int kw = 0; kw < CK; ++kw)
                {
                    const int wp = w + g.PW - kw;
                    const int ow = wp / SW;
                    const bool ok = hok && wp >= 0 && wp % SW == 0 && ow < OW;
                    v[kh * CK + kw] = ok ? cs[(rb + ow) * t.LS + kh * CK + kw] : 0.f;
                }
            }
#pragma unroll
            for (int q = 0; q < CK * CK; ++q)
                acc += v[q];
        }
        else
        {
            for (int kh = 0; kh < KH; ++kh)
            {
                const int hp = h + g.PH - kh;
                if (hp < 0 || hp % SH != 0)
                    continue;
                const int oh = hp / SH;
                if (oh >= OH)
                    continue;
                for (int kw = 0; kw < KW; ++kw)
                {
                    const int wp = w + g.PW - kw;
                    if (wp < 0 || wp % SW != 0)
                        continue;
                    const int ow = wp / SW;
                    if (ow >= OW)
                        continue;
                    acc += cs[((oh - oh_lo) * t.owr + (ow - ow_lo)) * t.LS + kh * KW + kw];
                }
            }
        }
        dst0[(cl * H + h) * W + w] = acc;
    }
}

// Matrix layout, 3x3 / padding 1 / stride 1 or 2, the streaming form. The tile kernel above re-reads the col rows of a
// tile's halo and reads 144-byte runs that straddle 128-byte lines: about 2.3 times the matrix passes from L2 to LDS.
// Here a workgroup owns one image, eight channels (288 bytes of every col row: 18 whole 16-byte pieces) and a band
// of rows of output positions, and walks down the band: LDS keeps four position rows ([OW positions][72 floats] each,
// as the loads deliver them); while the image rows under position row r are summed (row r itself from position rows
// r-1, r, r+1 at stride 1; rows 2r and 2r+1 from position rows r and r+1 at stride 2), the rows r+2 and r+3 are on their
// way in registers. Every col row of the band is read once, plus one halo row above and below the band. Lanes run along
// (pixel, channel) with the channel fastest: the LDS addresses ow*72 + c*9 + tap of a wave fall into 32 different banks.
// Taps are added in ascending (kh, kw), absent ones left out — the sums of the other col2im kernels, bit for bit.
constexpr int kRowsCT = 8, kRowsRun = kRowsCT * 9, kRowsNT = 512, kRowsQ = 2;  // quads of a position row per thread: OW * 18 <= 2 * 512

// The lanes of the summing phase: a wave takes eight pixels of one image row (lane = pixel * 8 + channel), so the row and
// with it the position rows of its taps are the same for the whole wave (scalar work), and what depends on the pixel and
// the channel (the offsets of the three kw inside a position row, which of them exist) is worked out once per thread.
// Images up to 64 pixels wide put 8 / ceil(W / 8) rows side by side on the eight waves; wider ones go through a row in
// steps of 64 pixels.
struct RowsLanes
{
    int wave, c, wl, wpr, rpp, rip, wg0;
    __device__ RowsLanes(int t, int W)
    {
        wave = __builtin_amdgcn_readfirstlane(t >> 6);
        c = t & (kRowsCT - 1);
        wl = (t & 63) >> 3;
        wpr = (W + 7) / 8;
        rpp = wpr <= 8 ? 8 / wpr : 1;
        rip = wpr <= 8 ? wave / wpr : 0;
        wg0 = wpr <= 8 ? wave - rip * wpr : wave;
    }
};

// one pixel's sum: taps in ascending (kh, kw); a tap that does not exist would add +0.0f to a sum that is never -0.0f,
// so leaving it out gives the same float. `row_of(oh)` is the offset of position row `oh` in LDS.
template <int S, typename RowOf>
__device__ __forceinline__ float col2im_pixel3x3(const float *sh, RowOf row_of, int h, int OH, const int (&off)[3],
                                                 const bool (&wok)[3])
{
    float acc = 0.f;
#pragma unroll
    for (int kh = 0; kh < 3; ++kh)
    {
        const int hp = h + 1 - kh, oh = S == 1 ? hp : hp >> 1;
        if (hp >= 0 && (S == 1 || (hp & 1) == 0) && oh < OH)
        {
            const float *row = sh + row_of(oh) + kh * 3;
#pragma unroll
            for (int kw = 0; kw < 3; ++kw)
            {
                const float x = row[off[kw]];
                acc += wok[kw] ? x : 0.f;
            }
        }
    }
    return acc;
}

// the three kw of pixel column `w`: offset inside a position row (0 where the tap does not exist) and whether it exists
template <int S>
__device__ __forceinline__ void col2im_taps_of_column(int w, int c, int W, int OW, int (&off)[3], bool (&wok)[3])
{
#pragma unroll
    for (int kw = 0; kw < 3; ++kw)
    {
        const int wp = w + 1 - kw, ow = S == 1 ? wp : wp >> 1;
        wok[kw] = w < W && wp >= 0 && (S == 1 || (wp & 1) == 0) && ow < OW;
        off[kw] = wok[kw] ? ow * kRowsRun + c * 9 + kw : 0;
    }
}

template <int S>
__global__ __launch_bounds__(kRowsNT, 2) void col2im_rows3x3_kernel(const float *__restrict__ col, float *__restrict__ img, int N,
                                                                     int C, int H, int W, int OH, int OW, int band,
                                                                     int nbands, unsigned xcds)
{
    extern __shared__ float sh_rows[];
    const int t = threadIdx.x;
    const int slot_floats = OW * kRowsRun, quads = OW * (kRowsRun / 4), K = C * 9;
    unsigned vb;
    {
        const unsigned nb = gridDim.x, bid = blockIdx.x;
        const unsigned loc = bid / xcds, xcd = bid - loc * xcds, full = nb / xcds, rem = nb - full * xcds;
        vb = xcd * full + (xcd < rem ? xcd : rem) + loc;
    }
    const int cchunks = C / kRowsCT;
    const int cc = (int)(vb % (unsigned)cchunks);
    vb /= (unsigned)cchunks;
    const int b = (int)(vb % (unsigned)nbands), n = (int)(vb / (unsigned)nbands);
    // the band in rows of output positions; the last band also takes the image rows below the last position row's
    const int r0 = b * band, r1 = (r0 + band < OH) ? r0 + band : OH, c0 = cc * kRowsCT;
    const int h_end = (b == nbands - 1) ? H : S * r1;
    const float *src = col + (int64_t)n * OH * OW * K + c0 * 9;

    f32x4 ra[kRowsQ], rb[kRowsQ];
    int roff[kRowsQ];  // this thread's quads of a position row: offset inside the row, -1 past its end
#pragma unroll
    for (int q = 0; q < kRowsQ; ++q)
    {
        const int e = t + q * kRowsNT;
        const int pos = e / (kRowsRun / 4), qq = e - pos * (kRowsRun / 4);
        roff[q] = e < quads ? pos * K + qq * 4 : -1;
        ra[q] = rb[q] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    auto load_row = [&](int oh, f32x4 (&r)[kRowsQ]) {
        // position rows outside the image, or below the band's halo, are never read back: skip them
        const bool live = oh >= 0 && oh < OH && oh <= r1;
        const float *row = src + (int64_t)oh * OW * K;
#pragma unroll
        for (int q = 0; q < kRowsQ; ++q)
            if (live && roff[q] >= 0)
                r[q] = *reinterpret_cast<const f32x4 *>(row + roff[q]);
    };
    auto store_row = [&](int oh, const f32x4 (&r)[kRowsQ]) {
        float *dst = sh_rows + (oh & 3) * slot_floats;
#pragma unroll
        for (int q = 0; q < kRowsQ; ++q)
            if (roff[q] >= 0)
                *reinterpret_cast<f32x4 *>(dst + (t + q * kRowsNT) * 4) = r[q];
    };
    // the image rows under position row r
    const RowsLanes ln(t, W);
    auto sum_rows = [&](int r) {
        if (ln.rip >= ln.rpp)
            return;
#pragma unroll 1
        for (int wg = ln.wg0; wg < ln.wpr; wg += 8)
        {
            const int w = wg * 8 + ln.wl;
            int off[3];
            bool wok[3];
            col2im_taps_of_column<S>(w, ln.c, W, OW, off, wok);
#pragma unroll 1
            for (int h = S * r + ln.rip; h < S * r + S && h < h_end; h += ln.rpp)
            {
                const float acc = col2im_pixel3x3<S>(sh_rows, [&](int oh) { return (oh & 3) * slot_floats; }, h, OH, off, wok);
                if (w < W)
                    img[((int64_t)(n * C + c0 + ln.c) * H + h) * W + w] = acc;
            }
        }
    };

    // the three position rows the first iteration needs, then two more on their way
    load_row(r0 - 1, ra);
    load_row(r0, rb);
    if (r0 - 1 >= 0)
        store_row(r0 - 1, ra);
    load_row(r0 + 1, ra);
    store_row(r0, rb);
    load_row(r0 + 2, rb);
    store_row(r0 + 1, ra);
    load_row(r0 + 3, ra);
    __syncthreads();
    // invariant at the top of an iteration for position row r: LDS holds position rows r-1, r, r+1; the registers hold
    // r+2 (the set stored first) and r+3. Row r+2 goes into the slot row r-2 left, which nobody reads any more.
#pragma unroll 1
    for (int r = r0; r < r1; r += 2)
    {
        store_row(r + 2, rb);
        load_row(r + 4, rb);
        sum_rows(r);
        __syncthreads();
        if (r + 1 >= r1)
            break;
        store_row(r + 3, ra);
        load_row(r + 5, ra);
        sum_rows(r + 1);
        __syncthreads();
    }
}

// Matrix layout, 3x3 / stride 2 / padding 1, short rows of positions: the walk above keeps too few bytes in flight when a
// position row is only a few KB. Here a workgroup takes its whole band of position rows (and the one below: image row
// 2r+1 also reads position row r+1) into LDS at once, eight 16-byte loads deep per thread, and sums its image rows after
// one barrier. Same lanes, same LDS layout, same order of the taps as the walk.
constexpr int kBandLdsBytes = 64 * 1024;

__global__ __launch_bounds__(kRowsNT, 2) void col2im_band3x3s2_kernel(const float *__restrict__ col, float *__restrict__ img, int N,
                                                                       int C, int H, int W, int OH, int OW, int band,
                                                                       int nbands, unsigned xcds)
{
    extern __shared__ float sh_rows[];
    const int t = threadIdx.x;
    const int K = C * 9;
    unsigned vb;
    {
        const unsigned nb = gridDim.x, bid = blockIdx.x;
        const unsigned loc = bid / xcds, xcd = bid - loc * xcds, full = nb / xcds, rem = nb - full * xcds;
        vb = xcd * full + (xcd < rem ? xcd : rem) + loc;
    }
    const int cchunks = C / kRowsCT;
    const int cc = (int)(vb % (unsigned)cchunks);
    vb /= (unsigned)cchunks;
    const int b = (int)(vb % (unsigned)nbands), n = (int)(vb / (unsigned)nbands);
    const int r0 = b * band, r1 = (r0 + band < OH) ? r0 + band : OH, c0 = cc * kRowsCT;
    const int rows_in = (r1 < OH ? r1 + 1 : OH) - r0;  // with the row below the band where the image has one
    const int h0 = 2 * r0, h_end = (b == nbands - 1) ? H : 2 * r1;
    const float *src = col + ((int64_t)n * OH + r0) * OW * K + c0 * 9;
    const int quads = rows_in * OW * (kRowsRun / 4);
    constexpr int kDeep = 8;
#pragma unroll 1
    for (int e0 = t; e0 < quads; e0 += kDeep * kRowsNT)
    {
        f32x4 r[kDeep];
#pragma unroll
        for (int q = 0; q < kDeep; ++q)
        {
            const int e = e0 + q * kRowsNT;
            const int pos = e / (kRowsRun / 4), qq = e - pos * (kRowsRun / 4);
            if (e < quads)
                r[q] = *reinterpret_cast<const f32x4 *>(src + (int64_t)pos * K + qq * 4);
        }
#pragma unroll
        for (int q = 0; q < kDeep; ++q)
        {
            const int e = e0 + q * kRowsNT;
            if (e < quads)
                *reinterpret_cast<f32x4 *>(sh_rows + e * 4) = r[q];
        }
    }
    __syncthreads();
    const RowsLanes ln(t, W);
    if (ln.rip >= ln.rpp)
        return;
    const int row_floats = OW * kRowsRun;
#pragma unroll 1
    for (int wg = ln.wg0; wg < ln.wpr; wg += 8)
    {
        const int w = wg * 8 + ln.wl;
        int off[3];
        bool wok[3];
        col2im_taps_of_column<2>(w, ln.c, W, OW, off, wok);
#pragma unroll 1
        for (int h = h0 + ln.rip; h < h_end; h += ln.rpp)
        {
            const float acc = col2im_pixel3x3<2>(sh_rows, [&](int oh) { return (oh - r0) * row_floats; }, h, OH, off, wok);
            if (w < W)
                img[((int64_t)(n * C + c0 + ln.c) * H + h) * W + w] = acc;
        }
    }
}

bool col2im_rows3x3_ok(const ConvGeom &g, const float *col)
{
    return g.KH == 3 && g.KW == 3 && g.SH == g.SW && (g.SH == 1 || g.SH == 2) && g.PH == 1 && g.PW == 1 &&
           g.C % kRowsCT == 0 && g.OW <= 56 && g.OW >= 2 && g.OH >= 2 && g.W >= 4 && reinterpret_cast<uintptr_t>(col) % 16 == 0 &&
           g.N * g.C * g.H * g.W < (1ll << 31) && g.N * (g.C / kRowsCT) * g.OH < (1ll << 31) &&
           g.OH * g.OW * g.C * 9 < (1ll << 31);
}

// Tile shape for col2im_tile_kernel: the staged rectangle must fit in a third of a CU's LDS, there should be enough
// workgroups to fill the chip, and among those the tile that re-reads the fewest col rows wins. False when the
// shape needs the general kernel (64-bit offsets, windows too large to stage).
bool plan_col2im_tile(const ConvGeom &g, Col2imTile &best)
{
    const int64_t KHW64 = (int64_t)g.KH * g.KW;
    if (KHW64 > 160 || g.OH * g.OW * g.C * KHW64 >= (1ll << 31) || g.C * g.H * g.W >= (1ll << 31) || g.N >= (1 << 20))
        return false;
    const int KHW = (int)KHW64, H = (int)g.H, W = (int)g.W, C = (int)g.C;
    double best_cost = 0;
    bool found = false;
    const int tw_opts[3] = {W <= 64 ? W : 64, (W <= 64 && W % 2 == 0 && W / 2 >= 8) ? W / 2 : 0, W > 64 ? 32 : 0};
    for (int twi = 0; twi < 3; ++twi)
    {
        const int TW = tw_opts[twi];
        if (TW <= 0)
            continue;
        for (int CT = 16; CT >= 1; CT >>= 1)
        {
            if (CT > C && CT != 1)
                continue;
            const int LS = (CT * KHW) | 1;
            for (int TH = 1; TH <= H && TH <= 32; ++TH)
            {
                const int ohr = (TH + g.KH - 2) / g.SH + 1, owr = (TW + g.KW - 2) / g.SW + 1;
                const size_t lds = (size_t)ohr * owr * LS * sizeof(float);
                if (lds > 53 * 1024)
                    break;
                Col2imTile t{TH, TW, CT, (int)odl::ceil_div(H, TH), (int)odl::ceil_div(W, TW), (int)odl::ceil_div(C, CT),
                             ohr, owr, LS, 0u, 0u};
                const double blocks = (double)g.N * t.htiles * t.wtiles * t.ctiles;
                if (blocks >= (double)(1ll << 31))
                    continue;
                // col rows staged per image pixel relative to the rows a pixel needs; short runs, idle lanes and a
                // half-empty chip are charged on top
                double cost = (double)ohr * owr * g.SH * g.SW / ((double)TH * TW);
                if (CT * KHW * 4 < 256)
                    cost *= 1.0 + 0.5 * (256.0 - CT * KHW * 4) / 256.0;
                cost *= 64.0 / ((64 / TW) * TW);
                if (blocks < 4096)
                    cost *= 1.0 + 0.25 * (4096.0 / blocks - 1.0);
                if (!found || cost < best_cost)
                    best = t, best_cost = cost, found = true;
            }
        }
    }
    if (!found)
        return false;
    const unsigned q4 = (unsigned)(best.CT * KHW / 4);
    best.q4_magic = q4 > 1 ? (unsigned)(((1ull << 32) + q4 - 1) / q4) : 0u;
    best.owr_magic = best.owr > 1 ? (unsigned)(((1ull << 32) + best.owr - 1) / best.owr) : 0u;
    best.xcds = (unsigned)odl::chip().xcds;
    return true;
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
        Im2colTile t;
        if (plan_im2col_tile(g, t))
        {
            const size_t lds = (size_t)64 * t.LS * sizeof(float);
            const unsigned nbt = t.mtiles * (unsigned)t.ctiles;
            if (g.KH == 3 && g.KW == 3)
                hipLaunchKernelGGL((im2col_tile_kernel<3>), dim3(nbt), dim3(256), lds, st, img, col, g, t);
            else if (g.KH == 1 && g.KW == 1)
                hipLaunchKernelGGL((im2col_tile_kernel<1>), dim3(nbt), dim3(256), lds, st, img, col, g, t);
            else
                hipLaunchKernelGGL((im2col_tile_kernel<0>), dim3(nbt), dim3(256), lds, st, img, col, g, t);
            ODL_LAUNCH_CHECK();
            return ODL_OK;
        }
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
        const int cs = (g.SH == g.SW && (g.SH == 1 || g.SH == 2)) ? g.SH : 0;
        if (col2im_rows3x3_ok(g, col))
        {
            const int64_t per_band = g.N * (g.C / kRowsCT);
            const int64_t row_bytes = g.OW * kRowsRun * (int64_t)sizeof(float);
            const unsigned xcds = (unsigned)odl::chip().xcds;
            if (g.SH == 2 && 5 * row_bytes <= kBandLdsBytes)
            {
                // whole bands in LDS: four position rows or more a band (the row below it is read twice)
                const int64_t most = kBandLdsBytes / row_bytes - 1;
                int64_t nbands = odl::ceil_div((int64_t)2 * odl::device_cus(), per_band);
                if (nbands > g.OH / 4)
                    nbands = g.OH / 4;
                if (nbands < odl::ceil_div(g.OH, most))
                    nbands = odl::ceil_div(g.OH, most);
                const int band = (int)odl::ceil_div(g.OH, nbands);
                nbands = odl::ceil_div(g.OH, band);
                const size_t lds = (size_t)((band + 1 < g.OH ? band + 1 : g.OH) * row_bytes);
                hipLaunchKernelGGL(col2im_band3x3s2_kernel, dim3((unsigned)(per_band * nbands)), dim3(kRowsNT), lds, st, col, img,
                                   (int)g.N, (int)g.C, (int)g.H, (int)g.W, (int)g.OH, (int)g.OW, band, (int)nbands, xcds);
                ODL_LAUNCH_CHECK();
                return ODL_OK;
            }
            // bands of position rows: enough workgroups for four per compute unit where the image allows, seven rows or more
            int64_t nbands = odl::ceil_div((int64_t)4 * odl::device_cus(), per_band);
            if (nbands > g.OH / 7)
                nbands = g.OH / 7;
            if (nbands < 1)
                nbands = 1;
            const int band = (int)odl::ceil_div(g.OH, nbands);
            nbands = odl::ceil_div(g.OH, band);
            const size_t lds = (size_t)(4 * row_bytes);
            const dim3 grid((unsigned)(per_band * nbands)), block(kRowsNT);
            if (g.SH == 1)
                hipLaunchKernelGGL(col2im_rows3x3_kernel<1>, grid, block, lds, st, col, img, (int)g.N, (int)g.C, (int)g.H,
                                   (int)g.W, (int)g.OH, (int)g.OW, band, (int)nbands, xcds);
            else
                hipLaunchKernelGGL(col2im_rows3x3_kernel<2>, grid, block, lds, st, col, img, (int)g.N, (int)g.C, (int)g.H,
                                   (int)g.W, (int)g.OH, (int)g.OW, band, (int)nbands, xcds);
            ODL_LAUNCH_CHECK();
            return ODL_OK;
        }
        Col2imTile t;
        // the staged kernel pays off at stride 1, where neighbouring pixels share most of their col rows
        if (cs == 1 && plan_col2im_tile(g, t))
        {
            const unsigned nbt = (unsigned)(g.N * t.htiles * t.wtiles * t.ctiles);
            const size_t lds = (size_t)t.ohr * t.owr * t.LS * sizeof(float);
#define ODL_COL2IM_TILE(CKV, CSV) \
    hipLaunchKernelGGL((col2im_tile_kernel<CKV, CSV>), dim3(nbt), dim3(256), lds, st, col, img, g, t)
            if (g.KH == 3 && g.KW == 3 && cs == 1)
                ODL_COL2IM_TILE(3, 1);
            else if (g.KH == 3 && g.KW == 3 && cs == 2)
                ODL_COL2IM_TILE(3, 2);
            else if (cs == 1)
                ODL_COL2IM_TILE(0, 1);
            else
                ODL_COL2IM_TILE(0, 0);
#undef ODL_COL2IM_TILE
            ODL_LAUNCH_CHECK();
            return ODL_OK;
        }
        const int wtiles = (int)odl::ceil_div(g.W, 16), ctiles = (int)odl::ceil_div(g.C, 64);
        const int64_t nb = g.N * g.H * wtiles * ctiles;
        ODL_REQUIRE(nb < (1ll << 31) && g.N * g.OH * g.OW * g.C * g.KH * g.KW < (1ll << 40), "col2im: too large");
#define ODL_COL2IM_CASE(KHV, KWV, CSV)                                                                               \
    hipLaunchKernelGGL((col2im_matrix_kernel<KHV, KWV, CSV>), dim3((unsigned)nb), dim3(256), 0, st, col, img, g, wtiles, \
                       ctiles)
        const bool k3 = g.KH == 3 && g.KW == 3 && g.OH * g.OW * g.C * 9 < (1ll << 31);  // 32-bit row offsets
        if (k3 && cs == 1)
            ODL_COL2IM_CASE(3, 3, 1);
        else if (k3 && cs == 2)
            ODL_COL2IM_CASE(3, 3, 2);
        else if (k3)
            ODL_COL2IM_CASE(3, 3, 0);
        else
            ODL_COL2IM_CASE(0, 0, 0);
#undef ODL_COL2IM_CASE
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

// whether small problems go to the direct kernel (odl_hip_set_conv_direct; on unless switched off for a measurement)
static std::atomic<int> g_direct{1};

// 16-byte aligned stand-in used by the workspace queries, which see shapes only
static const float *const kAlignedProbe = reinterpret_cast<const float *>(uintptr_t(256));

// A strided convolution whose gathered forward would be cut into four or more K slices (few output tiles, a long K) goes
// through the col matrix instead: im2col, then one product on the straight-to-LDS kernel with the NCHW store, bias and
// activation in its epilogue — no partial outputs, no slice sum, no filter re-order
// (x[32,128,28,28] * W[256,128,3,3] / stride 2: 56.9 -> 54.5 us). Decided from the shape alone, so that the workspace
// query and the call agree.
static bool forward_by_col_matrix(int64_t N, int64_t C, int64_t OC, int KH, int KW, int SH, int SW, int64_t OH, int64_t OW)
{
    const int64_t M = N * OH * OW, K = C * KH * KW;
    // (from about a GFLOP on: below that both ways are a few launch latencies and the extra launch loses)
    return (SH > 1 || SW > 1) && K % 4 == 0 && K >= 128 && M * K * (int64_t)sizeof(float) <= (256ll << 20) &&
           2 * M * K * OC >= (1ll << 30) && odl::conv_implicit_forward_splits(OC, M, K) >= 4;
}

size_t odl_hip_conv2d_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH,
                                      int SW, int PH, int PW)
{
    if (KH <= 0 || KW <= 0 || SH <= 0 || SW <= 0)
        return 0;
    const int64_t OH = outsize(H, KH, SH, PH), OW = outsize(W, KW, SW, PW);
    if (OH <= 0 || OW <= 0)
        return 0;
    if (g_direct.load(std::memory_order_relaxed) && odl::conv_direct_ok(N, C, H, W, OC, KH, KW, SH, SW, PH, PW, OH, OW))
        return align256(odl::conv_direct_packed_bytes(C, OC, KH, KW, PH, W));  // the filter copy of a caller that keeps none
    if (odl::conv_small_forward_ok(N, C, H, W, OC, KH, KW, OH, OW))
        return 0;
    if (odl::conv_implicit_forward_ok(kAlignedProbe, N, C, H, W, OC, KH, KW, OH, OW))
    {
        // no im2col matrix: K-slice partials for small outputs, or the filter copy of the LDS-patch kernel
        size_t need = odl::conv_implicit_forward_workspace(N, C, H, W, OC, KH, KW, OH, OW);
        if (odl::conv_patch_forward_ok(kAlignedProbe, N, C, H, W, OC, KH, KW, SH, SW, PH, PW))
            need = std::max(need, odl::conv_patch_forward_workspace(N, C, H, W, OC));
        if (forward_by_col_matrix(N, C, OC, KH, KW, SH, SW, OH, OW))
            need = std::max(need, (size_t)(N * OH * OW * C * KH * KW) * sizeof(float));
        return align256(need);
    }
    return align256((size_t)(N * OH * OW * C * KH * KW) * sizeof(float));
}

int odl_hip_conv2d_act(const float *x, const float *w, const float *b, int64_t N, int64_t C, int64_t H, int64_t W,
                       int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, int activation, float *y,
                       void *workspace, size_t workspace_bytes, void *stream)
{
    return odl_hip_conv2d_act_packed(x, w, nullptr, b, N, C, H, W, OC, KH, KW, SH, SW, PH, PW, activation, y, workspace,
                                     workspace_bytes, stream);
}

size_t odl_hip_conv2d_packed_weights_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH,
                                           int SW, int PH, int PW)
{
    if (KH <= 0 || KW <= 0 || SH <= 0 || SW <= 0)
        return 0;
    const int64_t OH = outsize(H, KH, SH, PH), OW = outsize(W, KW, SW, PW);
    if (OH > 0 && OW > 0 && g_direct.load(std::memory_order_relaxed) &&
        odl::conv_direct_ok(N, C, H, W, OC, KH, KW, SH, SW, PH, PW, OH, OW))
        return odl::conv_direct_packed_bytes(C, OC, KH, KW, PH, W);
    if (OH <= 0 || OW <= 0 || odl::conv_small_forward_ok(N, C, H, W, OC, KH, KW, OH, OW) ||
        !odl::conv_implicit_forward_ok(kAlignedProbe, N, C, H, W, OC, KH, KW, OH, OW) ||
        forward_by_col_matrix(N, C, OC, KH, KW, SH, SW, OH, OW))
        return 0;
    return odl::conv_implicit_forward_packed_bytes(N, C, H, W, OC, KH, KW);
}

int odl_hip_conv2d_pack_weights(const float *w, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH,
                                int SW, int PH, int PW, float *packed, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(w && packed && C > 0 && OC > 0 && KH > 0 && KW > 0 && SH > 0 && SW > 0, "conv2d_pack_weights: bad argument");
    ODL_REQUIRE(odl_hip_conv2d_packed_weights_bytes(N, C, H, W, OC, KH, KW, SH, SW, PH, PW) > 0,
                "conv2d_pack_weights: a forward over this shape reads the filter as it lies");
    const int64_t OH = outsize(H, KH, SH, PH), OW = outsize(W, KW, SW, PW);
    if (g_direct.load(std::memory_order_relaxed) && odl::conv_direct_ok(N, C, H, W, OC, KH, KW, SH, SW, PH, PW, OH, OW))
        return odl::conv_direct_pack(w, C, OC, KH, KW, PH, W, packed, odl::as_stream(stream));
    return odl::conv_implicit_forward_pack(w, C, OC, KH, KW, packed, odl::as_stream(stream));
}

int odl_hip_conv2d_act_packed(const float *x, const float *w, const float *packed, const float *b, int64_t N, int64_t C,
                              int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW,
                              int activation, float *y, void *workspace, size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(activation == -1 || activation == 0 || activation == 7,
                "conv2d: activation must be -1 (none), 0 (relu) or 7 (silu), the unary operator numbers; got %d", activation);
    const int act = activation == 0 ? 1 : (activation == 7 ? 2 : 0);
    ConvGeom g;
    int rc = make_geom(g, "conv2d", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    ODL_REQUIRE(OC > 0, "conv2d: OC must be positive");
    const int64_t M = N * g.OH * g.OW, K = C * KH * KW;
    if (M == 0)
        return ODL_OK;
    hipStream_t st = odl::as_stream(stream);
    // small problems: one launch whatever the window, no workspace (the same shape always takes the same kernel)
    if (g_direct.load(std::memory_order_relaxed) && odl::conv_direct_ok(N, C, H, W, OC, KH, KW, SH, SW, PH, PW, g.OH, g.OW))
    {
        if (packed == nullptr)
        {
            // a caller that keeps no filter copy: one is made in the workspace first
            const size_t need = odl::conv_direct_packed_bytes(C, OC, KH, KW, PH, W);
            ODL_REQUIRE(workspace != nullptr && workspace_bytes >= need && reinterpret_cast<uintptr_t>(workspace) % 16 == 0,
                        "conv2d: this shape needs a 16-byte aligned workspace of %zu bytes, got %zu", need, workspace_bytes);
            rc = odl::conv_direct_pack(w, C, OC, KH, KW, PH, W, static_cast<float *>(workspace), st);
            if (rc != ODL_OK)
                return rc;
            packed = static_cast<const float *>(workspace);
        }
        return odl::conv_direct(x, 0, packed, b, nullptr, 0, y, 0, N, C, H, W, OC, KH, KW, SH, PH, g.OH, g.OW, act, st);
    }
    // a 1x1 window at stride 1 is a plain product per image, y[n] = W . x[n]: operands straight into LDS, bias and
    // activation in the epilogue, the output already NCHW (no K slices, no second launch)
    if (KH == 1 && KW == 1 && SH == 1 && SW == 1 && PH == 0 && PW == 0 && odl::conv1x1_dma_ok(x, w, N, C, H * W, OC))
        return odl::conv1x1_dma(x, w, b, y, N, C, H * W, OC, act, st);
    if (odl::conv_small_forward_ok(N, C, H, W, OC, KH, KW, g.OH, g.OW))
        return odl::conv_small_forward(x, w, b, y, N, C, H, W, OC, KH, KW, SH, SW, PH, PW, g.OH, g.OW, act, st);
    if (odl::conv_patch_forward_ok(x, N, C, H, W, OC, KH, KW, SH, SW, PH, PW) &&
        workspace_bytes >= odl::conv_patch_forward_workspace(N, C, H, W, OC) && reinterpret_cast<uintptr_t>(workspace) % 16 == 0 &&
        workspace)
        return odl::conv_patch_forward(x, w, b, y, N, C, H, W, OC, act, workspace, workspace_bytes, st);
    // (whether or not the caller brought a re-ordered filter copy: the same shape always takes the same kernels)
    const bool by_col = forward_by_col_matrix(N, C, OC, KH, KW, SH, SW, g.OH, g.OW) && workspace &&
                        workspace_bytes >= align256((size_t)(M * K) * sizeof(float)) &&
                        ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(workspace)) & 15) == 0;
    if (!by_col && odl::conv_implicit_forward_ok(w, N, C, H, W, OC, KH, KW, g.OH, g.OW))
        return odl::conv_implicit_forward(x, w, b, y, N, C, H, W, OC, KH, KW, SH, SW, PH, PW, g.OH, g.OW, act, workspace,
                                          workspace_bytes, st,
                                          (packed && reinterpret_cast<uintptr_t>(packed) % 16 == 0) ? packed : nullptr);
    // explicit path: col = im2col(x), then y^T[OC, M] = W2d[OC,K] . col[M,K]^T stored as y[n][oc][p] (+ bias per channel)
    const size_t need = align256((size_t)(M * K) * sizeof(float));
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= need,
                "conv2d: this shape/alignment needs a workspace of %zu bytes, got %zu", need, workspace_bytes);
    float *col = static_cast<float *>(workspace);
    rc = im2col_launch(x, col, g, 1, st);
    if (rc != ODL_OK)
        return rc;
    return odl::sgemm_launch(0, 1, OC, M, K, w, K, col, K, y, 0, b, /*EPI_NCHW_ROWB*/ 2, g.OH * g.OW, 1, nullptr, 0,
                             st, act);
}

int odl_hip_conv2d_relu_max_pool2d_ok(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW,
                                      int PH, int PW, int PKH, int PKW, int PSH, int PSW, int PPH, int PPW)
{
    if (!(KH == 3 && KW == 3 && SH == 1 && SW == 1 && PH == 1 && PW == 1))
        return 0;
    if (!(PKH == 2 && PKW == 2 && PSH == 2 && PSW == 2 && PPH == 0 && PPW == 0) || H < 2 || W < 2 || H % 2 != 0 || W % 2 != 0)
        return 0;
    if (N < 1 || C < 1 || OC < 1)
        return 0;
    // exactly the layers whose convolution alone runs as the thread-per-pixel kernel: the pooled values are then its bits
    if (g_direct.load(std::memory_order_relaxed) && odl::conv_direct_ok(N, C, H, W, OC, KH, KW, SH, SW, PH, PW, H, W))
        return 0;
    return odl::conv_small_forward_ok(N, C, H, W, OC, KH, KW, H, W) ? 1 : 0;
}

int odl_hip_conv2d_relu_max_pool2d(const float *x, const float *w, const float *b, int64_t N, int64_t C, int64_t H, int64_t W,
                                   int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, int PKH, int PKW, int PSH,
                                   int PSW, int PPH, int PPW, float *y, uint64_t *idx, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(x != nullptr && w != nullptr && y != nullptr, "conv2d_relu_max_pool2d: null tensor");
    if (!odl_hip_conv2d_relu_max_pool2d_ok(N, C, H, W, OC, KH, KW, SH, SW, PH, PW, PKH, PKW, PSH, PSW, PPH, PPW))
        return odl::fail(ODL_ERR_INVALID_ARG, "conv2d_relu_max_pool2d: this layer pair has no one-pass kernel (ask "
                                              "odl_hip_conv2d_relu_max_pool2d_ok first)");
    return odl::conv_small_forward_pool(x, w, b, y, idx, nullptr, N, C, H, W, OC, /*relu*/ 1, odl::as_stream(stream));
}

int odl_hip_conv2d_relu_max_pool2d_compact(const float *x, const float *w, const float *b, int64_t N, int64_t C, int64_t H,
                                           int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, int PKH,
                                           int PKW, int PSH, int PSW, int PPH, int PPW, float *y, uint8_t *idx8, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(x != nullptr && w != nullptr && y != nullptr && idx8 != nullptr, "conv2d_relu_max_pool2d: null tensor");
    if (!odl_hip_conv2d_relu_max_pool2d_ok(N, C, H, W, OC, KH, KW, SH, SW, PH, PW, PKH, PKW, PSH, PSW, PPH, PPW))
        return odl::fail(ODL_ERR_INVALID_ARG, "conv2d_relu_max_pool2d: this layer pair has no one-pass kernel (ask "
                                              "odl_hip_conv2d_relu_max_pool2d_ok first)");
    return odl::conv_small_forward_pool(x, w, b, y, nullptr, idx8, N, C, H, W, OC, /*relu*/ 1, odl::as_stream(stream));
}

int odl_hip_set_conv_direct(int enabled)
{
    g_direct.store(enabled ? 1 : 0, std::memory_order_relaxed);
    return ODL_OK;
}

int odl_hip_conv2d_fused_ok(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH,
                            int PW)
{
    if (N <= 0 || C <= 0 || H <= 0 || W <= 0 || KH <= 0 || KW <= 0 || SH <= 0 || SW <= 0 || PH < 0 || PW < 0)
        return 0;
    const int64_t OH = outsize(H, KH, SH, PH), OW = outsize(W, KW, SW, PW);
    return OH > 0 && OW > 0 && odl::conv_direct_ok(N, C, H, W, OC, KH, KW, SH, SW, PH, PW, OH, OW) ? 1 : 0;
}

int odl_hip_conv2d_fused(const float *x, int64_t x_image_stride, const float *packed, const float *b, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW,
                         int activation, const float *residual, int64_t residual_image_stride, float *y,
                         int64_t y_image_stride, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(activation == -1 || activation == 0 || activation == 7,
                "conv2d: activation must be -1 (none), 0 (relu) or 7 (silu), the unary operator numbers; got %d", activation);
    ConvGeom g;
    int rc = make_geom(g, "conv2d", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    ODL_REQUIRE(OC > 0 && x && packed && y, "conv2d_fused: null operand or OC <= 0");
    if (N == 0)
        return ODL_OK;
    ODL_REQUIRE(odl::conv_direct_ok(N, C, H, W, OC, KH, KW, SH, SW, PH, PW, g.OH, g.OW),
                "conv2d_fused: shape not covered (ask odl_hip_conv2d_fused_ok first)");
    ODL_REQUIRE((x_image_stride == 0 || x_image_stride >= C * H * W) && (y_image_stride == 0 || y_image_stride >= OC * g.OH * g.OW) &&
                    (residual_image_stride == 0 || residual_image_stride >= OC * g.OH * g.OW),
                "conv2d_fused: an image stride is shorter than the image it strides over");
    ODL_REQUIRE(x_image_stride < (1ll << 40) && y_image_stride < (1ll << 40) && residual_image_stride < (1ll << 40),
                "conv2d_fused: image stride too large");
    const int act = activation == 0 ? 1 : (activation == 7 ? 2 : 0);
    return odl::conv_direct(x, x_image_stride, packed, b, residual, residual_image_stride, y, y_image_stride, N, C, H, W, OC,
                            KH, KW, SH, PH, g.OH, g.OW, act, odl::as_stream(stream));
}

int odl_hip_conv2d_fused_group_ok(int count, int64_t N, const int64_t *host_C, const int64_t *host_H, const int64_t *host_W,
                                  const int64_t *host_OC)
{
    if (count < 1 || count > 4 || N <= 0 || !host_C || !host_H || !host_W || !host_OC)
        return 0;
    for (int s = 0; s < count; ++s)
        if (host_C[s] <= 0 || host_H[s] <= 0 || host_W[s] <= 0 || host_OC[s] <= 0 ||
            !odl::conv_direct_ok(N, host_C[s], host_H[s], host_W[s], host_OC[s], 1, 1, 1, 1, 0, 0, host_H[s], host_W[s]))
            return 0;
    return 1;
}

int odl_hip_conv2d_fused_group(int count, const float *const *host_x, const int64_t *host_x_image_stride, const float *const *host_packed,
                               const float *const *host_b, int64_t N, const int64_t *host_C, const int64_t *host_H,
                               const int64_t *host_W, const int64_t *host_OC, int activation, float *const *host_y,
                               const int64_t *host_y_image_stride, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(activation == -1 || activation == 0 || activation == 7,
                "conv2d: activation must be -1 (none), 0 (relu) or 7 (silu), the unary operator numbers; got %d", activation);
    ODL_REQUIRE(count >= 1 && count <= 4, "conv2d_fused_group: 1 to 4 members, got %d", count);
    ODL_REQUIRE(host_x && host_x_image_stride && host_packed && host_C && host_H && host_W && host_OC && host_y && host_y_image_stride,
                "conv2d_fused_group: null argument");
    ODL_REQUIRE(N >= 0, "conv2d_fused_group: N must not be negative");
    if (N == 0)
        return ODL_OK;
    ODL_REQUIRE(odl_hip_conv2d_fused_group_ok(count, N, host_C, host_H, host_W, host_OC),
                "conv2d_fused_group: shape not covered (ask odl_hip_conv2d_fused_group_ok first)");
    for (int s = 0; s < count; ++s)
    {
        ODL_REQUIRE(host_x[s] && host_packed[s] && host_y[s], "conv2d_fused_group: null operand of member %d", s);
        const int64_t xi = host_C[s] * host_H[s] * host_W[s], yi = host_OC[s] * host_H[s] * host_W[s];
        ODL_REQUIRE((host_x_image_stride[s] == 0 || host_x_image_stride[s] >= xi) && (host_y_image_stride[s] == 0 || host_y_image_stride[s] >= yi),
                    "conv2d_fused_group: an image stride of member %d is shorter than the image it strides over", s);
        ODL_REQUIRE(host_x_image_stride[s] < (1ll << 40) && host_y_image_stride[s] < (1ll << 40), "conv2d_fused_group: image stride too large");
    }
    const int act = activation == 0 ? 1 : (activation == 7 ? 2 : 0);
    return odl::conv_direct_group(count, host_x, host_x_image_stride, host_packed, host_b, host_y, host_y_image_stride, N, host_C, host_H,
                                  host_W, host_OC, act, odl::as_stream(stream));
}

int odl_hip_conv2d_fused_pair(const float *x, int64_t x_image_stride, const float *packed, const float *b, int64_t N, int64_t C,
                              int64_t H, int64_t W, int64_t OC, int64_t split, int KH, int KW, int SH, int SW, int PH, int PW,
                              int activation, float *y_first, int64_t y_first_image_stride, float *y_second,
                              int64_t y_second_image_stride, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(activation == -1 || activation == 0 || activation == 7,
                "conv2d: activation must be -1 (none), 0 (relu) or 7 (silu), the unary operator numbers; got %d", activation);
    ConvGeom g;
    int rc = make_geom(g, "conv2d", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    ODL_REQUIRE(x && packed && y_first && y_second, "conv2d_fused_pair: null operand");
    ODL_REQUIRE(split > 0 && split < OC, "conv2d_fused_pair: the first convolution's filter count (%lld) must lie inside (0, %lld)",
                (long long)split, (long long)OC);
    if (N == 0)
        return ODL_OK;
    ODL_REQUIRE(odl::conv_direct_ok(N, C, H, W, OC, KH, KW, SH, SW, PH, PW, g.OH, g.OW),
                "conv2d_fused_pair: shape not covered (ask odl_hip_conv2d_fused_ok with the two filter counts added)");
    const int64_t plane = g.OH * g.OW;
    ODL_REQUIRE((x_image_stride == 0 || x_image_stride >= C * H * W) && (y_first_image_stride == 0 || y_first_image_stride >= split * plane) &&
                    (y_second_image_stride == 0 || y_second_image_stride >= (OC - split) * plane),
                "conv2d_fused_pair: an image stride is shorter than the image it strides over");
    ODL_REQUIRE(x_image_stride < (1ll << 40) && y_first_image_stride < (1ll << 40) && y_second_image_stride < (1ll << 40),
                "conv2d_fused_pair: image stride too large");
    const int act = activation == 0 ? 1 : (activation == 7 ? 2 : 0);
    return odl::conv_direct(x, x_image_stride, packed, b, nullptr, 0, y_first, y_first_image_stride, N, C, H, W, OC, KH, KW, SH, PH,
                            g.OH, g.OW, act, odl::as_stream(stream), y_second, y_second_image_stride, split);
}

int odl_hip_conv2d(const float *x, const float *w, const float *b, int64_t N, int64_t C, int64_t H, int64_t W,
                   int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, float *y, void *workspace,
                   size_t workspace_bytes, void *stream)
{
    return odl_hip_conv2d_act(x, w, b, N, C, H, W, OC, KH, KW, SH, SW, PH, PW, -1, y, workspace, workspace_bytes, stream);
}

namespace
{
// The small jobs of a backward pass in one launch: workgroups [0, n_bias) sum a channel of gy each (the longest job
// first), the next n_fold add the weight gradient's partial tiles, the last n_pack make the input-gradient kernel's
// filter copy. Any of the three counts may be zero.
struct SideJobs
{
    odl::SideBias bias;
    odl::SideFold fold;
    odl::SidePack pack;
    unsigned n_bias, n_fold, n_pack;
};

__global__ __launch_bounds__(1024) void conv_backward_side_kernel(const SideJobs j)
{
    __shared__ odl::side_f32x4 lds[1024];
    const unsigned b = blockIdx.x;
    if (b < j.n_bias)
        odl::side_bias(j.bias, b, reinterpret_cast<float *>(lds));
    else if (b < j.n_bias + j.n_fold)
        odl::side_fold(j.fold, b - j.n_bias, lds);
    else
        odl::side_pack(j.pack, b - j.n_bias - j.n_fold, j.n_pack);
}

// workspace regions of conv2d_backward, in order: [col][split-K partials][permuted weights][bias partials]
struct BwdPlan
{
    bool stem;                      // one input channel, 3x3/s1/p1: all three gradients in one pass over gy
    bool wgrad_small, dgrad_small;  // few input channels: the direct kernels, no matrices at all
    bool wgrad_rows;                // 3x3/p1 at stride 1 or 2: output rows walked with the input rows in LDS
    bool wgrad_image;               // 3x3/s1/p1 over small images with few channels: an image at a time resident in LDS
    bool dgrad_patch;               // 3x3/s1/p1: the gradient patch stays in LDS
    bool wgrad_implicit, dgrad_implicit;
    size_t col_bytes, splitk_bytes, wp_bytes, red_bytes;
    size_t total() const { return col_bytes + splitk_bytes + wp_bytes + red_bytes; }
};

BwdPlan plan_backward(const float *gy, const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                      int SH, int SW, int PH, int PW, int64_t OH, int64_t OW)
{
    BwdPlan p{};
    const int64_t M = N * OH * OW, K = C * KH * KW;
    if (odl::conv_stem_backward_ok(gy, N, C, H, W, OC, KH, KW, SH, SW, PH, PW))
    {
        p.stem = true;
        p.splitk_bytes = align256(odl::conv_stem_backward_workspace(N, OC));
        return p;
    }
    p.wgrad_small = odl::conv_small_wgrad_ok(gy, N, C, H, W, OC, KH, KW, OH, OW);
    p.dgrad_small = odl::conv_small_dgrad_ok(gy, N, C, H, W, OC, KH, KW, OH, OW);
    // 3x3 at stride 1 keeps the image size only with a padding of 1
    const int pad = (OH == H && OW == W) ? 1 : -1;
    p.wgrad_rows = !p.wgrad_small && odl::conv_wgrad_rows_ok(gy, x, N, C, H, W, OC, KH, KW, SH, SW, PH, PW, OH, OW);
    p.wgrad_image = !p.wgrad_small && !p.wgrad_rows && odl::conv_image_wgrad_ok(gy, x, N, C, H, W, OC, KH, KW, SH, SW, PH, PW);
    p.wgrad_implicit = !p.wgrad_small && !p.wgrad_rows && !p.wgrad_image && odl::conv_implicit_wgrad_ok(gy, N, C, H, W, OC, KH, KW, OH, OW);
    p.dgrad_patch = !p.dgrad_small && odl::conv_patch_dgrad_ok(gy, N, C, H, W, OC, KH, KW, SH, SW, pad, pad);
    p.dgrad_implicit = !p.dgrad_small && !p.dgrad_patch && odl::conv_implicit_dgrad_ok(gy, N, C, H, W, OC, KH, KW, SH, SW);
    const bool no_col = (p.wgrad_small || p.wgrad_rows || p.wgrad_image || p.wgrad_implicit) && (p.dgrad_small || p.dgrad_patch || p.dgrad_implicit);
    p.col_bytes = no_col ? 0 : align256((size_t)(M * K) * sizeof(float));
    p.splitk_bytes = align256(p.wgrad_small      ? odl::conv_small_wgrad_workspace(N, C, OC, KH, KW, OH, OW)
                              : p.wgrad_rows     ? odl::conv_wgrad_rows_workspace(N, C, H, W, OC, KH, KW, SH, SW, PH, PW, OH, OW)
                              : p.wgrad_image    ? odl::conv_image_wgrad_workspace(N, C, H, W, OC)
                              : p.wgrad_implicit ? odl::conv_implicit_wgrad_workspace(N, C, OC, KH, KW, OH, OW)
                                                 : odl::sgemm_workspace(OC, K, M, 0));
    p.wp_bytes = p.dgrad_small      ? align256(odl::conv_small_dgrad_workspace(C, OC, KH, KW))
                 : p.dgrad_patch    ? align256(odl::conv_patch_dgrad_workspace(N, C, H, W, OC))
                 : p.dgrad_implicit ? align256(odl::conv_implicit_dgrad_workspace(C, OC, KH, KW, N * H * W))
                                    : 0;
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
    return plan_backward(kAlignedProbe, kAlignedProbe, N, C, H, W, OC, KH, KW, SH, SW, PH, PW, OH, OW).total();
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
    const BwdPlan p = plan_backward(gy, x, N, C, H, W, OC, KH, KW, SH, SW, PH, PW, g.OH, g.OW);
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= p.total(),
                "conv2d_backward: this shape/alignment needs a workspace of %zu bytes, got %zu", p.total(),
                workspace_bytes);
    hipStream_t st = odl::as_stream(stream);
    char *ws = static_cast<char *>(workspace);
    float *col = reinterpret_cast<float *>(ws);
    void *splitk_ws = ws + p.col_bytes;
    void *wp_ws = ws + p.col_bytes + p.splitk_bytes;
    void *red_ws = ws + p.col_bytes + p.splitk_bytes + p.wp_bytes;

    if (p.stem)
        return odl::conv_stem_backward(gy, x, w, gx, gw, gb, N, H, W, OC, splitk_ws, p.splitk_bytes, st);
    // gy2d: gy's NCHW buffer read as a row-major [M, OC] matrix exactly as it lies (conv2d.cpp:548)
    // With the row-walking weight gradient, the jobs that follow it — the sum of its partial tiles, the bias gradient,
    // the filter copy of the LDS-patch input gradient — run side by side in one launch.
    const int64_t P = g.OH * g.OW;
    const bool side = gw && p.wgrad_rows;
    const bool side_bias = side && gb && P % 4 == 0 && N * P < (1ll << 31) && OC <= 4096 && reinterpret_cast<uintptr_t>(gy) % 16 == 0;
    const bool side_pack = side && gx && p.dgrad_patch;
    const bool image_pack = gw && !side && p.wgrad_image && !p.wgrad_small && gx && !p.dgrad_small && p.dgrad_patch;
    if (side)
    {
        SideJobs j{};
        rc = odl::conv_wgrad_rows(gy, x, gw, N, C, H, W, OC, SH, g.OH, g.OW, splitk_ws, p.splitk_bytes, st, &j.fold);
        if (rc != ODL_OK)
            return rc;
        j.n_fold = (unsigned)odl::ceil_div(j.fold.n4, 256);
        if (side_bias)
        {
            j.bias = odl::SideBias{gy, gb, (unsigned)(N * P), (unsigned)P, (unsigned)OC, odl::make_fastdiv((unsigned)(P / 4))};
            j.n_bias = (unsigned)OC;
        }
        if (side_pack)
        {
            j.pack = odl::conv_patch_dgrad_pack(w, C, OC, wp_ws);
            j.n_pack = (unsigned)std::min<int64_t>(odl::ceil_div((int64_t)j.pack.Cin * 9 * j.pack.Mpad, 1024), 128);
        }
        hipLaunchKernelGGL(conv_backward_side_kernel, dim3(j.n_bias + j.n_fold + j.n_pack), dim3(1024), 0, st, j);
        ODL_LAUNCH_CHECK();
    }
    else if (gw)
    {
        if (p.wgrad_small)
            rc = odl::conv_small_wgrad(gy, x, gw, N, C, H, W, OC, KH, KW, SH, SW, PH, PW, g.OH, g.OW, splitk_ws,
                                       p.splitk_bytes, st);
        else if (p.wgrad_image)  // (with the bias gradient, if asked for, and the input gradient's filter copy)
        {
            odl::SidePack pack{};
            if (image_pack)
                pack = odl::conv_patch_dgrad_pack(w, C, OC, wp_ws);
            const unsigned n_pack = (unsigned)std::min<int64_t>(odl::ceil_div((int64_t)pack.Cin * 9 * pack.Mpad, 1024), 128);
            rc = odl::conv_image_wgrad(gy, x, gw, gb, N, C, H, W, OC, splitk_ws, p.splitk_bytes, st, image_pack ? &pack : nullptr,
                                       n_pack);
        }
        else if (p.wgrad_implicit)
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
    if (gb && !side_bias && !(gw && p.wgrad_image))
    {
        rc = odl::sum_nchw_channels_launch(gy, N, OC, g.OH * g.OW, gb, red_ws, p.red_bytes, st);
        if (rc != ODL_OK)
            return rc;
    }
    if (gx)
    {
        if (p.dgrad_small)
            rc = odl::conv_small_dgrad(gy, w, gx, N, C, H, W, OC, KH, KW, SH, SW, PH, PW, g.OH, g.OW, wp_ws, p.wp_bytes, st);
        else if (p.dgrad_patch)
            rc = odl::conv_patch_dgrad(gy, w, gx, N, C, H, W, OC, wp_ws, p.wp_bytes, st, side_pack || image_pack);
        else if (p.dgrad_implicit)
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
