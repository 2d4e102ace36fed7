// Max pooling forward (values + window-local uint64 indices) and backward.
// Matches src/mat/origin/cpu/pooling/max_pool2d.cpp:40-224: the window scan starts at cell (0,0), moves
// kh-major, replaces only on strict >, and padding cells count as 0.0 (the reference pools over a zero-padded
// im2col buffer). The reference materialises that 6-D buffer (KH*KW times the input); here each output reads
// its window straight from x, and the backward is a gather per input pixel that adds the matching upstream
// gradients in ascending (kh, kw) — the order of the reference's col2im — so gx is bit-identical.
#include "odl_common.h"

namespace
{
struct PoolGeom
{
    int64_t N, C, H, W, OH, OW;
    int KH, KW, SH, SW, PH, PW;
};

__global__ void max_pool_fwd_kernel(const float *__restrict__ x, float *__restrict__ y, uint64_t *__restrict__ idx,
                                    PoolGeom g)
{
    const int64_t total = g.N * g.C * g.OH * g.OW;
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total)
        return;
    const int64_t ow = t % g.OW, oh = (t / g.OW) % g.OH, nc = t / (g.OW * g.OH);
    const float *p = x + nc * g.H * g.W;
    const int64_t h0 = oh * g.SH - g.PH, w0 = ow * g.SW - g.PW;
    float mv = 0.f;
    uint64_t mi = 0;
    for (int kh = 0; kh < g.KH; ++kh)
    {
        const int64_t h = h0 + kh;
        for (int kw = 0; kw < g.KW; ++kw)
        {
            const int64_t w = w0 + kw;
            const float v = (h >= 0 && h < g.H && w >= 0 && w < g.W) ? p[h * g.W + w] : 0.f;
            if ((kh | kw) == 0)
                mv = v;  // max_pool2d.cpp:110-113
            else if (v > mv)
            {
                mv = v;
                mi = (uint64_t)(kh * g.KW + kw);
            }
        }
    }
    y[t] = mv;
    if (idx)
        idx[t] = mi;
}

__global__ void max_pool_bwd_kernel(const float *__restrict__ gy, const uint64_t *__restrict__ idx,
                                    float *__restrict__ gx, PoolGeom g)
{
    const int64_t total = g.N * g.C * g.H * g.W;
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total)
        return;
    const int64_t w = t % g.W, h = (t / g.W) % g.H, nc = t / (g.W * g.H);
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
            const int64_t o = (nc * g.OH + oh) * g.OW + ow;
            // the reference decodes the index with int arithmetic (max_pool2d.cpp:203-205)
            if ((int)idx[o] == kh * g.KW + kw)
                acc += gy[o];
        }
    }
    gx[t] = acc;
}

// The same two kernels with 32-bit index arithmetic and (for the usual windows)
// kernel size and stride fixed at compile time: on a 64-wide wave the 64-bit divisions and modulos of the general
// kernels above cost several times the memory traffic they serve.
template <int CK, int CS, typename IdxT>
__device__ inline void max_pool_fwd_plane_body(const float *__restrict__ x, float *__restrict__ y, IdxT *__restrict__ idx,
                                               const PoolGeom &g)
{
    const int KH = CK > 0 ? CK : g.KH, KW = CK > 0 ? CK : g.KW;
    const int SH = CS > 0 ? CS : g.SH, SW = CS > 0 ? CS : g.SW;
    const int H = (int)g.H, W = (int)g.W, OW = (int)g.OW;
    const unsigned plane = (unsigned)(g.OH * g.OW);
    const unsigned t = blockIdx.x * 256u + threadIdx.x;
    if (t >= (unsigned)(g.N * g.C) * plane)
        return;
    const unsigned nc = t / plane, r = t - nc * plane;
    const int oh = (int)(r / (unsigned)OW), ow = (int)r - oh * OW;
    const int h0 = oh * SH - g.PH, w0 = ow * SW - g.PW;
    {
        const float *p = x + (int64_t)nc * H * W;
        float mv = 0.f;
        int mi = 0;
#pragma unroll
        for (int kh = 0; kh < KH; ++kh)
        {
            const int h = h0 + kh;
#pragma unroll
            for (int kw = 0; kw < KW; ++kw)
            {
                const int w = w0 + kw;
                const float v = ((unsigned)h < (unsigned)H && (unsigned)w < (unsigned)W) ? p[h * W + w] : 0.f;
                if ((kh | kw) == 0)
                    mv = v;  // max_pool2d.cpp:110-113
                else if (v > mv)
                {
                    mv = v;
                    mi = kh * KW + kw;
                }
            }
        }
        y[t] = mv;
        if (idx)
            idx[t] = (IdxT)mi;
    }
}

template <int CK, int CS>
__global__ __launch_bounds__(256) void max_pool_fwd_plane_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                                 uint64_t *__restrict__ idx, PoolGeom g)
{
    max_pool_fwd_plane_body<CK, CS, uint64_t>(x, y, idx, g);
}

// The same with the window-local index in a byte (windows of up to 256 cells): for callers that keep the indices to
// themselves — a fused layer's backward — an eighth of the index bytes written here and read back there.
template <int CK, int CS>
__global__ __launch_bounds__(256) void max_pool_fwd_plane_u8_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                                    uint8_t *__restrict__ idx, PoolGeom g)
{
    max_pool_fwd_plane_body<CK, CS, uint8_t>(x, y, idx, g);
}

template <int CK, int CS>
__global__ __launch_bounds__(256) void max_pool_bwd_plane_kernel(const float *__restrict__ gy,
                                                                 const uint64_t *__restrict__ idx,
                                                                 float *__restrict__ gx, PoolGeom g)
{
    const int KH = CK > 0 ? CK : g.KH, KW = CK > 0 ? CK : g.KW;
    const int SH = CS > 0 ? CS : g.SH, SW = CS > 0 ? CS : g.SW;
    const int W = (int)g.W, OH = (int)g.OH, OW = (int)g.OW;
    const unsigned plane = (unsigned)(g.H * g.W);
    const int oplane = OH * OW;
    const unsigned t = blockIdx.x * 256u + threadIdx.x;
    if (t >= (unsigned)(g.N * g.C) * plane)
        return;
    const unsigned nc = t / plane, r = t - nc * plane;
    const int h = (int)(r / (unsigned)W), w = (int)r - h * W;
    {
        const float *gp = gy + (int64_t)nc * oplane;
        const uint64_t *ip = idx + (int64_t)nc * oplane;
        float acc = 0.f;
#pragma unroll
        for (int kh = 0; kh < KH; ++kh)
        {
            const int hp = h + g.PH - kh;
            const int oh = hp / SH;
            const bool hok = hp >= 0 && hp % SH == 0 && oh < OH;
#pragma unroll
            for (int kw = 0; kw < KW; ++kw)
            {
                const int wp = w + g.PW - kw;
                const int ow = wp / SW;
                if (hok && wp >= 0 && wp % SW == 0 && ow < OW)
                {
                    const int o = oh * OW + ow;
                    // the reference decodes the index with int arithmetic (max_pool2d.cpp:203-205)
                    if ((int)ip[o] == kh * KW + kw)
                        acc += gp[o];
                }
            }
        }
        gx[t] = acc;
    }
}

// Overlapping windows (3x3/2, 5x5/1 ...: a cell is read by several outputs; windows that do not overlap gain nothing from
// the staging and keep the kernels above) over planes that fit LDS: a workgroup copies `ppw` whole (n, c) planes into LDS
// with coalesced loads and scans the windows there — the K*K reads per output (per input pixel, in the backward, an
// 8-byte index and a gradient each) then cost LDS bandwidth instead of K*K trips through the vector cache (5x5/1 over
// [64,256,40,40]: forward 175 us, backward 788 us with the kernels above). Scan order and comparisons are theirs.
template <int CK, int CS>
__global__ __launch_bounds__(256) void max_pool_fwd_lds_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                               uint64_t *__restrict__ idx, PoolGeom g, int ppw, unsigned planes)
{
    extern __shared__ float pool_sh[];
    const int KH = CK > 0 ? CK : g.KH, KW = CK > 0 ? CK : g.KW;
    const int SH = CS > 0 ? CS : g.SH, SW = CS > 0 ? CS : g.SW;
    const int H = (int)g.H, W = (int)g.W, OW = (int)g.OW;
    const int iplane = H * W, oplane = (int)(g.OH * g.OW);
    const unsigned nc0 = blockIdx.x * (unsigned)ppw;
    const int np = planes - nc0 < (unsigned)ppw ? (int)(planes - nc0) : ppw;
    const float *src = x + (int64_t)nc0 * iplane;
    for (int e = threadIdx.x; e < np * iplane; e += 256)
        pool_sh[e] = src[e];
    __syncthreads();
    float *yo = y + (int64_t)nc0 * oplane;
    uint64_t *io = idx ? idx + (int64_t)nc0 * oplane : nullptr;
    for (int t = threadIdx.x; t < np * oplane; t += 256)
    {
        const int pl = t / oplane, r = t - pl * oplane;
        const int oh = r / OW, ow = r - oh * OW;
        const int h0 = oh * SH - g.PH, w0 = ow * SW - g.PW;
        const float *p = pool_sh + pl * iplane;
        float mv = 0.f;
        int mi = 0;
#pragma unroll
        for (int kh = 0; kh < KH; ++kh)
        {
            const int h = h0 + kh;
#pragma unroll
            for (int kw = 0; kw < KW; ++kw)
            {
                const int w = w0 + kw;
                const bool in = (unsigned)h < (unsigned)H && (unsigned)w < (unsigned)W;
                const float xv = p[in ? h * W + w : 0];
                const float v = in ? xv : 0.f;
                if ((kh | kw) == 0)
                    mv = v;  // max_pool2d.cpp:110-113
                else if (v > mv)
                {
                    mv = v;
                    mi = kh * KW + kw;
                }
            }
        }
        yo[t] = mv;
        if (io)
            io[t] = (uint64_t)mi;
    }
}

template <int CK, int CS>
__global__ __launch_bounds__(256) void max_pool_bwd_lds_kernel(const float *__restrict__ gy, const uint64_t *__restrict__ idx,
                                                               float *__restrict__ gx, PoolGeom g, int ppw, unsigned planes)
{
    extern __shared__ float pool_sh[];
    const int KH = CK > 0 ? CK : g.KH, KW = CK > 0 ? CK : g.KW;
    const int SH = CS > 0 ? CS : g.SH, SW = CS > 0 ? CS : g.SW;
    const int W = (int)g.W, OH = (int)g.OH, OW = (int)g.OW;
    const int iplane = (int)(g.H * g.W), oplane = OH * OW;
    const unsigned nc0 = blockIdx.x * (unsigned)ppw;
    const int np = planes - nc0 < (unsigned)ppw ? (int)(planes - nc0) : ppw;
    float *gsh = pool_sh;                                          // [ppw * oplane] gradients
    int *ish = reinterpret_cast<int *>(pool_sh + ppw * oplane);    // [ppw * oplane] window offsets
    const float *gsrc = gy + (int64_t)nc0 * oplane;
    const uint64_t *isrc = idx + (int64_t)nc0 * oplane;
    for (int e = threadIdx.x; e < np * oplane; e += 256)
    {
        gsh[e] = gsrc[e];
        ish[e] = (int)isrc[e];  // the reference decodes the index with int arithmetic (max_pool2d.cpp:203-205)
    }
    __syncthreads();
    float *out = gx + (int64_t)nc0 * iplane;
    for (int t = threadIdx.x; t < np * iplane; t += 256)
    {
        const int pl = t / iplane, r = t - pl * iplane;
        const int h = r / W, w = r - h * W;
        const float *gp = gsh + pl * oplane;
        const int *ip = ish + pl * oplane;
        float acc = 0.f;
#pragma unroll
        for (int kh = 0; kh < KH; ++kh)
        {
            const int hp = h + g.PH - kh;
            const int oh = hp / SH;
            const bool hok = hp >= 0 && hp % SH == 0 && oh < OH;
#pragma unroll
            for (int kw = 0; kw < KW; ++kw)
            {
                const int wp = w + g.PW - kw;
                const int ow = wp / SW;
                if (hok && wp >= 0 && wp % SW == 0 && ow < OW)
                {
                    const int o = oh * OW + ow;
                    if (ip[o] == kh * KW + kw)
                        acc += gp[o];
                }
            }
        }
        out[t] = acc;
    }
}

// planes per workgroup for the two kernels above (0: the planes do not fit): about 2048 staged elements per workgroup,
// fewer while that would leave compute units without one, within 48 KB of LDS
int planes_per_workgroup(int64_t planes, int64_t staged_per_plane, int bytes_per_elem)
{
    const int64_t cap = 48 * 1024 / bytes_per_elem;
    if (staged_per_plane > cap || planes < 1)
        return 0;
    int64_t ppw = 2048 / staged_per_plane;
    if (ppw > cap / staged_per_plane)
        ppw = cap / staged_per_plane;
    while (ppw > 1 && odl::ceil_div(planes, ppw) < 4 * (int64_t)odl::device_cus())
        --ppw;
    return (int)(ppw < 1 ? 1 : ppw);
}

// Windows that tile the image exactly (stride = window, no padding, H = OH*K, W = OW*K — the 2x2/2 pooling of the
// networks on this path): every input cell belongs to one window, so the gradient is written from the output's side.
// A thread owns one pooled output: it reads its index and its gradient (two independent, coalesced loads — the
// gather kernel above chains the index load and the gradient load, and with one cell per thread that chain is all a
// wave ever does) and writes the K x K cells of its window, gy at the indexed cell and zero elsewhere. The stored
// values are the gather kernel's: 0.f + gy, or 0.f.
template <int K>
__global__ __launch_bounds__(256) void max_pool_bwd_tiled_kernel(const float *__restrict__ gy,
                                                                 const uint64_t *__restrict__ idx,
                                                                 float *__restrict__ gx, unsigned total, int OW,
                                                                 unsigned oplane)
{
    const unsigned o = blockIdx.x * 256u + threadIdx.x;
    if (o >= total)
        return;
    const int hit = (int)idx[o];  // the reference decodes the index with int arithmetic (max_pool2d.cpp:203-205)
    const float v = 0.f + gy[o];
    const unsigned nc = o / oplane, r = o - nc * oplane;
    const int oh = (int)(r / (unsigned)OW), ow = (int)r - oh * OW;
    const int W = OW * K;
    float *dst = gx + ((int64_t)nc * oplane * (K * K)) + (int64_t)(oh * K) * W + ow * K;
#pragma unroll
    for (int kh = 0; kh < K; ++kh)
    {
        if (K == 2)
        {
            float2 row;
            row.x = hit == kh * K ? v : 0.f;
            row.y = hit == kh * K + 1 ? v : 0.f;
            *reinterpret_cast<float2 *>(dst + kh * W) = row;  // W and the window start are even: 8-byte aligned
        }
        else
        {
#pragma unroll
            for (int kw = 0; kw < K; ++kw)
                dst[kh * W + kw] = hit == kh * K + kw ? v : 0.f;
        }
    }
}

// The same with the gradient of the ReLU that produced the pooled tensor folded in: every cell is multiplied by
// (x > 0 ? 1 : 0) as it is written — the product src/operators/activation/relu.cpp:23-29 forms on the pooling gradient
// in a pass of its own (the sign of a zero included).
template <int K>
__global__ __launch_bounds__(256) void max_pool_bwd_tiled_relu_kernel(const float *__restrict__ gy,
                                                                      const uint64_t *__restrict__ idx,
                                                                      const float *__restrict__ x, float *__restrict__ gx,
                                                                      unsigned total, int OW, unsigned oplane)
{
    const unsigned o = blockIdx.x * 256u + threadIdx.x;
    if (o >= total)
        return;
    const int hit = (int)idx[o];
    const float v = 0.f + gy[o];
    const unsigned nc = o / oplane, r = o - nc * oplane;
    const int oh = (int)(r / (unsigned)OW), ow = (int)r - oh * OW;
    const int W = OW * K;
    const int64_t at = ((int64_t)nc * oplane * (K * K)) + (int64_t)(oh * K) * W + ow * K;
#pragma unroll
    for (int kh = 0; kh < K; ++kh)
    {
        if (K == 2)
        {
            const float2 xr = *reinterpret_cast<const float2 *>(x + at + kh * W);
            float2 row;
            row.x = (hit == kh * K ? v : 0.f) * ((xr.x > 0.f) ? 1.f : 0.f);
            row.y = (hit == kh * K + 1 ? v : 0.f) * ((xr.y > 0.f) ? 1.f : 0.f);
            *reinterpret_cast<float2 *>(gx + at + kh * W) = row;
        }
        else
        {
#pragma unroll
            for (int kw = 0; kw < K; ++kw)
                gx[at + kh * W + kw] = (hit == kh * K + kw ? v : 0.f) * ((x[at + kh * W + kw] > 0.f) ? 1.f : 0.f);
        }
    }
}

// The same from the pooled tensor y alone: the cell that receives the gradient is the window's maximum, whose value is
// y[o], so (x > 0) there is (y[o] > 0); every other cell gets the +0 it gets above. The input of the pooling is not
// read (and need not exist any more: conv_small.hip's one-pass convolution + ReLU + pooling never writes it).
template <int K, typename IdxT>
__global__ __launch_bounds__(256) void max_pool_bwd_tiled_relu_pooled_kernel(const float *__restrict__ gy,
                                                                             const IdxT *__restrict__ idx,
                                                                             const float *__restrict__ y, float *__restrict__ gx,
                                                                             unsigned total, int OW, unsigned oplane)
{
    const unsigned o = blockIdx.x * 256u + threadIdx.x;
    if (o >= total)
        return;
    const int hit = (int)idx[o];
    const float v = (0.f + gy[o]) * ((y[o] > 0.f) ? 1.f : 0.f);
    const unsigned nc = o / oplane, r = o - nc * oplane;
    const int oh = (int)(r / (unsigned)OW), ow = (int)r - oh * OW;
    const int W = OW * K;
    const int64_t at = ((int64_t)nc * oplane * (K * K)) + (int64_t)(oh * K) * W + ow * K;
#pragma unroll
    for (int kh = 0; kh < K; ++kh)
    {
        if (K == 2)
        {
            float2 row;
            row.x = hit == kh * K ? v : 0.f;
            row.y = hit == kh * K + 1 ? v : 0.f;
            *reinterpret_cast<float2 *>(gx + at + kh * W) = row;
        }
        else
        {
#pragma unroll
            for (int kw = 0; kw < K; ++kw)
                gx[at + kh * W + kw] = hit == kh * K + kw ? v : 0.f;
        }
    }
}

// gx[i] *= (x[i] > 0 ? 1 : 0) for the window shapes without a fused kernel
__global__ __launch_bounds__(256) void relu_mask_inplace_kernel(float *__restrict__ gx, const float *__restrict__ x, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n)
        gx[i] = gx[i] * ((x[i] > 0.f) ? 1.f : 0.f);
}

// Forward of the 2x2 / stride 2 / no padding pooling over an image whose rows hold a multiple of four floats: a thread
// owns two neighbouring outputs, reads the four cells under them from each of the two image rows with one 16-byte load
// and stores the two maxima (8 bytes) and the two indices (16 bytes) together. The comparisons are those of the general
// kernel: window cells in row-major order, a later cell wins only when it is greater (max_pool2d.cpp:110-139).
__global__ __launch_bounds__(256) void max_pool_fwd_pair_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                                uint64_t *__restrict__ idx, unsigned pairs, int OW2,
                                                                unsigned oplane2)
{
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
    const unsigned t = blockIdx.x * 256u + threadIdx.x;
    if (t >= pairs)
        return;
    const unsigned nc = t / oplane2, r = t - nc * oplane2;
    const int oh = (int)(r / (unsigned)OW2), op = (int)r - oh * OW2;  // op: which pair of the output row
    const int W = OW2 * 4;
    const float *p = x + (int64_t)nc * oplane2 * 8 + (int64_t)(2 * oh) * W + 4 * op;
    const f32x4 top = *reinterpret_cast<const f32x4 *>(p), bot = *reinterpret_cast<const f32x4 *>(p + W);
    f32x2 mv;
    u64x2 mi;
#pragma unroll
    for (int j = 0; j < 2; ++j)
    {
        float m = top[2 * j];
        int w = 0;
        if (top[2 * j + 1] > m)
            m = top[2 * j + 1], w = 1;
        if (bot[2 * j] > m)
            m = bot[2 * j], w = 2;
        if (bot[2 * j + 1] > m)
            m = bot[2 * j + 1], w = 3;
        mv[j] = m, mi[j] = (unsigned long long)w;
    }
    *reinterpret_cast<f32x2 *>(y + 2 * (int64_t)t) = mv;
    if (idx)
        *reinterpret_cast<u64x2 *>(idx + 2 * (int64_t)t) = mi;
}

bool tiles_exactly(const PoolGeom &g)
{
    return g.KH == g.KW && g.SH == g.KH && g.SW == g.KW && g.PH == 0 && g.PW == 0 && g.H == g.OH * g.KH &&
           g.W == g.OW * g.KW && (g.KH == 2 || g.KH == 3);
}

// the 32-bit kernels take everything whose element counts fit
bool plane_ok(const PoolGeom &g)
{
    return g.N * g.C * g.H * g.W < (1ll << 31) - 256 && g.N * g.C * g.OH * g.OW < (1ll << 31) - 256 &&
           (int64_t)g.KH * g.KW < (1 << 20);
}

dim3 plane_grid(int64_t plane, int64_t ncount)
{
    return dim3((unsigned)odl::ceil_div(plane * ncount, 256));
}

// CASE(kernel, stride) for the windows the networks on this path use; anything else runs with run-time sizes
#define ODL_POOL_DISPATCH(KERNEL, ...)                                               \
    do                                                                               \
    {                                                                                \
        const bool sq = g.KH == g.KW && g.SH == g.SW;                                \
        if (sq && g.KH == 2 && g.SH == 2)                                            \
            hipLaunchKernelGGL((KERNEL<2, 2>), grid, dim3(256), 0, st, __VA_ARGS__); \
        else if (sq && g.KH == 3 && g.SH == 2)                                       \
            hipLaunchKernelGGL((KERNEL<3, 2>), grid, dim3(256), 0, st, __VA_ARGS__); \
        else if (sq && g.KH == 3 && g.SH == 1)                                       \
            hipLaunchKernelGGL((KERNEL<3, 1>), grid, dim3(256), 0, st, __VA_ARGS__); \
        else if (sq && g.KH == 5 && g.SH == 1)                                       \
            hipLaunchKernelGGL((KERNEL<5, 1>), grid, dim3(256), 0, st, __VA_ARGS__); \
        else                                                                         \
            hipLaunchKernelGGL((KERNEL<0, 0>), grid, dim3(256), 0, st, __VA_ARGS__); \
    } while (0)

#define ODL_POOL_DISPATCH_LDS(KERNEL, LDS, ...)                                          \
    do                                                                                   \
    {                                                                                    \
        const bool sq = g.KH == g.KW && g.SH == g.SW;                                    \
        if (sq && g.KH == 3 && g.SH == 2)                                                \
            hipLaunchKernelGGL((KERNEL<3, 2>), grid, dim3(256), LDS, st, __VA_ARGS__);   \
        else if (sq && g.KH == 3 && g.SH == 1)                                           \
            hipLaunchKernelGGL((KERNEL<3, 1>), grid, dim3(256), LDS, st, __VA_ARGS__);   \
        else if (sq && g.KH == 5 && g.SH == 1)                                           \
            hipLaunchKernelGGL((KERNEL<5, 1>), grid, dim3(256), LDS, st, __VA_ARGS__);   \
        else                                                                             \
            hipLaunchKernelGGL((KERNEL<0, 0>), grid, dim3(256), LDS, st, __VA_ARGS__);   \
    } while (0)

int make_geom(PoolGeom &g, const char *who, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW,
              int PH, int PW)
{
    ODL_REQUIRE(N >= 0 && C >= 0 && H > 0 && W > 0, "%s: bad input shape", who);
    ODL_REQUIRE(KH > 0 && KW > 0 && SH > 0 && SW > 0 && PH >= 0 && PW >= 0, "%s: bad kernel/stride/pad", who);
    g = PoolGeom{N, C, H, W, (H + 2 * (int64_t)PH - KH) / SH + 1, (W + 2 * (int64_t)PW - KW) / SW + 1,
                 KH, KW, SH, SW, PH, PW};
    ODL_REQUIRE(g.OH > 0 && g.OW > 0, "%s: invalid output size OH=%lld, OW=%lld", who, (long long)g.OH,
                (long long)g.OW);
    return ODL_OK;
}
// `count` K x K / stride 1 / padding K/2 max pools one after the other over an (n, c) plane that stays in LDS: stage j reads
// the plane stage j-1 wrote and writes its own both to LDS and to y[n, (j-1)*C + c] (a detector's SPPF block:
// y1 = pool(x), y2 = pool(y1), y3 = pool(y2), all three concatenated). Each stage scans its windows exactly as
// max_pool_fwd_lds_kernel does (first cell, then strict >, padding cells 0.0), so the values are those of `count`
// separate calls. x and y carry their own distance between images: either may be a run of channels of a wider tensor.
template <int CK>
__global__ __launch_bounds__(256) void max_pool_chain_kernel(const float *__restrict__ x, int64_t x_bs, float *__restrict__ y,
                                                              int64_t y_bs, int C, int H, int W, int K_, int count)
{
    extern __shared__ float chain_sh[];  // two planes
    const int K = CK > 0 ? CK : K_;
    const int plane = H * W, P = K / 2;
    const int n = blockIdx.x / C, c = blockIdx.x - n * C;
    const float *src = x + (int64_t)n * x_bs + (int64_t)c * plane;
    float *cur = chain_sh, *nxt = chain_sh + plane;
    for (int e = threadIdx.x; e < plane; e += 256)
        cur[e] = src[e];
    __syncthreads();
    for (int j = 0; j < count; ++j)
    {
        float *dst = y + (int64_t)n * y_bs + ((int64_t)j * C + c) * plane;
        for (int t = threadIdx.x; t < plane; t += 256)
        {
            const int oh = t / W, ow = t - oh * W;
            float mv = 0.f;
#pragma unroll
            for (int kh = 0; kh < K; ++kh)
            {
                const int h = oh - P + kh;
#pragma unroll
                for (int kw = 0; kw < K; ++kw)
                {
                    const int w = ow - P + kw;
                    const bool in = (unsigned)h < (unsigned)H && (unsigned)w < (unsigned)W;
                    const float xv = cur[in ? h * W + w : 0];
                    const float v = in ? xv : 0.f;
                    if ((kh | kw) == 0)
                        mv = v;
                    else if (v > mv)
                        mv = v;
                }
            }
            nxt[t] = mv;
            dst[t] = mv;
        }
        // the next stage reads this one out of LDS: wait for the LDS writes only, not for the stores to memory
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        float *tmp = cur;
        cur = nxt, nxt = tmp;
    }
}
}  // namespace

extern "C" {

int odl_hip_max_pool2d_chain(const float *x, int64_t x_image_stride, int64_t N, int64_t C, int64_t H, int64_t W, int K,
                             int count, float *y, int64_t y_image_stride, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(x && y && N >= 0 && C > 0 && H > 0 && W > 0, "max_pool2d_chain: bad shape or null operand");
    ODL_REQUIRE(K >= 1 && K % 2 == 1 && K <= 15 && count >= 1 && count <= 8, "max_pool2d_chain: odd window up to 15, 1 to 8 stages");
    ODL_REQUIRE(H * W * 2 * (int64_t)sizeof(float) <= 64 * 1024, "max_pool2d_chain: the plane must fit LDS twice (%lld x %lld)",
                (long long)H, (long long)W);
    ODL_REQUIRE((x_image_stride == 0 || x_image_stride >= C * H * W) && (y_image_stride == 0 || y_image_stride >= count * C * H * W),
                "max_pool2d_chain: an image stride is shorter than the image");
    ODL_REQUIRE(N * C < (1ll << 31), "max_pool2d_chain: too many planes");
    if (N == 0)
        return ODL_OK;
    const size_t lds = (size_t)(2 * H * W) * sizeof(float);
    const int64_t xs = x_image_stride ? x_image_stride : C * H * W, ys = y_image_stride ? y_image_stride : count * C * H * W;
    const dim3 grid((unsigned)(N * C)), block(256);
    if (K == 5)
        hipLaunchKernelGGL(max_pool_chain_kernel<5>, grid, block, lds, odl::as_stream(stream), x, xs, y, ys, (int)C, (int)H, (int)W, K, count);
    else if (K == 3)
        hipLaunchKernelGGL(max_pool_chain_kernel<3>, grid, block, lds, odl::as_stream(stream), x, xs, y, ys, (int)C, (int)H, (int)W, K, count);
    else
        hipLaunchKernelGGL(max_pool_chain_kernel<0>, grid, block, lds, odl::as_stream(stream), x, xs, y, ys, (int)C, (int)H, (int)W, K, count);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_max_pool2d(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW,
                       int PH, int PW, float *y, uint64_t *idx, void *stream)
{
    ODL_REQUIRE_DEVICE();
    PoolGeom g;
    int rc = make_geom(g, "max_pool2d", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    const int64_t total = N * C * g.OH * g.OW;
    if (total == 0)
        return ODL_OK;
    hipStream_t st = odl::as_stream(stream);
    if (plane_ok(g) && tiles_exactly(g) && g.KH == 2 && g.W % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
        (reinterpret_cast<uintptr_t>(y) & 7) == 0 && (reinterpret_cast<uintptr_t>(idx) & 15) == 0)
    {
        const unsigned pairs = (unsigned)(total / 2);
        hipLaunchKernelGGL(max_pool_fwd_pair_kernel, dim3((unsigned)odl::ceil_div((int64_t)pairs, 256)), dim3(256), 0, st,
                           x, y, idx, pairs, (int)(g.OW / 2), (unsigned)(g.OH * g.OW / 2));
    }
    else if (plane_ok(g) && (g.KH > g.SH || g.KW > g.SW) && N * C < (1ll << 31) && planes_per_workgroup(N * C, H * W, 4) > 0)
    {
        const int ppw = planes_per_workgroup(N * C, H * W, 4);
        const dim3 grid((unsigned)odl::ceil_div(N * C, ppw));
        const size_t lds = (size_t)ppw * H * W * sizeof(float);
        ODL_POOL_DISPATCH_LDS(max_pool_fwd_lds_kernel, lds, x, y, idx, g, ppw, (unsigned)(N * C));
    }
    else if (plane_ok(g))
    {
        const dim3 grid = plane_grid(g.OH * g.OW, N * C);
        ODL_POOL_DISPATCH(max_pool_fwd_plane_kernel, x, y, idx, g);
    }
    else
        hipLaunchKernelGGL(max_pool_fwd_kernel, dim3((unsigned)odl::ceil_div(total, 256)), dim3(256), 0, st, x, y, idx,
                           g);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_max_pool2d_backward(const float *gy, const uint64_t *idx, int64_t N, int64_t C, int64_t H, int64_t W,
                                int KH, int KW, int SH, int SW, int PH, int PW, float *gx, void *stream)
{
    ODL_REQUIRE_DEVICE();
    PoolGeom g;
    int rc = make_geom(g, "max_pool2d_backward", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    ODL_REQUIRE(idx != nullptr, "max_pool2d_backward: indices not found");
    const int64_t total = N * C * H * W;
    if (total == 0)
        return ODL_OK;
    hipStream_t st = odl::as_stream(stream);
    if (plane_ok(g) && tiles_exactly(g) && (reinterpret_cast<uintptr_t>(gx) & 7) == 0)
    {
        const unsigned outputs = (unsigned)(N * C * g.OH * g.OW);
        const dim3 grid((unsigned)odl::ceil_div((int64_t)outputs, 256));
        if (g.KH == 2)
            hipLaunchKernelGGL((max_pool_bwd_tiled_kernel<2>), grid, dim3(256), 0, st, gy, idx, gx, outputs, (int)g.OW,
                               (unsigned)(g.OH * g.OW));
        else
            hipLaunchKernelGGL((max_pool_bwd_tiled_kernel<3>), grid, dim3(256), 0, st, gy, idx, gx, outputs, (int)g.OW,
                               (unsigned)(g.OH * g.OW));
    }
    else if (plane_ok(g) && (g.KH > g.SH || g.KW > g.SW) && N * C < (1ll << 31) &&
             planes_per_workgroup(N * C, g.OH * g.OW, 8) > 0)
    {
        const int ppw = planes_per_workgroup(N * C, g.OH * g.OW, 8);
        const dim3 grid((unsigned)odl::ceil_div(N * C, ppw));
        const size_t lds = (size_t)ppw * g.OH * g.OW * 8;
        ODL_POOL_DISPATCH_LDS(max_pool_bwd_lds_kernel, lds, gy, idx, gx, g, ppw, (unsigned)(N * C));
    }
    else if (plane_ok(g))
    {
        const dim3 grid = plane_grid(H * W, N * C);
        ODL_POOL_DISPATCH(max_pool_bwd_plane_kernel, gy, idx, gx, g);
    }
    else
        hipLaunchKernelGGL(max_pool_bwd_kernel, dim3((unsigned)odl::ceil_div(total, 256)), dim3(256), 0, st, gy, idx, gx,
                           g);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_max_pool2d_backward_relu(const float *gy, const uint64_t *idx, const float *x, int64_t N, int64_t C, int64_t H,
                                     int64_t W, int KH, int KW, int SH, int SW, int PH, int PW, float *gx, void *stream)
{
    ODL_REQUIRE_DEVICE();
    PoolGeom g;
    int rc = make_geom(g, "max_pool2d_backward_relu", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    ODL_REQUIRE(idx != nullptr && x != nullptr, "max_pool2d_backward_relu: indices or pooled input missing");
    const int64_t total = N * C * H * W;
    if (total == 0)
        return ODL_OK;
    hipStream_t st = odl::as_stream(stream);
    if (plane_ok(g) && tiles_exactly(g) && ((reinterpret_cast<uintptr_t>(gx) | reinterpret_cast<uintptr_t>(x)) & 7) == 0)
    {
        const unsigned outputs = (unsigned)(N * C * g.OH * g.OW);
        const dim3 grid((unsigned)odl::ceil_div((int64_t)outputs, 256));
        if (g.KH == 2)
            hipLaunchKernelGGL((max_pool_bwd_tiled_relu_kernel<2>), grid, dim3(256), 0, st, gy, idx, x, gx, outputs, (int)g.OW,
                               (unsigned)(g.OH * g.OW));
        else
            hipLaunchKernelGGL((max_pool_bwd_tiled_relu_kernel<3>), grid, dim3(256), 0, st, gy, idx, x, gx, outputs, (int)g.OW,
                               (unsigned)(g.OH * g.OW));
        ODL_LAUNCH_CHECK();
        return ODL_OK;
    }
    rc = odl_hip_max_pool2d_backward(gy, idx, N, C, H, W, KH, KW, SH, SW, PH, PW, gx, stream);
    if (rc != ODL_OK)
        return rc;
    hipLaunchKernelGGL(relu_mask_inplace_kernel, dim3((unsigned)odl::ceil_div(total, 256)), dim3(256), 0, st, gx, x, total);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

}  // extern "C"

template <typename IdxT>
static int pool_backward_relu_pooled(const float *gy, const IdxT *idx, const float *y, int64_t N, int64_t C, int64_t H, int64_t W,
                                     int KH, int KW, int SH, int SW, int PH, int PW, float *gx, void *stream)
{
    ODL_REQUIRE_DEVICE();
    PoolGeom g;
    int rc = make_geom(g, "max_pool2d_backward_relu_pooled", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    ODL_REQUIRE(idx != nullptr && y != nullptr && gy != nullptr && gx != nullptr, "max_pool2d_backward_relu_pooled: null tensor");
    if (N * C * H * W == 0)
        return ODL_OK;
    // windows that tile the image: each cell belongs to one window, so the mask of the pooled value is the mask of the cell
    ODL_REQUIRE(plane_ok(g) && tiles_exactly(g) && (reinterpret_cast<uintptr_t>(gx) & 7) == 0,
                "max_pool2d_backward_relu_pooled: only for windows that tile the image (2x2/2, 3x3/3, no padding)");
    const unsigned outputs = (unsigned)(N * C * g.OH * g.OW);
    const dim3 grid((unsigned)odl::ceil_div((int64_t)outputs, 256));
    hipStream_t st = odl::as_stream(stream);
    if (g.KH == 2)
        hipLaunchKernelGGL((max_pool_bwd_tiled_relu_pooled_kernel<2, IdxT>), grid, dim3(256), 0, st, gy, idx, y, gx, outputs,
                           (int)g.OW, (unsigned)(g.OH * g.OW));
    else
        hipLaunchKernelGGL((max_pool_bwd_tiled_relu_pooled_kernel<3, IdxT>), grid, dim3(256), 0, st, gy, idx, y, gx, outputs,
                           (int)g.OW, (unsigned)(g.OH * g.OW));
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

extern "C" {

int odl_hip_max_pool2d_backward_relu_pooled(const float *gy, const uint64_t *idx, const float *y, int64_t N, int64_t C,
                                            int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH, int PW, float *gx,
                                            void *stream)
{
    return pool_backward_relu_pooled<uint64_t>(gy, idx, y, N, C, H, W, KH, KW, SH, SW, PH, PW, gx, stream);
}

int odl_hip_max_pool2d_backward_relu_pooled_compact(const float *gy, const uint8_t *idx8, const float *y, int64_t N, int64_t C,
                                                    int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH, int PW,
                                                    float *gx, void *stream)
{
    return pool_backward_relu_pooled<uint8_t>(gy, idx8, y, N, C, H, W, KH, KW, SH, SW, PH, PW, gx, stream);
}

int odl_hip_max_pool2d_compact(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW,
                               int PH, int PW, float *y, uint8_t *idx8, void *stream)
{
    ODL_REQUIRE_DEVICE();
    PoolGeom g;
    int rc = make_geom(g, "max_pool2d", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    ODL_REQUIRE(x != nullptr && y != nullptr && idx8 != nullptr, "max_pool2d_compact: null tensor");
    ODL_REQUIRE((int64_t)KH * KW <= 256 && plane_ok(g), "max_pool2d_compact: a window of at most 256 cells and 32-bit sizes");
    if (N * C * g.OH * g.OW == 0)
        return ODL_OK;
    hipStream_t st = odl::as_stream(stream);
    const dim3 grid = plane_grid(g.OH * g.OW, N * C);
    ODL_POOL_DISPATCH(max_pool_fwd_plane_u8_kernel, x, y, idx8, g);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

}  // extern "C"
