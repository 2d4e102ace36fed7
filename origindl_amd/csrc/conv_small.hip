// Convolutions over an image with very few channels — the first layer of an image network (1 or 3 channels under a
// 3x3 to 6x6 window). Their GEMM has a reduction of 9 to 27 terms (or, for the input gradient, 1 to 3 output rows): a
// 64- or 128-row MFMA tile would spend nearly all of its multiplies on padding, and the im2col matrix would be written
// and read for nothing. Here one thread owns one pixel and walks the few terms itself on the vector ALU; the filter is
// read through wave-uniform addresses, so it lives in scalar registers, and the kernels move the activations exactly
// once. Results follow src/mat/origin/cpu/conv/conv2d.cpp:404-599 like the GEMM path does: the output gradient is read
// as the row-major [N*OH*OW, OC] matrix that its NCHW buffer spells out as it lies (conv2d.cpp:548).
#include "odl_common.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace
{
struct SmallGeom
{
    int N, C, H, W, OC, OH, OW, SH, SW, PH, PW;
    unsigned total;            // pixels the grid covers: N*OH*OW (forward, weight gradient) or N*H*W (input gradient)
    odl::FastDiv by_w, by_h;   // the pixel decode: by (OW, OH) or by (W, H)
};

constexpr int kThreads = 256;

// v + (v of another lane of the same row of 16), the other lane picked by a DPP control; a lane whose source falls
// outside its row adds zero
template <int CTRL>
__device__ inline float dpp_add(float v)
{
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
constexpr int kRowShl = 0x100;         // row_shl:n — lane i reads lane i+n of its row
constexpr int kQuadSwap1 = 0xB1;       // quad_perm:[1,0,3,2] — lane i reads lane i^1
constexpr int kQuadSwap2 = 0x4E;       // quad_perm:[2,3,0,1] — lane i reads lane i^2
constexpr int kRowHalfMirror = 0x141;  // lane i reads lane 7-i of its half row
constexpr int kRowMirror = 0x140;      // lane i reads lane 15-i of its row

// y[n][oc][oh][ow] = act(sum_{c,kh,kw} x[n][c][oh*SH-PH+kh][ow*SW-PW+kw] * w[oc][c][kh][kw] + b[oc]); one thread per
// output pixel, OCB output channels per thread (blockIdx.y picks the group). The KH*KW window of one input channel is
// held in registers and reused by all OCB channels.
template <int KH, int KW, int OCB>
__global__ __launch_bounds__(kThreads) void conv_small_fwd_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                                 const float *__restrict__ bias, float *__restrict__ y,
                                                                 SmallGeom g, int act)
{
    const unsigned pix = blockIdx.x * kThreads + threadIdx.x;
    if (pix >= g.total)
        return;
    const unsigned t = odl::fastdiv(pix, g.by_w), ow = pix - t * g.OW;
    const unsigned n = odl::fastdiv(t, g.by_h), oh = t - n * g.OH;
    const int oc0 = blockIdx.y * OCB;
    const int ih0 = (int)oh * g.SH - g.PH, iw0 = (int)ow * g.SW - g.PW;
    float acc[OCB];
#pragma unroll
    for (int o = 0; o < OCB; ++o)
        acc[o] = 0.f;
    for (int c = 0; c < g.C; ++c)
    {
        const float *xp = x + ((size_t)n * g.C + c) * g.H * g.W;
        float xr[KH * KW];
#pragma unroll
        for (int kh = 0; kh < KH; ++kh)
#pragma unroll
            for (int kw = 0; kw < KW; ++kw)
            {
                const int ih = ih0 + kh, iw = iw0 + kw;
                const bool in = (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W;
                xr[kh * KW + kw] = in ? xp[ih * g.W + iw] : 0.f;
            }
        const float *wc = w + ((size_t)oc0 * g.C + c) * (KH * KW);
#pragma unroll
        for (int o = 0; o < OCB; ++o)
        {
            const float *wo = wc + (size_t)o * g.C * (KH * KW);  // the same address in every lane
#pragma unroll
            for (int j = 0; j < KH * KW; ++j)
                acc[o] = fmaf(xr[j], wo[j], acc[o]);
        }
    }
    const size_t plane = (size_t)g.OH * g.OW;
    float *yp = y + ((size_t)n * g.OC + oc0) * plane + (size_t)oh * g.OW + ow;
#pragma unroll
    for (int o = 0; o < OCB; ++o)
    {
        float v = acc[o];
        if (bias)
            v = v + bias[oc0 + o];
        yp[o * plane] = odl::apply_act(v, act);
    }
}

// A detector's stem — 6x6 / stride 2 / padding 2 over C input channels into 16 filters (YOLOv5's first layer,
// [N,3,H,W] -> [N,16,H/2,W/2]) — on the matrix cores. As a thread-per-pixel kernel it was 216 bounds-tested loads and
// 3456 multiply-adds in a row per thread (31 us at [4,3,320,320]). Here a workgroup takes one output row: the six input
// rows under it, with their zero borders, go to LDS once in whole-row loads, and y[oc][pixel] = sum_k w[oc][k] *
// patch[k][pixel] runs as 16x16x4 MFMAs over tiles of sixteen pixels — A, the filter, sits in registers for the whole
// kernel (C*9 steps of four k), B is one LDS read a step at an offset that is constant per lane and step plus twice the
// pixel. Rows of D are filters and columns pixels, so the stores are runs of sixteen pixels of one filter's plane.
#ifdef ODL_STEM6_DBG
__device__ unsigned long long g_stem6_dbg[1024 * 8];
#define ODL_STEM6_STAMP(i) do { if (threadIdx.x == 0 && blockIdx.x < 1024) g_stem6_dbg[blockIdx.x * 8 + (i)] = wall_clock64(); } while (0)
#else
#define ODL_STEM6_STAMP(i) do { } while (0)
#endif
template <int C>
__global__ __launch_bounds__(kThreads) void conv_stem6_mfma_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                                  const float *__restrict__ bias, float *__restrict__ y, int H,
                                                                  int W, int OH, int OW, int pitch, int act)
{
    constexpr int STEPS = C * 9;  // of four k = (c, kh, kw) each
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    extern __shared__ __attribute__((aligned(16))) float rows[];  // [C][6][pitch]: input columns -2 .. W+1 of six rows
    const int n = blockIdx.x / OH, oh = blockIdx.x - n * OH;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, j = lane & 15, kq = lane >> 4;
    ODL_STEM6_STAMP(0);
    // the lane's four filters' biases, asked for now (a load in the epilogue is a trip to memory in the way of the stores)
    float bv[4] = {0.f, 0.f, 0.f, 0.f};
    if (bias)
    {
#pragma unroll
        for (int r = 0; r < 4; ++r)
            bv[r] = bias[4 * kq + r];
    }
    // the filter: lane (j, kq) holds w[j][4s + kq] for every step s
    // (through LDS: read where it lies, every lane's 27 values are 27 loads of 64 scattered addresses a wave — more time
    // in the address unit than the whole product takes on the matrix cores)
    float *wl = rows + ((C * 6 * pitch + 3) & ~3);  // [16][C*36] (on a 16-byte boundary, and so is what follows it)
    for (int e = t; e < 16 * C * 36; e += kThreads)
        wl[e] = w[e];
    int koff[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
    {
        const int k = 4 * s + kq, c = k / 36, r = k - c * 36, kh = r / 6, kw = r - kh * 6;
        koff[s] = (c * 6 + kh) * pitch + kw;
    }
    ODL_STEM6_STAMP(1);
    // the six input rows: 2*oh - 2 .. 2*oh + 3 of each channel, zeros outside the image. All of a thread's loads are in
    // flight together (one after the other, each waiting for the last, they were most of the kernel's time): 16-byte
    // pieces where the rows allow it.
    if (W % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0)
    {
        const int quads = W / 4, total = C * 6 * quads;
        constexpr int U = 6;
        for (int e0 = t; e0 < total; e0 += U * kThreads)
        {
            f32x4 v[U];
            int at[U];
#pragma unroll
            for (int u = 0; u < U; ++u)
            {
                const int e = e0 + u * kThreads, ec = e < total ? e : e0;
                const int cr = ec / quads, q = ec - cr * quads, c = cr / 6, r = cr - c * 6;
                const int ih = 2 * oh - 2 + r;
                const bool in = e < total && (unsigned)ih < (unsigned)H;
                v[u] = *reinterpret_cast<const f32x4 *>(x + ((size_t)(n * C + c) * H + (in ? ih : 0)) * W + 4 * q);
                if (!in)
                    v[u] = f32x4{0.f, 0.f, 0.f, 0.f};
                at[u] = e < total ? cr * pitch + 2 + 4 * q : -1;
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (at[u] >= 0)
                {
                    float *d = rows + at[u];
                    d[0] = v[u][0], d[1] = v[u][1], d[2] = v[u][2], d[3] = v[u][3];
                }
        }
        for (int e = t; e < C * 6 * 4; e += kThreads)  // the two border columns on either side
        {
            const int cr = e >> 2, b = e & 3;
            rows[cr * pitch + (b < 2 ? b : W + b)] = 0.f;
        }
    }
    else
    {
#pragma unroll 8
        for (int e = t; e < C * 6 * pitch; e += kThreads)
        {
            const int cr = e / pitch, col = e - cr * pitch, c = cr / 6, r = cr - c * 6;
            const int ih = 2 * oh - 2 + r, iw = col - 2;
            const bool in = (unsigned)ih < (unsigned)H && (unsigned)iw < (unsigned)W;
            rows[e] = in ? x[((size_t)(n * C + c) * H + ih) * W + iw] : 0.f;
        }
    }
    __syncthreads();
    float aw[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
        aw[s] = wl[j * (C * 36) + 4 * s + kq];
    ODL_STEM6_STAMP(2);
    const int tiles = (OW + 15) / 16;
    constexpr int kWavesHere = kThreads / 64;
    // A wave takes every fourth tile, starting from a tile that turns with the workgroup (the waves with one tile more
    // than the others then fall on different SIMDs from one workgroup of a compute unit to the next), two tiles at a time
    // where it has two: the MFMAs of one accumulator wait for each other, those of two take turns.
    // The finished tiles meet in LDS (behind the rows and the filter) and leave as whole rows of one filter's plane: stored
    // from the registers every instruction wrote four 64-byte pieces of four planes, and the stores took twice the time
    // of the products.
    float *outs = wl + 16 * C * 36;  // [16][opitch]
    const int opitch = ((OW + 3) / 4 * 4) | 4;  // (4 mod 8: the four filters of a lane's store fall into different banks)
    auto store_tile = [&](int pix, const f32x4 &acc) {
        if (pix < OW)
        {
#pragma unroll
            for (int r = 0; r < 4; ++r)
            {
                const int oc = 4 * kq + r;
                float v = acc[r];
                if (bias)
                    v = v + bv[r];
                outs[oc * opitch + pix] = odl::apply_act(v, act);
            }
        }
    };
    const int first = (wave + (int)blockIdx.x) % kWavesHere;
    for (int tile = first; tile < tiles; tile += 2 * kWavesHere)
    {
        const int tile1 = tile + kWavesHere;
        const int pix0 = tile * 16 + j, pix1 = tile1 * 16 + j;
        const float *bp0 = rows + 2 * (pix0 < OW ? pix0 : OW - 1);  // (pixels past the row compute a copy that is not stored)
        f32x4 acc0 = {0.f, 0.f, 0.f, 0.f};
        if (tile1 < tiles)
        {
            const float *bp1 = rows + 2 * (pix1 < OW ? pix1 : OW - 1);
            f32x4 acc1 = {0.f, 0.f, 0.f, 0.f};
            // every B operand of the pair asked for before the first MFMA: the reads' latency is paid once, not once a batch
            float b0[STEPS], b1[STEPS];
#pragma unroll
            for (int s = 0; s < STEPS; ++s)
                b0[s] = bp0[koff[s]], b1[s] = bp1[koff[s]];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < STEPS; ++s)
            {
                acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(aw[s], b0[s], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(aw[s], b1[s], acc1, 0, 0, 0);
            }
            ODL_STEM6_STAMP(4);
            store_tile(pix0, acc0);
            store_tile(pix1, acc1);
            ODL_STEM6_STAMP(5);
        }
        else
        {
            float b0[STEPS];
#pragma unroll
            for (int s = 0; s < STEPS; ++s)
                b0[s] = bp0[koff[s]];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < STEPS; ++s)
                acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(aw[s], b0[s], acc0, 0, 0, 0);
            store_tile(pix0, acc0);
        }
    }
    __syncthreads();
    float *yrow = y + ((size_t)n * 16 * OH + oh) * OW;  // filter oc's row lies oc * OH * OW floats further
    if (OW % 4 == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0)
    {
        const int q = OW / 4;
        for (int e = t; e < 16 * q; e += kThreads)
        {
            const int oc = e / q, c4 = e - oc * q;
            *reinterpret_cast<f32x4 *>(yrow + (size_t)oc * OH * OW + 4 * c4) = *reinterpret_cast<const f32x4 *>(outs + oc * opitch + 4 * c4);
        }
    }
    else
    {
        for (int e = t; e < 16 * OW; e += kThreads)
        {
            const int oc = e / OW, c = e - oc * OW;
            yrow[(size_t)oc * OH * OW + c] = outs[oc * opitch + c];
        }
    }
    ODL_STEM6_STAMP(3);
}

// The 3x3 / stride 1 / padding 1 convolution above with ReLU and a 2x2 / stride 2 max pooling behind it in one pass: a
// thread owns one pooled pixel, computes the four convolution outputs under it (a 4x4 patch of each input channel in
// registers) for OCB channels, applies bias and activation and keeps the maximum and its place in the window. Per
// convolution output the terms are added in the order of conv_small_fwd_kernel, and the window is compared in the order
// of the pooling kernels (row-major, a later cell wins only when it is greater, max_pool2d.cpp:110-139): the pooled
// values and indices are those of the two kernels run one after the other — without the 4x larger tensor between them.
template <int OCB, typename IdxT>
__global__ __launch_bounds__(kThreads) void conv_small_fwd_pool_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                                      const float *__restrict__ bias, float *__restrict__ y,
                                                                      IdxT *__restrict__ idx, SmallGeom g, int act)
{
    // (g.OH, g.OW: the pooled extents; g.total = N * OH * OW)
    const unsigned pix = blockIdx.x * kThreads + threadIdx.x;
    if (pix >= g.total)
        return;
    const unsigned t = odl::fastdiv(pix, g.by_w), pw = pix - t * g.OW;
    const unsigned n = odl::fastdiv(t, g.by_h), ph = t - n * g.OH;
    const int oc0 = blockIdx.y * OCB;
    const int ih0 = 2 * (int)ph - 1, iw0 = 2 * (int)pw - 1;
    float acc[4][OCB];
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int o = 0; o < OCB; ++o)
            acc[q][o] = 0.f;
    for (int c = 0; c < g.C; ++c)
    {
        const float *xp = x + ((size_t)n * g.C + c) * g.H * g.W;
        // the 4x4 patch: rows 2ph-1 .. 2ph+2, columns 2pw-1 .. 2pw+2. With H and W even only its first and last row and
        // column can lie outside the image, and the two middle columns start at an even offset: one 8-byte load a row
        // where the image allows it
        float xr[4][4];
        const bool left = pw > 0, right = (int)pw + 1 < g.OW, pair_ok = (reinterpret_cast<uintptr_t>(xp) & 7) == 0;
#pragma unroll
        for (int r = 0; r < 4; ++r)
        {
            const int ih = ih0 + r;
            const bool row = (r != 0 || ph > 0) && (r != 3 || (int)ph + 1 < g.OH);
            const float *rp = xp + (row ? ih : 0) * g.W + 2 * (int)pw;
            float2 mid;
            if (pair_ok)
                mid = *reinterpret_cast<const float2 *>(rp);
            else
                mid.x = rp[0], mid.y = rp[1];
            const float l = left ? rp[-1] : 0.f, rr = right ? rp[2] : 0.f;
            xr[r][0] = row ? l : 0.f, xr[r][1] = row ? mid.x : 0.f, xr[r][2] = row ? mid.y : 0.f, xr[r][3] = row ? rr : 0.f;
        }
        const float *wc = w + ((size_t)oc0 * g.C + c) * 9;
#pragma unroll
        for (int o = 0; o < OCB; ++o)
        {
            const float *wo = wc + (size_t)o * g.C * 9;  // the same address in every lane
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int j = 0; j < 9; ++j)
                    acc[q][o] = fmaf(xr[q / 2 + j / 3][q % 2 + j % 3], wo[j], acc[q][o]);
        }
    }
    const size_t plane = (size_t)g.OH * g.OW;
    const size_t at = ((size_t)n * g.OC + oc0) * plane + (size_t)ph * g.OW + pw;
#pragma unroll
    for (int o = 0; o < OCB; ++o)
    {
        float v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            v[q] = acc[q][o];
            if (bias)
                v[q] = v[q] + bias[oc0 + o];
            v[q] = odl::apply_act(v[q], act);
        }
        float m = v[0];
        int win = 0;
        if (v[1] > m)
            m = v[1], win = 1;
        if (v[2] > m)
            m = v[2], win = 2;
        if (v[3] > m)
            m = v[3], win = 3;
        y[at + o * plane] = m;
        if (idx)
            idx[at + o * plane] = (IdxT)win;
    }
}

// The same convolution for the larger windows (5x5, 6x6): there the filter no longer fits the scalar registers, and
// reading it through them in pieces leaves the wave waiting on one short load after another. The workgroup stages its
// OCB channels' filter in LDS once, as [c][tap][oc], and every lane reads it from there 16 bytes at a time (one address
// for the whole wave); a thread computes two output pixels, half the grid apart, so that each filter read feeds two
// multiply-adds. Per output the terms are added in the same order as in the kernel above.
template <int KH, int KW, int OCB>
__global__ __launch_bounds__(kThreads) void conv_small_fwd_lds_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                                     const float *__restrict__ bias, float *__restrict__ y,
                                                                     SmallGeom g, int act, unsigned half)
{
    constexpr int KK = KH * KW;
    extern __shared__ __attribute__((aligned(16))) float wl[];  // [C][KK][OCB]
    const int oc0 = blockIdx.y * OCB;
    for (int e = threadIdx.x; e < g.C * KK * OCB; e += kThreads)
    {
        const int o = e % OCB, ck = e / OCB;
        wl[e] = w[(size_t)(oc0 + o) * g.C * KK + ck];
    }
    __syncthreads();
    const unsigned first = blockIdx.x * kThreads + threadIdx.x;
    bool live[2];
    unsigned n[2], oh[2], ow[2];
#pragma unroll
    for (int p = 0; p < 2; ++p)
    {
        const unsigned pix = first + p * half;
        live[p] = first < half && pix < g.total;
        const unsigned pp = live[p] ? pix : 0;
        const unsigned t = odl::fastdiv(pp, g.by_w);
        ow[p] = pp - t * g.OW;
        n[p] = odl::fastdiv(t, g.by_h);
        oh[p] = t - n[p] * g.OH;
    }
    float acc[2][OCB];
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
        for (int o = 0; o < OCB; ++o)
            acc[p][o] = 0.f;
    for (int c = 0; c < g.C; ++c)
    {
        float xr[2][KK];
#pragma unroll
        for (int p = 0; p < 2; ++p)
        {
            const float *xp = x + ((size_t)n[p] * g.C + c) * g.H * g.W;
            const int ih0 = (int)oh[p] * g.SH - g.PH, iw0 = (int)ow[p] * g.SW - g.PW;
#pragma unroll
            for (int kh = 0; kh < KH; ++kh)
#pragma unroll
                for (int kw = 0; kw < KW; ++kw)
                {
                    const int ih = ih0 + kh, iw = iw0 + kw;
                    const bool in = live[p] && (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W;
                    xr[p][kh * KW + kw] = in ? xp[ih * g.W + iw] : 0.f;
                }
        }
        const f32x4 *wc = reinterpret_cast<const f32x4 *>(wl + (size_t)c * KK * OCB);
#pragma unroll
        for (int k = 0; k < KK; ++k)
#pragma unroll
            for (int q = 0; q < OCB / 4; ++q)
            {
                const f32x4 wv = wc[k * (OCB / 4) + q];
#pragma unroll
                for (int p = 0; p < 2; ++p)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        acc[p][q * 4 + j] = fmaf(xr[p][k], wv[j], acc[p][q * 4 + j]);
            }
    }
    const size_t plane = (size_t)g.OH * g.OW;
#pragma unroll
    for (int p = 0; p < 2; ++p)
    {
        if (!live[p])
            continue;
        float *yp = y + ((size_t)n[p] * g.OC + oc0) * plane + (size_t)oh[p] * g.OW + ow[p];
#pragma unroll
        for (int o = 0; o < OCB; ++o)
        {
            float v = acc[p][o];
            if (bias)
                v = v + bias[oc0 + o];
            yp[o * plane] = odl::apply_act(v, act);
        }
    }
}

// gW[oc][k] = sum_m gy2d[m][oc] * col[m][k], col[m][(c,kh,kw)] = x[n][c][oh*SH-PH+kh][ow*SW-PW+kw] for m = (n,oh,ow).
// A thread owns 8 consecutive channels of gy2d's rows m = first + i*rows_per_pass and all K = C*KH*KW columns: 8*K
// private sums. G = OC/8 = 2^LGG neighbouring lanes share a row, so a wave reads whole rows of gy2d, 16 bytes a lane. At
// the end the lanes of equal channel group are added — inside a row of 16 lanes by DPP moves, across rows and waves
// through LDS — and the workgroup writes one [OC][K] partial; conv_small_partial_sum_kernel adds the partials in a
// fixed order.
template <int C, int KH, int KW, int LGG>
__global__ __launch_bounds__(kThreads) void conv_small_wgrad_kernel(const float *__restrict__ gy, const float *__restrict__ x,
                                                                   float *__restrict__ part, SmallGeom g,
                                                                   unsigned rows_per_block)
{
    constexpr int K = C * KH * KW;
    constexpr int G = 1 << LGG, lgG = LGG;
    constexpr int EK = 8 * G * K;
    // partial sums kept per row of 16 lanes (16 of them in the workgroup) when that fits, else per wave (4)
    constexpr int NR = (16 * EK * 4 <= 48 * 1024) ? 16 : 4;
    __shared__ float red[NR * EK];
    const int ocg = threadIdx.x & (G - 1);
    const unsigned rows_per_pass = kThreads >> lgG;
    const unsigned m_begin = blockIdx.x * rows_per_block;
    const unsigned m_end = (m_begin + rows_per_block < g.total) ? m_begin + rows_per_block : g.total;
    float acc[8][K];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < K; ++j)
            acc[i][j] = 0.f;
    // U rows at a time, their loads issued together; a row past the end contributes zeros
    constexpr int U = K <= 9 ? 4 : 1;
    for (unsigned mb = m_begin + (threadIdx.x >> lgG); mb < m_end; mb += U * rows_per_pass)
    {
        float xr[U][K];
        f32x4 gr[U][2];
#pragma unroll
        for (int u = 0; u < U; ++u)
        {
            const unsigned m = mb + u * rows_per_pass;
            const bool live = m < m_end;
            const unsigned mm = live ? m : mb;
            const unsigned t = odl::fastdiv(mm, g.by_w), ow = mm - t * g.OW;
            const unsigned n = odl::fastdiv(t, g.by_h), oh = t - n * g.OH;
            const int ih0 = (int)oh * g.SH - g.PH, iw0 = (int)ow * g.SW - g.PW;
            const float *xp = x + (size_t)n * C * g.H * g.W;
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int kh = 0; kh < KH; ++kh)
#pragma unroll
                    for (int kw = 0; kw < KW; ++kw)
                    {
                        const int ih = ih0 + kh, iw = iw0 + kw;
                        const bool in = live && (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W;
                        xr[u][(c * KH + kh) * KW + kw] = in ? xp[((size_t)c * g.H + ih) * g.W + iw] : 0.f;
                    }
            const f32x4 *gp = reinterpret_cast<const f32x4 *>(gy + (size_t)mm * g.OC + ocg * 8);
            const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
            gr[u][0] = live ? gp[0] : zero;
            gr[u][1] = live ? gp[1] : zero;
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < K; ++j)
                    acc[i][j] = fmaf(gr[u][i / 4][i % 4], xr[u][j], acc[i][j]);
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < K; ++j)
        {
            float v = acc[i][j];
            if (LGG <= 0)
                v = dpp_add<kRowShl + 1>(v);
            if (LGG <= 1)
                v = dpp_add<kRowShl + 2>(v);
            if (LGG <= 2)
                v = dpp_add<kRowShl + 4>(v);
            v = dpp_add<kRowShl + 8>(v);  // lanes 0..G-1 of each row now hold the row's sums
            if (NR == 16)
            {
                if ((lane & 15) < G)
                    red[(wave * 4 + (lane >> 4)) * EK + (ocg * 8 + i) * K + j] = v;
            }
            else
            {
                v += __shfl_xor(v, 16);
                v += __shfl_xor(v, 32);
                if (lane < G)
                    red[wave * EK + (ocg * 8 + i) * K + j] = v;
            }
        }
    __syncthreads();
    float *out = part + (size_t)blockIdx.x * EK;
    for (int e = threadIdx.x; e < EK; e += kThreads)
    {
        float r[NR];
#pragma unroll
        for (int q = 0; q < NR; ++q)
            r[q] = red[q * EK + e];
#pragma unroll
        for (int w = NR / 2; w > 0; w /= 2)
#pragma unroll
            for (int q = 0; q < w; ++q)
                r[q] = r[q] + r[q + w];
        out[e] = r[0];
    }
}

// out[e] = sum_p part[p][e]: one wave per element, lane l adds partials l, l+64, ... in ascending order, then the
// lanes are added pairwise — the same order on every run
__global__ __launch_bounds__(kThreads) void conv_small_partial_sum_kernel(const float *__restrict__ part, int nparts, int E,
                                                                         float *__restrict__ out)
{
    const int e = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    if (e >= E)
        return;
    const int lane = threadIdx.x & 63;
    float s = 0.f;
    for (int p = lane; p < nparts; p += 64)
        s += part[(size_t)p * E + e];
    for (int off = 32; off > 0; off >>= 1)
        s += __shfl_xor(s, off);
    if (lane == 0)
        out[e] = s;
}

// wp[(tap*C + c)*OC + oc] = w[oc][c][tap]: for one tap and input channel the OC factors lie side by side
__global__ void conv_small_permute_kernel(const float *__restrict__ w, float *__restrict__ wp, int OC, int C, int KHW)
{
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= OC * C * KHW)
        return;
    const int oc = t % OC, c = (t / OC) % C, tap = t / (OC * C);
    wp[t] = w[((size_t)oc * C + c) * KHW + tap];
}

// gx[n][c][ih][iw] = sum over the taps (kh,kw) that reach the pixel of gx_col[m][(c,kh,kw)] =
// sum_oc gy2d[m][oc] * w[oc][c][kh][kw], m = (n, (ih+PH-kh)/SH, (iw+PW-kw)/SW) — the reference's GEMM followed by its
// col2im, without the matrix between them. L = OC/4 = 2^LGL neighbouring lanes share a pixel: lane `sub` holds
// channels 4*sub..4*sub+3 of every tap's factors in registers and reads those 16 bytes of each gy2d row, so a wave
// reads whole rows; the L partial sums meet through DPP moves. A thread walks kDgPixels pixels with the same factors.
// Every tap's row is loaded whether the tap reaches the pixel or not (row 0 stands in), so that the loads of all
// taps are in flight together; a tap that does not reach the pixel is left out of the sum.
constexpr int kDgThreads = 512, kDgPixels = 4;
template <int C, int KH, int KW, int LGL>
__global__ __launch_bounds__(kDgThreads) void conv_small_dgrad_kernel(const float *__restrict__ gy, const float *__restrict__ wp,
                                                                     float *__restrict__ gx, SmallGeom g)
{
    constexpr int L = 1 << LGL;
    constexpr int kPer = kDgThreads >> LGL;  // pixels per pass of the workgroup
    const int sub = threadIdx.x & (L - 1);
    const f32x4 *gy4 = reinterpret_cast<const f32x4 *>(gy);
    f32x4 wv[KH * KW][C];
#pragma unroll
    for (int tap = 0; tap < KH * KW; ++tap)
#pragma unroll
        for (int c = 0; c < C; ++c)
            wv[tap][c] = reinterpret_cast<const f32x4 *>(wp)[(tap * C + c) * L + sub];
    const bool unit = g.SH == 1 && g.SW == 1;
#pragma unroll 1
    for (int it = 0; it < kDgPixels; ++it)
    {
        const unsigned pix = (blockIdx.x * kDgPixels + it) * kPer + (threadIdx.x >> LGL);
        const bool live = pix < g.total;  // the same in all lanes of a pixel
        const unsigned pp = live ? pix : g.total - 1;
        const unsigned t = odl::fastdiv(pp, g.by_w), iw = pp - t * g.W;
        const unsigned n = odl::fastdiv(t, g.by_h), ih = t - n * g.H;
        float acc[C];
#pragma unroll
        for (int c = 0; c < C; ++c)
            acc[c] = 0.f;
#pragma unroll
        for (int kh = 0; kh < KH; ++kh)
        {
            const int th = (int)ih + g.PH - kh;
            const int oh = unit ? th : th / g.SH;
            const bool hit_h = th >= 0 && oh < g.OH && (unit || oh * g.SH == th);
#pragma unroll
            for (int kw = 0; kw < KW; ++kw)
            {
                const int tw = (int)iw + g.PW - kw;
                const int ow = unit ? tw : tw / g.SW;
                const bool hit = hit_h && tw >= 0 && ow < g.OW && (unit || ow * g.SW == tw);
                const size_t m = hit ? ((size_t)n * g.OH + oh) * g.OW + ow : 0;
                const f32x4 v = gy4[m * L + sub];
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    const f32x4 wq = wv[kh * KW + kw][c];
                    float s = v[0] * wq[0];
                    s = fmaf(v[1], wq[1], s);
                    s = fmaf(v[2], wq[2], s);
                    s = fmaf(v[3], wq[3], s);
                    acc[c] += hit ? s : 0.f;
                }
            }
        }
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            float v = acc[c];
            if (LGL >= 1)
                v = dpp_add<kQuadSwap1>(v);
            if (LGL >= 2)
                v = dpp_add<kQuadSwap2>(v);
            if (LGL >= 3)
                v = dpp_add<kRowHalfMirror>(v);  // the quads are uniform by now, so 7-i stands for i^4
            if (LGL >= 4)
                v = dpp_add<kRowMirror>(v);      // and 15-i for i^8
            if (sub == 0 && live)
                gx[((size_t)n * C + c) * g.H * g.W + (size_t)ih * g.W + iw] = v;
        }
    }
}

// The input gradient at stride 1, row-stationary: a workgroup owns a band of image rows of one image. First every row
// of gy2d the band needs (the band's rows plus KH-1 rows of halo) is read exactly once — L lanes a row, 16 bytes each —
// and turned into its KH*KW*C products gx_col[m][(c,kh,kw)] (per lane four multiply-adds a product, the L partial
// products joined by DPP moves), which go to LDS; then one thread per image pixel adds the pixel's taps from LDS in
// ascending (kh, kw) order, as col2im does. The per-pixel kernel above reads every gy2d row KH*KW times instead.
constexpr int kBandThreads = 256, kBandRows = 4;  // rows in flight per lane group
template <int C, int KH, int KW, int LGL>
__global__ __launch_bounds__(kBandThreads) void conv_small_dgrad_band_kernel(const float *__restrict__ gy,
                                                                            const float *__restrict__ wp,
                                                                            float *__restrict__ gx, SmallGeom g, int band_h,
                                                                            int nbands, int ldr)
{
    constexpr int L = 1 << LGL, KK = KH * KW;
    constexpr int kPer = kBandThreads >> LGL;  // gy2d rows per pass of the workgroup
    extern __shared__ float prod[];            // [rows of the band][ldr], ldr >= KK*C and odd
    const int n = blockIdx.x / nbands, band = blockIdx.x - n * nbands;
    const int h0 = band * band_h, h1 = (h0 + band_h < g.H) ? h0 + band_h : g.H;
    // output rows that reach the band: oh = ih + PH - kh
    const int r0 = (h0 + g.PH - (KH - 1) > 0) ? h0 + g.PH - (KH - 1) : 0;
    const int r1 = (h1 + g.PH < g.OH) ? h1 + g.PH : g.OH;
    const int nrows = (r1 > r0 ? r1 - r0 : 0) * g.OW;
    const int sub = threadIdx.x & (L - 1), grp = threadIdx.x >> LGL;
    const f32x4 *gy4 = reinterpret_cast<const f32x4 *>(gy) + ((size_t)n * g.OH + r0) * g.OW * L;
    f32x4 wv[KK][C];
#pragma unroll
    for (int tap = 0; tap < KK; ++tap)
#pragma unroll
        for (int c = 0; c < C; ++c)
            wv[tap][c] = reinterpret_cast<const f32x4 *>(wp)[(tap * C + c) * L + sub];
    for (int rb = grp; rb < nrows; rb += kPer * kBandRows)
    {
        f32x4 v[kBandRows];
#pragma unroll
        for (int u = 0; u < kBandRows; ++u)
        {
            const int r = rb + u * kPer;
            v[u] = gy4[(size_t)(r < nrows ? r : rb) * L + sub];
        }
#pragma unroll
        for (int u = 0; u < kBandRows; ++u)
        {
            const int r = rb + u * kPer;
#pragma unroll
            for (int tap = 0; tap < KK; ++tap)
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    const f32x4 wq = wv[tap][c];
                    float s = v[u][0] * wq[0];
                    s = fmaf(v[u][1], wq[1], s);
                    s = fmaf(v[u][2], wq[2], s);
                    s = fmaf(v[u][3], wq[3], s);
                    if (LGL >= 1)
                        s = dpp_add<kQuadSwap1>(s);
                    if (LGL >= 2)
                        s = dpp_add<kQuadSwap2>(s);
                    if (LGL >= 3)
                        s = dpp_add<kRowHalfMirror>(s);
                    if (LGL >= 4)
                        s = dpp_add<kRowMirror>(s);
                    if (sub == 0 && r < nrows)
                        prod[r * ldr + tap * C + c] = s;
                }
        }
    }
    __syncthreads();
    const int npix = (h1 - h0) * g.W;
    for (int p = threadIdx.x; p < npix; p += kBandThreads)
    {
        const int hl = (int)odl::fastdiv((unsigned)p, g.by_w), iw = p - hl * g.W;
        const int ih = h0 + hl;
        float acc[C];
#pragma unroll
        for (int c = 0; c < C; ++c)
            acc[c] = 0.f;
#pragma unroll
        for (int kh = 0; kh < KH; ++kh)
        {
            const int oh = ih + g.PH - kh;
            if (oh < r0 || oh >= r1)
                continue;
#pragma unroll
            for (int kw = 0; kw < KW; ++kw)
            {
                const int ow = iw + g.PW - kw;
                if (ow < 0 || ow >= g.OW)
                    continue;
                const float *q = prod + ((oh - r0) * g.OW + ow) * ldr + (kh * KW + kw) * C;
#pragma unroll
                for (int c = 0; c < C; ++c)
                    acc[c] += q[c];
            }
        }
#pragma unroll
        for (int c = 0; c < C; ++c)
            gx[(((size_t)n * C + c) * g.H + ih) * g.W + iw] = acc[c];
    }
}

// band height for the kernel above (0: use the per-pixel kernel): about 512 workgroups, and a band's products within
// 48 KB of LDS
int band_height(const SmallGeom &g, int C, int KH, int KW, int &nbands, int &ldr)
{
    if (g.SH != 1 || g.SW != 1)
        return 0;
    ldr = (KH * KW * C) | 1;
    int want = (int)odl::ceil_div(512, g.N);
    if (want < 1)
        want = 1;
    if (want > g.H)
        want = g.H;
    for (nbands = want; nbands <= g.H; ++nbands)
    {
        const int bh = (int)odl::ceil_div(g.H, nbands);
        if ((int64_t)(bh + KH - 1) * g.OW * ldr * (int64_t)sizeof(float) <= 48 * 1024)
        {
            nbands = (int)odl::ceil_div(g.H, bh);
            return bh;
        }
    }
    return 0;
}

bool aligned16(const void *p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

// the (C, KH, KW) triples the backward kernels are instantiated for
bool backward_shape(int64_t C, int KH, int KW)
{
    return KH == KW && ((C == 1 && (KH == 3 || KH == 5)) || (C == 3 && KH == 3));
}

SmallGeom make_small(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int SH, int SW, int PH, int PW, int64_t OH,
                     int64_t OW, bool over_image)
{
    SmallGeom g;
    g.N = (int)N, g.C = (int)C, g.H = (int)H, g.W = (int)W, g.OC = (int)OC, g.OH = (int)OH, g.OW = (int)OW;
    g.SH = SH, g.SW = SW, g.PH = PH, g.PW = PW;
    g.total = (unsigned)(over_image ? N * H * W : N * OH * OW);
    g.by_w = odl::make_fastdiv((unsigned)(over_image ? W : OW));
    g.by_h = odl::make_fastdiv((unsigned)(over_image ? H : OH));
    return g;
}

// sizes all of these kernels index with 32 bits
bool small_sizes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int64_t OH, int64_t OW)
{
    return N * OH * OW < (1ll << 31) && N * H * W < (1ll << 31) && C * H * W < (1ll << 31) && OC <= 4096 && H > 0 && W > 0 &&
           OH > 0 && OW > 0;
}

struct WgradPlan
{
    int lgG;
    unsigned rows_per_block, nblocks;
};

WgradPlan plan_wgrad(int64_t M, int64_t OC)
{
    WgradPlan p;
    p.lgG = OC == 8 ? 0 : (OC == 16 ? 1 : (OC == 32 ? 2 : 3));
    const unsigned rpp = (unsigned)kThreads >> p.lgG;
    // about three workgroups per compute unit at most, each a whole number of four-row rounds
    unsigned rows = (unsigned)odl::ceil_div(M, 768);
    rows = (unsigned)odl::ceil_div(rows, 4 * rpp) * 4 * rpp;
    p.rows_per_block = rows;
    p.nblocks = (unsigned)odl::ceil_div(M, rows);
    return p;
}
}  // namespace

namespace odl
{
bool conv_small_forward_ok(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int64_t OH, int64_t OW)
{
    if (!(KH == KW && (KH == 3 || KH == 5 || KH == 6)) || OC % 16 != 0 || OC > 128)
        return false;
    // few enough terms that the matrix units would mostly multiply padding: a short reduction, or a narrow output
    if (!(C * KH * KW <= 32 || (OC <= 16 && C <= 4)))
        return false;
    if (C * KH * KW * 16 * 4 > 48 * 1024)  // the staged filter of the larger windows
        return false;
    return small_sizes(N, C, H, W, OC, OH, OW);
}

int conv_small_forward(const float *x, const float *w, const float *b, float *y, int64_t N, int64_t C, int64_t H, int64_t W,
                       int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, int64_t OH, int64_t OW, int act,
                       hipStream_t st)
{
    const SmallGeom g = make_small(N, C, H, W, OC, SH, SW, PH, PW, OH, OW, false);
    if (KH == 6 && KW == 6 && SH == 2 && SW == 2 && PH == 2 && PW == 2 && C == 3 && OC == 16 && N * OH < (1ll << 31) &&
        ((W + 4) * 18 + 4 + 16 * 108 + 16 * (OW + 8)) * 4 <= 64 * 1024)
    {
        // a detector's stem: a workgroup per output row, the products on the matrix cores
        const int pitch = (int)W + 4;
        hipLaunchKernelGGL((conv_stem6_mfma_kernel<3>), dim3((unsigned)(N * OH)), dim3(kThreads),
                           (size_t)(3 * 6 * pitch + 4 + 16 * 3 * 36 + 16 * ((((int)OW + 3) / 4 * 4) | 4)) * sizeof(float), st, x, w, b, y,
                           (int)H, (int)W, (int)OH, (int)OW, pitch, act);
    }
    else if (KH == 3)
    {
        const dim3 grid((unsigned)ceil_div(g.total, kThreads), (unsigned)(OC / 16));
        hipLaunchKernelGGL((conv_small_fwd_kernel<3, 3, 16>), grid, dim3(kThreads), 0, st, x, w, b, y, g, act);
    }
    else
    {
        // two pixels a thread: the second one `half` pixels after the first
        const unsigned half = (unsigned)ceil_div(g.total, 2);
        const dim3 grid((unsigned)ceil_div(half, kThreads), (unsigned)(OC / 16));
        const size_t lds = (size_t)C * KH * KW * 16 * sizeof(float);
        if (KH == 5)
            hipLaunchKernelGGL((conv_small_fwd_lds_kernel<5, 5, 16>), grid, dim3(kThreads), lds, st, x, w, b, y, g, act, half);
        else
            hipLaunchKernelGGL((conv_small_fwd_lds_kernel<6, 6, 16>), grid, dim3(kThreads), lds, st, x, w, b, y, g, act, half);
    }
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

// 3x3 / stride 1 / padding 1 + activation + 2x2 / stride 2 pooling, H and W even; y [N, OC, H/2, W/2], idx may be null
// (idx: 8-byte indices, or idx8: one byte each, or neither)
int conv_small_forward_pool(const float *x, const float *w, const float *b, float *y, uint64_t *idx, uint8_t *idx8, int64_t N,
                            int64_t C, int64_t H, int64_t W, int64_t OC, int act, hipStream_t st)
{
    SmallGeom g = make_small(N, C, H, W, OC, 1, 1, 1, 1, H / 2, W / 2, false);
    // four channels a thread: eight times the pooled pixels in threads, enough waves to hide each other's filter loads
    const dim3 grid((unsigned)ceil_div(g.total, kThreads), (unsigned)(OC / 4));
    if (idx8)
        hipLaunchKernelGGL((conv_small_fwd_pool_kernel<4, uint8_t>), grid, dim3(kThreads), 0, st, x, w, b, y, idx8, g, act);
    else
        hipLaunchKernelGGL((conv_small_fwd_pool_kernel<4, uint64_t>), grid, dim3(kThreads), 0, st, x, w, b, y, idx, g, act);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

bool conv_small_wgrad_ok(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int64_t OH,
                         int64_t OW)
{
    return backward_shape(C, KH, KW) && (OC == 8 || OC == 16 || OC == 32 || OC == 64) && aligned16(gy) &&
           small_sizes(N, C, H, W, OC, OH, OW);
}

size_t conv_small_wgrad_workspace(int64_t N, int64_t C, int64_t OC, int KH, int KW, int64_t OH, int64_t OW)
{
    return (size_t)plan_wgrad(N * OH * OW, OC).nblocks * (size_t)(OC * C * KH * KW) * sizeof(float);
}

int conv_small_wgrad(const float *gy, const float *x, float *gw, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
                     int KH, int KW, int SH, int SW, int PH, int PW, int64_t OH, int64_t OW, void *workspace,
                     size_t workspace_bytes, hipStream_t st)
{
    const SmallGeom g = make_small(N, C, H, W, OC, SH, SW, PH, PW, OH, OW, false);
    const WgradPlan p = plan_wgrad(N * OH * OW, OC);
    const int EK = (int)(OC * C * KH * KW);
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= (size_t)p.nblocks * EK * sizeof(float),
                "conv2d_backward: the weight-gradient partials need %zu bytes, got %zu",
                (size_t)p.nblocks * EK * sizeof(float), workspace_bytes);
    float *part = static_cast<float *>(workspace);
#define ODL_SMALL_WGRAD(CV, KV, LG)                                                                                \
    hipLaunchKernelGGL((conv_small_wgrad_kernel<CV, KV, KV, LG>), dim3(p.nblocks), dim3(kThreads), 0, st, gy, x, part, g, \
                       p.rows_per_block)
#define ODL_SMALL_WGRAD_G(CV, KV)     \
    do                                \
    {                                 \
        if (p.lgG == 0)               \
            ODL_SMALL_WGRAD(CV, KV, 0); \
        else if (p.lgG == 1)          \
            ODL_SMALL_WGRAD(CV, KV, 1); \
        else if (p.lgG == 2)          \
            ODL_SMALL_WGRAD(CV, KV, 2); \
        else                          \
            ODL_SMALL_WGRAD(CV, KV, 3); \
    } while (0)
    if (C == 1 && KH == 3)
        ODL_SMALL_WGRAD_G(1, 3);
    else if (C == 1)
        ODL_SMALL_WGRAD_G(1, 5);
    else
        ODL_SMALL_WGRAD_G(3, 3);
#undef ODL_SMALL_WGRAD_G
#undef ODL_SMALL_WGRAD
    ODL_LAUNCH_CHECK();
    hipLaunchKernelGGL(conv_small_partial_sum_kernel, dim3((unsigned)ceil_div(EK, kThreads / 64)), dim3(kThreads), 0, st,
                       part, (int)p.nblocks, EK, gw);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

bool conv_small_dgrad_ok(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int64_t OH,
                         int64_t OW)
{
    return backward_shape(C, KH, KW) && (OC == 8 || OC == 16 || OC == 32 || OC == 64) && aligned16(gy) &&
           small_sizes(N, C, H, W, OC, OH, OW);
}

size_t conv_small_dgrad_workspace(int64_t C, int64_t OC, int KH, int KW)
{
    return (size_t)(OC * C * KH * KW) * sizeof(float);
}

int conv_small_dgrad(const float *gy, const float *w, float *gx, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
                     int KH, int KW, int SH, int SW, int PH, int PW, int64_t OH, int64_t OW, void *workspace,
                     size_t workspace_bytes, hipStream_t st)
{
    const SmallGeom g = make_small(N, C, H, W, OC, SH, SW, PH, PW, OH, OW, true);
    const int EK = (int)(OC * C * KH * KW);
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= (size_t)EK * sizeof(float) && aligned16(workspace),
                "conv2d_backward: the reordered filter needs %zu bytes at a 16-byte boundary, got %zu",
                (size_t)EK * sizeof(float), workspace_bytes);
    float *wp = static_cast<float *>(workspace);
    hipLaunchKernelGGL(conv_small_permute_kernel, dim3((unsigned)ceil_div(EK, 256)), dim3(256), 0, st, w, wp, (int)OC,
                       (int)C, KH * KW);
    ODL_LAUNCH_CHECK();
    const int lgL = OC == 8 ? 1 : (OC == 16 ? 2 : (OC == 32 ? 3 : 4));
    const dim3 grid((unsigned)ceil_div(g.total, (int64_t)kDgPixels * (kDgThreads >> lgL)));
    int nbands = 0, ldr = 0;
    const int band_h = band_height(g, (int)C, KH, KW, nbands, ldr);
    const dim3 band_grid((unsigned)(N * (band_h > 0 ? nbands : 1)));
    const size_t band_lds = band_h > 0 ? (size_t)(band_h + KH - 1) * OW * ldr * sizeof(float) : 0;
#define ODL_SMALL_DGRAD(CV, KV, LG)                                                                                     \
    do                                                                                                                  \
    {                                                                                                                   \
        if (band_h > 0)                                                                                                 \
            hipLaunchKernelGGL((conv_small_dgrad_band_kernel<CV, KV, KV, LG>), band_grid, dim3(kBandThreads), band_lds, \
                               st, gy, wp, gx, g, band_h, nbands, ldr);                                                 \
        else                                                                                                            \
            hipLaunchKernelGGL((conv_small_dgrad_kernel<CV, KV, KV, LG>), grid, dim3(kDgThreads), 0, st, gy, wp, gx, g);  \
    } while (0)
#define ODL_SMALL_DGRAD_OC(CV, KV)      \
    do                                  \
    {                                   \
        if (lgL == 1)                   \
            ODL_SMALL_DGRAD(CV, KV, 1); \
        else if (lgL == 2)              \
            ODL_SMALL_DGRAD(CV, KV, 2); \
        else if (lgL == 3)              \
            ODL_SMALL_DGRAD(CV, KV, 3); \
        else                            \
            ODL_SMALL_DGRAD(CV, KV, 4); \
    } while (0)
    if (C == 1 && KH == 3)
        ODL_SMALL_DGRAD_OC(1, 3);
    else if (C == 1)
        ODL_SMALL_DGRAD_OC(1, 5);
    else
        ODL_SMALL_DGRAD_OC(3, 3);
#undef ODL_SMALL_DGRAD_OC
#undef ODL_SMALL_DGRAD
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}
}  // namespace odl
