// Backward pass of a one-channel 3x3 / stride 1 / padding 1 convolution — the first layer of an image network on
// grey-scale input (the reference's MNIST CNN, tests/example/mnist/conv_mnist.cpp) — in one pass over the output gradient.
//
// The three results of src/mat/origin/cpu/conv/conv2d.cpp:514-599 all read gy: gW and gx read its NCHW buffer as a
// row-major [N*OH*OW, OC] matrix exactly as it lies (conv2d.cpp:548), gb reads it as NCHW (566-580). With one input
// channel the products are 9 terms wide; as three kernels plus their small helpers (a partial-sum fold, a filter
// permutation, two passes for the bias) the backward was six launches that each read all of gy or waited on one that
// did. Here one workgroup takes one image at a time: the image's gy block (OC x H*W floats, contiguous, and both readings
// of it stay inside the block) goes to LDS once, and out of LDS come
//   gW[oc][tap] += sum_p gy2d[p][oc] * x[p + tap]          lanes along oc, rows of the image dealt over the waves
//   gb[oc]      += sum_q block[oc*P + q]                    the NCHW reading of the same floats
//   gx[pixel]    = sum_taps (sum_oc gy2d[p][oc] * w[oc][tap])  per output pixel p first, then gathered per input pixel
//                                                           in ascending (kh, kw), the order of the reference's col2im
// The filter and bias gradients are kept in registers across the workgroup's images, added over its waves in a fixed
// order at the end and written as one partial per workgroup; a second small launch adds the partials in workgroup order.
#include "odl_common.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace
{
constexpr int kT = 1024;  // threads per workgroup: sixteen waves, the one workgroup a compute unit's LDS holds

struct StemGeom
{
    const float *gy, *x, *w;
    float *gx, *part;  // part[workgroup][OC*9 + OC]
    int N, H, W, P;    // P = H*W
};

// (time stamps of a workgroup's phases for a test harness that includes this file with ODL_STEM_DBG defined; nothing otherwise)
#ifdef ODL_STEM_DBG
__device__ unsigned long long g_stem_dbg[256 * 16];
#define ODL_STEM_STAMP(i) do { if (threadIdx.x == 0 && blockIdx.x < 256) g_stem_dbg[blockIdx.x * 16 + (i)] = wall_clock64(); } while (0)
#else
#define ODL_STEM_STAMP(i) do { } while (0)
#endif

template <int OC>
__global__ __launch_bounds__(kT) void conv_stem_backward_kernel(const StemGeom g, const float *__restrict__ wf)
{
    constexpr int LDG = OC + 1;   // floats per gy2d row in LDS: odd, so that lanes along the rows meet different banks
    constexpr int G = kT / OC;    // groups of OC lanes
    extern __shared__ float lds[];
    const int P = g.P, W = g.W, H = g.H, PW = W + 2;
    float *gs = lds;                      // [P][LDG]
    float *xs = gs + P * LDG;             // [(H+2)][(W+2)], zero border
    float *gc = xs + (H + 2) * PW;        // [P][9]
    const int t = threadIdx.x, oc = t % OC, grp = t / OC;
    // (wf, the filter, is read through addresses that are the same for every lane: it travels through scalar loads and
    // sits in scalar registers; out of LDS its nine factors per filter were nine reads a lane for nine multiply-adds)

    for (int i = t; i < (H + 2) * PW; i += kT)
        xs[i] = 0.f;

    float acc[9], accb = 0.f;
#pragma unroll
    for (int k = 0; k < 9; ++k)
        acc[k] = 0.f;

    ODL_STEM_STAMP(0);
    for (int n = blockIdx.x; n < g.N; n += gridDim.x)
    {
        __syncthreads();  // the previous image has been read
        ODL_STEM_STAMP(1);
        const float *blk = g.gy + (int64_t)n * OC * P;
        // (the input pixels and eight 16-byte pieces of the block in flight per thread — a 28 x 28 image with 32 filters
        // is one such round, one trip to memory; a lane's four floats belong to one gy2d row)
        constexpr int U = 8;
        const int quads = OC * P / 4;
        const float xv = t < P ? g.x[(int64_t)n * P + t] : 0.f;
        const bool quadsums = P % 4 == 0;  // then no 16-byte piece lies across two channels of the NCHW reading
        float *ps = gc;                    // [OC * P / 4] sums of the pieces, in the space of the products that come later
        for (int e0 = t; e0 < quads; e0 += U * kT)
        {
            f32x4 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u)
            {
                const int e4 = e0 + u * kT;
                v[u] = *reinterpret_cast<const f32x4 *>(blk + 4 * (e4 < quads ? e4 : e0));
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
            {
                const int e4 = e0 + u * kT;
                if (e4 < quads)
                {
                    const int e = 4 * e4, p = e / OC, c0 = e % OC;
                    float *d = gs + p * LDG + c0;
                    d[0] = v[u][0], d[1] = v[u][1], d[2] = v[u][2], d[3] = v[u][3];
                    if (quadsums)  // (for the bias gradient, below)
                        ps[e4] = (v[u][0] + v[u][1]) + (v[u][2] + v[u][3]);
                }
            }
        }
        for (int i = t; i < P; i += kT)
        {
            const int h = i / W, w = i - h * W;
            xs[(h + 1) * PW + w + 1] = i == t ? xv : g.x[(int64_t)n * P + i];
        }
        __syncthreads();
        ODL_STEM_STAMP(2);

        // ---- filter gradient: the group's rows of the image, a window of the padded input sliding along each
        for (int oh = grp; oh < H; oh += G)
        {
            const float *r0 = xs + oh * PW, *r1 = r0 + PW, *r2 = r1 + PW;
            float a0 = r0[0], a1 = r0[1], b0 = r1[0], b1 = r1[1], c0 = r2[0], c1 = r2[1];
            const float *grow = gs + (oh * W) * LDG + oc;
            // one output pixel: its gy2d value times the window (p, q, r = the window's columns, left to right)
#define ODL_STEM_PIXEL(ow_, pa, qa, ra, pb, qb, rb, pc, qc, rc)                                                  \
    {                                                                                                            \
        ra = r0[(ow_) + 2], rb = r1[(ow_) + 2], rc = r2[(ow_) + 2];                                              \
        const float gv = grow[(ow_) * LDG];                                                                      \
        acc[0] = fmaf(gv, pa, acc[0]), acc[1] = fmaf(gv, qa, acc[1]), acc[2] = fmaf(gv, ra, acc[2]);             \
        acc[3] = fmaf(gv, pb, acc[3]), acc[4] = fmaf(gv, qb, acc[4]), acc[5] = fmaf(gv, rb, acc[5]);             \
        acc[6] = fmaf(gv, pc, acc[6]), acc[7] = fmaf(gv, qc, acc[7]), acc[8] = fmaf(gv, rc, acc[8]);             \
    }
            float a2, b2, c2;
            int ow = 0;
            for (; ow + 3 <= W; ow += 3)  // three pixels a turn: the window's columns change roles instead of registers
            {
                ODL_STEM_PIXEL(ow, a0, a1, a2, b0, b1, b2, c0, c1, c2)
                ODL_STEM_PIXEL(ow + 1, a1, a2, a0, b1, b2, b0, c1, c2, c0)
                ODL_STEM_PIXEL(ow + 2, a2, a0, a1, b2, b0, b1, c2, c0, c1)
            }
            for (; ow < W; ++ow)
            {
                ODL_STEM_PIXEL(ow, a0, a1, a2, b0, b1, b2, c0, c1, c2)
                a0 = a1, a1 = a2, b0 = b1, b1 = b2, c0 = c1, c1 = c2;
            }
#undef ODL_STEM_PIXEL
        }
        ODL_STEM_STAMP(3);
        // ---- bias gradient: channel oc of the NCHW reading is the block's floats oc*P .. oc*P + P - 1 — the sums of its
        // 16-byte pieces where the pieces respect the channels, else float by float out of the gy2d rows
        // (for this sum alone the thread stands for channel t / G and takes every G-th piece or float from its t % G-th on,
        // so that neighbouring lanes read neighbouring words)
        if (quadsums)
            for (int q = t % G; q < P / 4; q += G)
                accb += ps[(t / G) * (P / 4) + q];
        else
            for (int q = t % G; q < P; q += G)
            {
                const int e = (t / G) * P + q;
                accb += gs[(e / OC) * LDG + e % OC];
            }
        __syncthreads();  // the pieces' sums have been read: their space takes the products now
        ODL_STEM_STAMP(4);
        // ---- the nine (sum over oc) products of every output pixel
        if (g.gx)
        {
            for (int p = t; p < P; p += kT)
            {
                float c[9];
#pragma unroll
                for (int k = 0; k < 9; ++k)
                    c[k] = 0.f;
                const float *row = gs + p * LDG;
#pragma unroll 4
                for (int o = 0; o < OC; ++o)
                {
                    const float gv = row[o];
#pragma unroll
                    for (int k = 0; k < 9; ++k)
                        c[k] = fmaf(gv, wf[o * 9 + k], c[k]);
                }
#pragma unroll
                for (int k = 0; k < 9; ++k)
                    gc[p * 9 + k] = c[k];
            }
            __syncthreads();
            ODL_STEM_STAMP(5);
            // ---- and their gather per input pixel: tap (kh, kw) of output pixel (ih - kh + 1, iw - kw + 1)
            for (int i = t; i < P; i += kT)
            {
                const int ih = i / W, iw = i - ih * W;
                float s = 0.f;
#pragma unroll
                for (int kh = 0; kh < 3; ++kh)
                {
                    const int oh = ih - kh + 1;
                    if (oh < 0 || oh >= H)
                        continue;
#pragma unroll
                    for (int kw = 0; kw < 3; ++kw)
                    {
                        const int ow = iw - kw + 1;
                        if (ow >= 0 && ow < W)
                            s += gc[(oh * W + ow) * 9 + kh * 3 + kw];
                    }
                }
                g.gx[(int64_t)n * P + i] = s;
            }
        }
    }

    // ---- the groups' sums, added in group order: one partial per workgroup
    ODL_STEM_STAMP(6);
    __syncthreads();
    float *red = gs;                 // [G][OC*9] the groups' filter sums
    float *redb = red + G * OC * 9;  // [OC][G] the channels' shares of the bias sum
#pragma unroll
    for (int k = 0; k < 9; ++k)
        red[grp * (OC * 9) + oc * 9 + k] = acc[k];
    redb[t] = accb;  // (channel t / G, its t % G-th share)
    __syncthreads();
    for (int e = t; e < OC * 10; e += kT)
    {
        const float *from = e < OC * 9 ? red + e : redb + (e - OC * 9) * G;
        const int step = e < OC * 9 ? OC * 9 : 1;
        float s = from[0];
        for (int q = 1; q < G; ++q)
            s += from[q * step];
        g.part[(int64_t)blockIdx.x * (OC * 10) + e] = s;
    }
    ODL_STEM_STAMP(7);
}

// gw[e] / gb[e - OC*9] = sum over the workgroups' partials in workgroup order. 64 elements x 16 groups of partials per
// workgroup: a wave reads 64 neighbouring floats of one partial (whole lines), group q adds partials q, q + 16, ...,
// and the groups' sums are added in group order — the same order on every run.
__global__ __launch_bounds__(1024) void conv_stem_fold_kernel(const float *__restrict__ part, int nparts, int OC, float *gw, float *gb)
{
    __shared__ float sums[16][64];
    const int E = OC * 10, lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int e = blockIdx.x * 64 + lane;
    float s = 0.f;
    if (e < E)
    {
#pragma unroll 4
        for (int p = grp; p < nparts; p += 16)
            s += part[(int64_t)p * E + e];
    }
    sums[grp][lane] = s;
    __syncthreads();
    if (grp == 0 && e < E)
    {
        float v = sums[0][lane];
#pragma unroll
        for (int q = 1; q < 16; ++q)
            v += sums[q][lane];
        if (e < OC * 9)
        {
            if (gw)
                gw[e] = v;
        }
        else if (gb)
            gb[e - OC * 9] = v;
    }
}

size_t lds_bytes(int64_t OC, int64_t H, int64_t W)
{
    const size_t image = (size_t)(H * W * (OC + 1) + (H + 2) * (W + 2) + H * W * 9) * sizeof(float);
    const size_t groups = (size_t)kT * 10 * sizeof(float);  // the groups' sums at the end: [kT / OC][OC * 9] and [OC][kT / OC]
    return image > groups ? image : groups;
}

int workgroups(int64_t N)
{
    const int cus = odl::device_cus();
    return (int)(N < cus ? N : cus);
}

template <int OC>
hipError_t allow_lds_of()
{
    static const hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(&conv_stem_backward_kernel<OC>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    return rc;
}
}  // namespace

namespace odl
{
bool conv_stem_backward_ok(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW,
                           int PH, int PW)
{
    if (!(C == 1 && KH == 3 && KW == 3 && SH == 1 && SW == 1 && PH == 1 && PW == 1))
        return false;
    if (!(OC == 8 || OC == 16 || OC == 32) || N < 1 || H < 1 || W < 1 ||
        (reinterpret_cast<uintptr_t>(gy) & 15) != 0)
        return false;
    // an image's gradient block, input and per-pixel products in LDS; 32-bit offsets inside an image
    return lds_bytes(OC, H, W) <= 150 * 1024 && N * OC * H * W < (1ll << 40);
}

size_t conv_stem_backward_workspace(int64_t N, int64_t OC)
{
    return (size_t)workgroups(N) * (size_t)(OC * 10) * sizeof(float);
}

// gx, gw, gb may each be null
int conv_stem_backward(const float *gy, const float *x, const float *w, float *gx, float *gw, float *gb, int64_t N, int64_t H,
                       int64_t W, int64_t OC, void *workspace, size_t workspace_bytes, hipStream_t st)
{
    const size_t need = conv_stem_backward_workspace(N, OC);
    if (!workspace || workspace_bytes < need)
        return fail(ODL_ERR_INVALID_ARG, "conv2d_backward: needs a workspace of %zu bytes, got %zu", need, workspace_bytes);
    StemGeom g{gy, x, w, gx, static_cast<float *>(workspace), (int)N, (int)H, (int)W, (int)(H * W)};
    const int nb = workgroups(N);
    const size_t lds = lds_bytes(OC, H, W);
    if (OC == 8)
    {
        ODL_HIP_CHECK(allow_lds_of<8>());
        hipLaunchKernelGGL(conv_stem_backward_kernel<8>, dim3(nb), dim3(kT), lds, st, g, w);
    }
    else if (OC == 16)
    {
        ODL_HIP_CHECK(allow_lds_of<16>());
        hipLaunchKernelGGL(conv_stem_backward_kernel<16>, dim3(nb), dim3(kT), lds, st, g, w);
    }
    else
    {
        ODL_HIP_CHECK(allow_lds_of<32>());
        hipLaunchKernelGGL(conv_stem_backward_kernel<32>, dim3(nb), dim3(kT), lds, st, g, w);
    }
    ODL_LAUNCH_CHECK();
    if (gw || gb)
    {
        hipLaunchKernelGGL(conv_stem_fold_kernel, dim3((unsigned)ceil_div(OC * 10, 64)), dim3(1024), 0, st, g.part, nb, (int)OC, gw, gb);
        ODL_LAUNCH_CHECK();
    }
    return ODL_OK;
}
}  // namespace odl
