// Convolution forward for small problems (a detector's layers at batch 1-8: a few hundred MFLOP, outputs of a few
// hundred KB), where a tiled GEMM spends its time in launch, prologue and a K-slice reduction rather than in arithmetic.
//   y[n, oc, oh, ow] = act(b[oc] + sum_{c,kh,kw} x[n, c, oh*s-p+kh, ow*s-p+kw] * W[oc, c, kh, kw]) (+ r[n, oc, oh, ow])
// the reference's forward (src/mat/origin/cpu/nn/conv2d.cpp:230-300 through im2col + matmul; the detector's runner calls it
// per node, src/pnnx/pnnx_graph.cpp:286-528, then its SiLU / add / cat nodes one by one).
//
// One wave owns a 32 (output channels) x 32 (output pixels) tile on v_mfma_f32_32x32x2_f32 and reads its operands
// straight from global memory (the whole layer lives in L2): per step a lane loads four consecutive channels of one
// filter row (16 bytes) and the four matching input values of its pixel, which feed four MFMAs. The filter is read
// from a copy laid out for exactly this access — per (tile of 32 output channels, tap, group of 8 channels) one
// contiguous 1 KB block [lane half][row][4 channels], so a wave's load is eight whole cache lines — made once per
// set of weights (or into the workspace on every call for a caller that does not keep it). No LDS staging and no
// barrier in the K loop. The waves of a workgroup are `pixel tiles` x `K shares`: a long K (3x3 over 128 channels)
// is cut into shares of whole channel groups, one wave each, summed through LDS in share order in the epilogue,
// which also adds the bias, applies the activation, adds a residual tensor and stores NCHW. Input, output and
// residual each carry their own distance between images, so any of them can be a channel slice of a wider tensor
// (the destination of a concatenation).
#include "odl_common.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

namespace
{
struct DirectArgs
{
    const float *x, *w, *bias, *res;
    float *y, *y2;               // filters [0, split) go to y, filters [split, OC) to y2 (two convolutions run as one)
    int64_t x_bs, y_bs, y2_bs, res_bs;  // floats from one image to the next
    int split;
    int C, H, W, OC, OH, OW, KH, KW, S, P;
    int M;             // N * OH * OW output pixels
    int act;           // 0 none, 1 relu, 2 silu
    int KS, WP;        // K shares and pixel tiles of a workgroup (KS * WP waves)
    int chunks;        // channel groups of eight per K share
    int octiles;
    odl::FastDiv d_ohw, d_ow, d_chunks, d_kw;
    // A detect stage (the DET kernels only): the filters are [anchor][classes + 5]; every output goes through the sigmoid
    // and the box decoding and is stored to rows[n][anchor * OH * OW + pixel][channel] instead of y.
    const float *det_grid, *det_anchor;
    float *det_rows;
    int64_t det_grid_elems, det_anchor_elems, det_rows_bs;
    float det_stride;
    int det_CI, det_aH, det_aW;
    odl::FastDiv d_ci;
};

#ifdef ODL_DIRECT_DBG
__device__ unsigned long long g_direct_dbg[4096 * 8];
#define ODL_DIRECT_STAMP(i) do { if (threadIdx.x == 0 && blockIdx.x < 4096) g_direct_dbg[blockIdx.x * 8 + (i)] = wall_clock64(); } while (0)
#else
#define ODL_DIRECT_STAMP(i) do { } while (0)
#endif

constexpr int kPitch = 33;    // floats per row of a partial tile in LDS

// wd[((tile * KHW + tap) * groups + grp) * 256 + (half * 32 + row) * 4 + j] = w[tile*32 + row][grp*8 + half*4 + j][tap]
// (rows past OC are zero)
__global__ void pack_direct_kernel(const float *__restrict__ w, float *__restrict__ wd, int C, int OC, int KHW, int64_t total)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total)
        return;
    const int j = (int)(t & 3), row = (int)((t >> 2) & 31), half = (int)((t >> 7) & 1);
    int64_t blk = t >> 8;
    const int groups = C / 8;
    const int grp = (int)(blk % groups);
    blk /= groups;
    const int tap = (int)(blk % KHW), tile = (int)(blk / KHW);
    const int oc = tile * 32 + row, c = grp * 8 + half * 4 + j;
    wd[t] = oc < OC ? w[((int64_t)oc * C + c) * KHW + tap] : 0.f;
}

// The sums of the workgroup's outputs over the K shares, then bias, activation, residual, store: E outputs per thread
// (32 consecutive threads along the pixels of one output channel). Straight-line code: the residual loads first, the
// stores last, nothing that waits for a store.
template <int E, bool RES>
__device__ __forceinline__ void direct_epilogue(const DirectArgs &g, const float *partial, const float *bias_s, int m_base,
                                                int oc0, int OHW)
{
    const int nthreads = 64 * g.KS * g.WP;
    int64_t off[E];
    float res[E], v[E];
    bool ok[E], second[E];
#pragma unroll
    for (int i = 0; i < E; ++i)
    {
        const int e = threadIdx.x + i * nthreads;
        const int tp = e >> 10, rr = (e >> 5) & 31, col = e & 31;
        const int mm = m_base + tp * 32 + col, oc = oc0 + rr;
        ok[i] = mm < g.M && oc < g.OC;
        const unsigned mc = ok[i] ? (unsigned)mm : 0u;
        const unsigned nn = odl::fastdiv(mc, g.d_ohw), px = mc - nn * (unsigned)OHW;
        const int64_t o = (int64_t)(ok[i] ? oc : 0) * OHW + px;
        second[i] = oc >= g.split;
        off[i] = second[i] ? (int64_t)nn * g.y2_bs + o - (int64_t)g.split * OHW : (int64_t)nn * g.y_bs + o;
        if (RES)
            res[i] = g.res[(int64_t)nn * g.res_bs + o];
    }
#pragma unroll
    for (int i = 0; i < E; ++i)
    {
        const int e = threadIdx.x + i * nthreads;
        const int tp = e >> 10, rr = (e >> 5) & 31, col = e & 31;
        const float *src = partial + ((size_t)tp * g.KS * 32 + rr) * kPitch + col;
        float a = src[0];
        for (int s = 1; s < g.KS; ++s)
            a += src[(size_t)s * 32 * kPitch];
        v[i] = odl::apply_act(a + bias_s[rr], g.act);
        if (RES)
            v[i] = res[i] + v[i];
    }
#pragma unroll
    for (int i = 0; i < E; ++i)
        if (ok[i])
            (second[i] ? g.y2 : g.y)[off[i]] = v[i];
}

// The same sums for a detect stage: bias, then the steps of the decoding kernel (sigmoid as -x, exp, 1 + ., 1 / .; boxes
// (2s + grid) * stride and (2s)^2 * anchor) on every output, stored as rows [pixel][channel]: 32 consecutive threads
// along the channels of one pixel, so a store covers consecutive floats of a row.
template <int E>
__device__ __forceinline__ void direct_epilogue_detect(const DirectArgs &g, const float *partial, const float *bias_s, int m_base,
                                                       int oc0, int OHW)
{
    // sixteen waves: a thread keeps its channel and its pixel column for all of its E outputs, one per pixel tile
    const int col = (int)(threadIdx.x >> 5), rr = (int)(threadIdx.x & 31);
    const int oc = oc0 + rr;
    if (oc >= g.OC)
        return;
    const int anc = (int)odl::fastdiv((unsigned)oc, g.d_ci), c = oc - anc * g.det_CI;
    const float bias = bias_s[rr];
    const int sh_ = (g.det_aH > 0 && g.OH > g.det_aH) ? g.OH / g.det_aH : 1;
    const int sw_ = (g.det_aW > 0 && g.OW > g.det_aW) ? g.OW / g.det_aW : 1;
    float *rows = g.det_rows + (int64_t)anc * OHW * g.det_CI + c;
#pragma unroll
    for (int i = 0; i < E; ++i)
    {
        const int mm = m_base + i * 32 + col;
        if (mm < g.M)
        {
            const float *src = partial + ((size_t)i * g.KS * 32 + rr) * kPitch + col;
            float a = src[0];
            for (int s = 1; s < g.KS; ++s)
                a += src[(size_t)s * 32 * kPitch];
            float v = 1.0f / (1.0f + expf(-(a + bias)));
            const unsigned nn = odl::fastdiv((unsigned)mm, g.d_ohw), px = (unsigned)mm - nn * (unsigned)OHW;
            if (c < 4)
            {
                const int h = (int)odl::fastdiv(px, g.d_ow), w = (int)px - h * g.OW;
                const float t = v * 2.0f;
                if (c < 2)
                {
                    const int64_t gi = ((int64_t)anc * OHW + px) * 2 + c;
                    v = (t + (gi < g.det_grid_elems ? g.det_grid[gi] : 0.0f)) * g.det_stride;
                }
                else
                {
                    int ah = h / sh_, aw = w / sw_;
                    ah = ah < g.det_aH - 1 ? ah : g.det_aH - 1;
                    aw = aw < g.det_aW - 1 ? aw : g.det_aW - 1;
                    const int64_t ai = ((int64_t)anc * g.det_aH * g.det_aW + (int64_t)ah * g.det_aW + aw) * 2 + (c - 2);
                    v = (t * t) * (ai < g.det_anchor_elems ? g.det_anchor[ai] : 1.0f);
                }
            }
            rows[(int64_t)nn * g.det_rows_bs + (int64_t)px * g.det_CI] = v;
        }
    }
}

// What follows the K loop: the tile's sums (this wave's share of K in acc) to their places in y.
template <bool RES, bool DET = false>
__device__ __forceinline__ void direct_finish(const DirectArgs &g, const f32x16 &acc, float bias_v, float *bias_s, float *partial,
                                              int wv, int pt, int l32, int half, int m_base, int oc0, int OHW, unsigned n, unsigned r)
{
    ODL_DIRECT_STAMP(3);
    if (threadIdx.x < 32)
        bias_s[threadIdx.x] = bias_v;
    if (DET)
    {
        // (through LDS whatever the number of K shares: the rows are written along the channels, the lanes hold pixels)
        float *mine = partial + (size_t)wv * 32 * kPitch;
#pragma unroll
        for (int q = 0; q < 16; ++q)
            mine[(8 * (q / 4) + 4 * half + (q % 4)) * kPitch + l32] = acc[q];
        __syncthreads();
        if (g.KS == 1)
            direct_epilogue_detect<16>(g, partial, bias_s, m_base, oc0, OHW);
        else if (g.KS == 2)
            direct_epilogue_detect<8>(g, partial, bias_s, m_base, oc0, OHW);
        else if (g.KS == 4)
            direct_epilogue_detect<4>(g, partial, bias_s, m_base, oc0, OHW);
        else if (g.KS == 8)
            direct_epilogue_detect<2>(g, partial, bias_s, m_base, oc0, OHW);
        else
            direct_epilogue_detect<1>(g, partial, bias_s, m_base, oc0, OHW);
        return;
    }
    if (g.KS == 1)
    {
        // accumulator register q of a lane: row 8*(q/4) + 4*half + q%4, column l32
        __syncthreads();  // the bias rows
        const int mm = m_base + pt * 32 + l32;
        if (mm < g.M)
        {
            const int64_t pix = (int64_t)r;
            float *yp = g.y + (int64_t)n * g.y_bs + pix;
            float *yp2 = g.y2 + (int64_t)n * g.y2_bs + pix - (int64_t)g.split * OHW;
            float rv[16];
            if (RES)
            {
                // (a row past OC reads the last row's residual and is not stored)
                const float *rp = g.res + (int64_t)n * g.res_bs + pix;
#pragma unroll
                for (int q = 0; q < 16; ++q)
                {
                    const int oc = oc0 + 8 * (q / 4) + 4 * half + (q % 4);
                    rv[q] = rp[(int64_t)(oc < g.OC ? oc : g.OC - 1) * OHW];
                }
            }
#pragma unroll
            for (int q = 0; q < 16; ++q)
            {
                const int rr = 8 * (q / 4) + 4 * half + (q % 4);
                float v = odl::apply_act(acc[q] + bias_s[rr], g.act);
                if (RES)
                    v = rv[q] + v;
                if (oc0 + rr < g.OC)
                    (oc0 + rr >= g.split ? yp2 : yp)[(int64_t)(oc0 + rr) * OHW] = v;
            }
        }
        ODL_DIRECT_STAMP(5);
        return;
    }
    float *mine = partial + (size_t)wv * 32 * kPitch;
#pragma unroll
    for (int q = 0; q < 16; ++q)
        mine[(8 * (q / 4) + 4 * half + (q % 4)) * kPitch + l32] = acc[q];
    __syncthreads();
    ODL_DIRECT_STAMP(4);
    // 1024 outputs a pixel tile over 64 * KS * WP threads: 16 / KS outputs a thread
    if (g.KS == 2)
        direct_epilogue<8, RES>(g, partial, bias_s, m_base, oc0, OHW);
    else if (g.KS == 4)
        direct_epilogue<4, RES>(g, partial, bias_s, m_base, oc0, OHW);
    else if (g.KS == 8)
        direct_epilogue<2, RES>(g, partial, bias_s, m_base, oc0, OHW);
    else
        direct_epilogue<1, RES>(g, partial, bias_s, m_base, oc0, OHW);
    ODL_DIRECT_STAMP(5);
}

// kDepth: operand groups in flight per wave. Every load instruction costs the compute unit's one address unit 16
// clocks whether or not its data is used, so the depth divides the group count (3 for 3x3 windows, 4 otherwise) and no
// group is loaded twice.
template <int kDepth, bool RES, bool DET = false>
__device__ __forceinline__ void conv_direct_tile(const DirectArgs &g, const unsigned bid)
{
    extern __shared__ float lds[];  // bias[32], then partial[WP * KS][32][kPitch] when KS > 1
    ODL_DIRECT_STAMP(0);
    float *bias_s = lds, *partial = lds + 32;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int pt = wv / g.KS, ks = wv - pt * g.KS;
    const int oct = (int)(bid % (unsigned)g.octiles);
    const int m_base = (int)(bid / (unsigned)g.octiles) * 32 * g.WP;
    const int oc0 = oct * 32;
    const int HW = g.H * g.W, OHW = g.OH * g.OW, KHW = g.KH * g.KW;
    // the bias rows of the tile: asked for now, put into LDS after the K loop (no wait here)
    const float bias_v = (threadIdx.x < 32 && g.bias && oc0 + (int)threadIdx.x < g.OC) ? g.bias[oc0 + threadIdx.x] : 0.f;
    // a lane past the last pixel reads the last pixel's operands; its results are never stored
    int m = m_base + pt * 32 + l32;
    m = m < g.M ? m : g.M - 1;
    const unsigned n = odl::fastdiv((unsigned)m, g.d_ohw), r = (unsigned)m - n * (unsigned)OHW;
    const int oh = (int)odl::fastdiv(r, g.d_ow), ow = (int)r - oh * g.OW;
    const int ih0 = oh * g.S - g.P, iw0 = ow * g.S - g.P;
    const int groups = g.C >> 3;
    const int grp0 = ks * g.chunks;
    const float *xb = g.x + (int64_t)n * g.x_bs + (int64_t)(grp0 * 8 + 4 * half) * HW;
    // this wave's first block of the filter copy; consecutive groups and then consecutive taps follow each other
    const float *wb = g.w + ((int64_t)oct * KHW * groups + grp0) * 256 + lane * 4;

    const int total = KHW * g.chunks;
    ODL_DIRECT_STAMP(1);
    // Operand groups are numbered tap-major, (tap, channel group); group q is loaded kDepth groups ahead of its use.
    // Inside the K loop the loads are unconditional and their addresses come from q by arithmetic alone, so the loop
    // body is one basic block and the loads of later groups stay in flight across the MFMAs of earlier ones; a q
    // past the end (only when kDepth does not divide the group count) loads the last group again, unused.
    f32x4 fa[kDepth], fb[kDepth];
    bool fok[kDepth];  // a tap in the padding: its group is replaced by zeros when it is used
    auto load = [&](int slot, int q) {
        q = q < total ? q : total - 1;
        const int tap = (int)odl::fastdiv((unsigned)q, g.d_chunks), cc = q - tap * g.chunks;
        const int kh = (int)odl::fastdiv((unsigned)tap, g.d_kw), kw = tap - kh * g.KW;
        const int ih = ih0 + kh, iw = iw0 + kw;
        fok[slot] = (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W;
        // (the padding tap reads the pixel's nearest valid neighbour)
        const int ihc = ih < 0 ? 0 : (ih >= g.H ? g.H - 1 : ih), iwc = iw < 0 ? 0 : (iw >= g.W ? g.W - 1 : iw);
        const float *px = xb + (ihc * g.W + iwc) + (int64_t)cc * 8 * HW;
        fa[slot] = *reinterpret_cast<const f32x4 *>(wb + ((int64_t)tap * groups + cc) * 256);
        fb[slot] = f32x4{px[0], px[HW], px[2 * HW], px[3 * HW]};
    };
    f32x16 acc = {0};
    auto use = [&](int slot) {
        const f32x4 a = fa[slot], b = fok[slot] ? fb[slot] : f32x4{0.f, 0.f, 0.f, 0.f};
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, b.w, acc, 0, 0, 0);
    };
#pragma unroll
    for (int d = 0; d < kDepth; ++d)
        if (d < total)
            load(d, d);
    int it = 0;
    for (; it + kDepth < total; it += kDepth)
    {
#pragma unroll
        for (int d = 0; d < kDepth; ++d)
        {
            use(d);
            load(d, it + d + kDepth);
            __builtin_amdgcn_sched_barrier(0);  // keep each group's loads where they are written: right behind its use
        }
    }
    ODL_DIRECT_STAMP(2);
    const int rem = total - it;  // groups left (1 .. kDepth), already loaded into slots 0 .. rem-1
#pragma unroll
    for (int d = 0; d < kDepth; ++d)
        if (d < rem)
            use(d);
    direct_finish<RES, DET>(g, acc, bias_v, bias_s, partial, wv, pt, l32, half, m_base, oc0, OHW, n, r);
}

template <int kDepth, bool RES>
__global__ __launch_bounds__(1024) void conv_direct_kernel(DirectArgs g)
{
    conv_direct_tile<kDepth, RES>(g, blockIdx.x);
}

// Several convolutions with 1x1 windows in one launch (the stage convolutions of a detect head: small, independent, each
// a launch's latency long on its own): workgroups [first[s], first[s + 1]) are member s's, each doing what
// conv_direct_kernel's workgroup of the same number does for that member alone. Every member is cut into sixteen waves
// a workgroup, its K shares as plan_direct gives them for the member alone, so its sums are formed in the same order.
constexpr int kGroupMax = 4;
struct DirectGroup
{
    DirectArgs g[kGroupMax];
    unsigned first[kGroupMax + 1];
};

template <bool DET>
__global__ __launch_bounds__(1024) void conv_direct_group_kernel(DirectGroup d, int count)
{
    int s = 0;
    for (int j = 1; j < count; ++j)
        s = blockIdx.x >= d.first[j] ? j : s;
    conv_direct_tile<4, false, DET>(d.g[s], blockIdx.x - d.first[s]);
}

// 3x3 windows with padding 1 (stride 1 or 2, rows of three pixels or more): the three taps of a window row are three
// consecutive input floats, so a lane fetches them with one 12-byte load and they feed three MFMAs, whose filter
// values — w[row][c][kh][0..2] — are one 16-byte load from a copy laid out [tile of 32 filters][channel pair][kh] x
// [lane half][row][kw, one pad]. A lane half is one channel of the pair. Two load instructions per three MFMAs instead
// of five per four: the compute unit's address unit, which every load occupies for 16 clocks, stops being the
// limit. A window that hangs over the left or right edge loads the three floats next to it and shifts them.
constexpr int kDepth3 = 6;
typedef float f32x3 __attribute__((ext_vector_type(3)));

template <bool RES>
__global__ __launch_bounds__(1024) void conv_direct3_kernel(DirectArgs g)
{
    extern __shared__ float lds[];  // bias[32], then partial[WP * KS][32][kPitch] when KS > 1
    float *bias_s = lds, *partial = lds + 32;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int pt = wv / g.KS, ks = wv - pt * g.KS;
    const unsigned bid = blockIdx.x;
    const int oct = (int)(bid % (unsigned)g.octiles);
    const int m_base = (int)(bid / (unsigned)g.octiles) * 32 * g.WP;
    const int oc0 = oct * 32;
    const int HW = g.H * g.W, OHW = g.OH * g.OW;
    const float bias_v = (threadIdx.x < 32 && g.bias && oc0 + (int)threadIdx.x < g.OC) ? g.bias[oc0 + threadIdx.x] : 0.f;
    int m = m_base + pt * 32 + l32;
    m = m < g.M ? m : g.M - 1;
    const unsigned n = odl::fastdiv((unsigned)m, g.d_ohw), r = (unsigned)m - n * (unsigned)OHW;
    const int oh = (int)odl::fastdiv(r, g.d_ow), ow = (int)r - oh * g.OW;
    const int ih0 = oh * g.S - 1, iw0 = ow * g.S - 1;
    // the window's three columns iw0 .. iw0+2: read from iwb .. iwb+2, which lie inside the row
    const int shift = iw0 < 0 ? 1 : (iw0 + 2 >= g.W ? 2 : 0);
    const int iwb = shift == 1 ? 0 : (shift == 2 ? g.W - 3 : iw0);
    const int pairs = g.C >> 1;                 // channel pairs; this wave's are [pair0, pair0 + 4 * chunks)
    const int pair0 = ks * g.chunks * 4;
    const float *xb = g.x + (int64_t)n * g.x_bs + (int64_t)(2 * pair0 + half) * HW + iwb;
    const float *wb = g.w + ((int64_t)oct * pairs + pair0) * 768 + lane * 4;
    const int total = 12 * g.chunks;            // groups: (channel pair, window row)
    f32x4 fa[kDepth3];
    f32x3 fb[kDepth3];
    bool fok[kDepth3];
    auto load = [&](int slot, int q) {
        q = q < total ? q : total - 1;
        const int pr = (int)(((unsigned)q * 43691u) >> 17), kh = q - 3 * pr;  // q / 3 for q < 98304
        const int ih = ih0 + kh;
        fok[slot] = (unsigned)ih < (unsigned)g.H;
        const int ihc = ih < 0 ? 0 : (ih >= g.H ? g.H - 1 : ih);
        const float *px = xb + (int64_t)pr * 2 * HW + ihc * g.W;
        fa[slot] = *reinterpret_cast<const f32x4 *>(wb + (int64_t)q * 256);
        fb[slot] = f32x3{px[0], px[1], px[2]};
    };
    f32x16 acc = {0};
    auto use = [&](int slot) {
        const f32x4 a = fa[slot];
        const f32x3 v = fb[slot];
        const bool ok = fok[slot];
        // the window's columns out of the three floats read (a column in the padding is zero)
        const float b0 = (ok && shift != 1) ? (shift == 2 ? v.y : v.x) : 0.f;
        const float b1 = ok ? (shift == 1 ? v.x : (shift == 2 ? v.z : v.y)) : 0.f;
        const float b2 = (ok && shift != 2) ? (shift == 1 ? v.y : v.z) : 0.f;
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b1, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b2, acc, 0, 0, 0);
    };
#pragma unroll
    for (int d = 0; d < kDepth3; ++d)
        load(d, d);  // (total is a multiple of 12)
    int it = 0;
    for (; it + kDepth3 < total; it += kDepth3)
    {
#pragma unroll
        for (int d = 0; d < kDepth3; ++d)
        {
            use(d);
            load(d, it + d + kDepth3);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int d = 0; d < kDepth3; ++d)
        use(d);
    direct_finish<RES>(g, acc, bias_v, bias_s, partial, wv, pt, l32, half, m_base, oc0, OHW, n, r);
}

// wd[(((tile * pairs + pair) * 3 + kh) * 64 + half * 32 + row) * 4 + kw] = w[tile*32 + row][2*pair + half][kh][kw], kw < 3
// (the fourth float of a lane and rows past OC are zero)
__global__ void pack_direct3_kernel(const float *__restrict__ w, float *__restrict__ wd, int C, int OC, int64_t total)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total)
        return;
    const int kw = (int)(t & 3), row = (int)((t >> 2) & 31), half = (int)((t >> 7) & 1);
    int64_t blk = t >> 8;
    const int kh = (int)(blk % 3);
    blk /= 3;
    const int pairs = C / 2;
    const int pair = (int)(blk % pairs), tile = (int)(blk / pairs);
    const int oc = tile * 32 + row, c = 2 * pair + half;
    wd[t] = (oc < OC && kw < 3) ? w[(((int64_t)oc * C + c) * 3 + kh) * 3 + kw] : 0.f;
}

// the 3x3 kernel above takes windows of 3x3 with padding 1 over rows of at least three pixels
inline bool direct_rows3(int KH, int KW, int P, int64_t W)
{
    return KH == 3 && KW == 3 && P == 1 && W >= 3;
}

int g_force_ks = 0, g_force_wp = 0;  // measurement overrides (0: the rule below)

// K shares and pixel tiles per workgroup: enough waves to give every SIMD of the chip one or two, shares of at least
// one channel group, at most sixteen waves a workgroup
void plan_direct(int64_t M, int64_t OC, int64_t C, int KHW, int &KS, int &WP, int &chunks)
{
    const int64_t tiles = odl::ceil_div(M, 32) * odl::ceil_div(OC, 32);
    const int64_t want = (int64_t)odl::device_cus() * 4 * 2;
    const int groups = (int)(C / 8);
    int ks = 1;
    while (ks < 16 && tiles * ks < want && groups % (2 * ks) == 0 && (int64_t)(groups / (2 * ks)) * KHW >= 2)
        ks *= 2;
    if (g_force_ks > 0 && groups % g_force_ks == 0)
        ks = g_force_ks;
    int wp = ks >= 4 ? 1 : 4 / ks;
    if (g_force_wp > 0 && (ks == 1 || ks * g_force_wp <= 16) && (g_force_wp & (g_force_wp - 1)) == 0)
        wp = g_force_wp;
    while (wp > 1 && (int64_t)32 * (wp - 1) >= M)
        --wp;
    KS = ks, WP = wp, chunks = groups / ks;
}
}  // namespace

namespace odl
{
// Shapes this kernel takes: channels in groups of eight (a lane's four consecutive channels, two lane halves), a
// problem small enough that the tiled kernels' fixed costs dominate, 32-bit offsets within an image.
bool conv_direct_ok(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW,
                    int64_t OH, int64_t OW)
{
    if (C <= 0 || C % 8 != 0 || SH != SW || PH != PW || KH <= 0 || KW <= 0 || KH * KW > 49 || OC <= 0)
        return false;
    const int64_t M = N * OH * OW, K = C * KH * KW;
    if (M <= 0 || M >= (1ll << 30) || C * H * W >= (1ll << 30) || OC * OH * OW >= (1ll << 30) || OC * K >= (1ll << 30))
        return false;
    // (measured against the tiled kernels: ahead up to about 1.6 GFLOP, even with the filter copy made on every call)
    return 2 * M * K * OC <= (3ll << 29);
}

size_t conv_direct_packed_bytes(int64_t C, int64_t OC, int KH, int KW, int P, int64_t W)
{
    const int per_channel = direct_rows3(KH, KW, P, W) ? 12 : KH * KW;  // (window rows padded to four floats)
    return (size_t)(ceil_div(OC, 32) * 32 * C * per_channel) * sizeof(float);
}

int conv_direct_pack(const float *w, int64_t C, int64_t OC, int KH, int KW, int P, int64_t W, float *packed, hipStream_t st)
{
    const int64_t total = (int64_t)(conv_direct_packed_bytes(C, OC, KH, KW, P, W) / sizeof(float));
    ODL_REQUIRE(total < (1ll << 31) && C % 8 == 0, "conv2d: filter too large or channels not a multiple of 8");
    if (direct_rows3(KH, KW, P, W))
        hipLaunchKernelGGL(pack_direct3_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, st, w, packed, (int)C, (int)OC, total);
    else
        hipLaunchKernelGGL(pack_direct_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, st, w, packed, (int)C, (int)OC,
                           KH * KW, total);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

// x, y, residual: NCHW with x_bs / y_bs / res_bs floats from one image to the next (0: dense). packed: the filter as
// conv_direct_pack lays it out (16-byte aligned). y2 (optional): the outputs of filters [split, OC) go there instead.
int conv_direct(const float *x, int64_t x_bs, const float *packed, const float *b, const float *res, int64_t res_bs, float *y,
                int64_t y_bs, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int S, int P, int64_t OH,
                int64_t OW, int act, hipStream_t st, float *y2, int64_t y2_bs, int64_t split)
{
    ODL_REQUIRE(packed != nullptr && reinterpret_cast<uintptr_t>(packed) % 16 == 0, "conv2d: the filter copy must be 16-byte aligned");
    DirectArgs g{};
    g.x = x, g.w = packed, g.bias = b, g.res = res, g.y = y;
    // two convolutions run as one: filters [0, split) fill y, the rest y2 (otherwise split = OC and y2 is never chosen)
    const int64_t first = y2 ? split : OC;
    g.y2 = y2 ? y2 : y, g.split = (int)first;
    g.x_bs = x_bs ? x_bs : C * H * W, g.y_bs = y_bs ? y_bs : first * OH * OW, g.res_bs = res_bs ? res_bs : OC * OH * OW;
    g.y2_bs = y2_bs ? y2_bs : (OC - first) * OH * OW;
    g.C = (int)C, g.H = (int)H, g.W = (int)W, g.OC = (int)OC, g.OH = (int)OH, g.OW = (int)OW, g.KH = KH, g.KW = KW, g.S = S, g.P = P;
    g.M = (int)(N * OH * OW), g.act = act;
    // a pair is cut into K shares as its larger member alone would be: each member then sums in the order of its own call
    const int64_t oc_plan = y2 ? (first > OC - first ? first : OC - first) : OC;
    plan_direct(g.M, oc_plan, C, KH * KW, g.KS, g.WP, g.chunks);
    g.octiles = (int)ceil_div(OC, 32);
    g.d_ohw = make_fastdiv((unsigned)(OH * OW)), g.d_ow = make_fastdiv((unsigned)OW);
    g.d_chunks = make_fastdiv((unsigned)g.chunks), g.d_kw = make_fastdiv((unsigned)KW);
    const int64_t blocks = ceil_div(g.M, 32 * g.WP) * g.octiles;
    ODL_REQUIRE(blocks < (1ll << 31), "conv2d: too many tiles");
    const size_t lds = (32 + (g.KS > 1 ? (size_t)g.KS * g.WP * 32 * kPitch : 0)) * sizeof(float);
    const dim3 grid((unsigned)blocks), block(64 * g.KS * g.WP);
    if (direct_rows3(KH, KW, P, W) && res)
        hipLaunchKernelGGL((conv_direct3_kernel<true>), grid, block, lds, st, g);
    else if (direct_rows3(KH, KW, P, W))
        hipLaunchKernelGGL((conv_direct3_kernel<false>), grid, block, lds, st, g);
    else if ((KH * KW) % 3 == 0 && res)
        hipLaunchKernelGGL((conv_direct_kernel<3, true>), grid, block, lds, st, g);
    else if ((KH * KW) % 3 == 0)
        hipLaunchKernelGGL((conv_direct_kernel<3, false>), grid, block, lds, st, g);
    else if (res)
        hipLaunchKernelGGL((conv_direct_kernel<4, true>), grid, block, lds, st, g);
    else
        hipLaunchKernelGGL((conv_direct_kernel<4, false>), grid, block, lds, st, g);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}
}  // namespace odl

namespace odl
{
int conv_direct_group(int count, const float *const *x, const int64_t *x_bs, const float *const *packed, const float *const *b,
                      float *const *y, const int64_t *y_bs, int64_t N, const int64_t *C, const int64_t *H, const int64_t *W,
                      const int64_t *OC, int act, hipStream_t st, const DetectRows *det)
{
    ODL_REQUIRE(count >= 1 && count <= kGroupMax, "conv2d_fused_group: 1 to %d members, got %d", kGroupMax, count);
    DirectGroup d{};
    int64_t blocks = 0;
    for (int s = 0; s < count; ++s)
    {
        ODL_REQUIRE(packed[s] != nullptr && reinterpret_cast<uintptr_t>(packed[s]) % 16 == 0,
                    "conv2d: the filter copy must be 16-byte aligned");
        DirectArgs &g = d.g[s];
        g.x = x[s], g.w = packed[s], g.bias = b ? b[s] : nullptr, g.res = nullptr, g.split = (int)OC[s];
        g.y = det ? nullptr : y[s], g.y2 = g.y;
        g.x_bs = x_bs[s] ? x_bs[s] : C[s] * H[s] * W[s], g.y_bs = (!det && y_bs[s]) ? y_bs[s] : OC[s] * H[s] * W[s];
        if (det)
        {
            g.det_grid = det[s].grid, g.det_anchor = det[s].anchor_grid, g.det_rows = det[s].rows;
            g.det_grid_elems = det[s].grid_elems, g.det_anchor_elems = det[s].anchor_elems, g.det_rows_bs = det[s].rows_image_stride;
            g.det_stride = det[s].stride, g.det_CI = det[s].CI, g.det_aH = det[s].anchor_H, g.det_aW = det[s].anchor_W;
            g.d_ci = make_fastdiv((unsigned)det[s].CI);
        }
        g.res_bs = g.y_bs, g.y2_bs = g.y_bs;
        g.C = (int)C[s], g.H = (int)H[s], g.W = (int)W[s], g.OC = (int)OC[s], g.OH = (int)H[s], g.OW = (int)W[s];
        g.KH = 1, g.KW = 1, g.S = 1, g.P = 0, g.M = (int)(N * H[s] * W[s]), g.act = act;
        int wp_alone;
        plan_direct(g.M, OC[s], C[s], 1, g.KS, wp_alone, g.chunks);
        g.WP = 16 / g.KS;  // (pixel tiles past the last pixel compute on the last pixel's operands and store nothing)
        g.octiles = (int)ceil_div(OC[s], 32);
        g.d_ohw = make_fastdiv((unsigned)(H[s] * W[s])), g.d_ow = make_fastdiv((unsigned)W[s]);
        g.d_chunks = make_fastdiv((unsigned)g.chunks), g.d_kw = make_fastdiv(1u);
        d.first[s] = (unsigned)blocks;
        blocks += ceil_div(g.M, 32 * g.WP) * g.octiles;
        ODL_REQUIRE(blocks < (1ll << 31), "conv2d: too many tiles");
    }
    for (int s = count; s <= kGroupMax; ++s)
        d.first[s] = (unsigned)blocks;
    const size_t lds = (32 + (size_t)16 * 32 * kPitch) * sizeof(float);
    if (det)
        hipLaunchKernelGGL(conv_direct_group_kernel<true>, dim3((unsigned)blocks), dim3(1024), lds, st, d, count);
    else
        hipLaunchKernelGGL(conv_direct_group_kernel<false>, dim3((unsigned)blocks), dim3(1024), lds, st, d, count);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}
}  // namespace odl

extern "C" int odl_hip_set_conv_direct_plan(int k_shares, int pixel_tiles)
{
    g_force_ks = k_shares, g_force_wp = pixel_tiles;
    return ODL_OK;
}
