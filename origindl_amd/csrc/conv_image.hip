// Weight and bias gradient of a 3x3 / stride 1 / padding 1 convolution over small images with few channels — the second
// layer of the reference's MNIST CNN (tests/example/mnist/conv_mnist.cpp: 32 -> 64 channels on 14 x 14) — with a whole
// image resident in LDS.
//
// gW[oc][c][kh][kw] = sum over m of gy2d[m][oc] * col[m][c*9 + kh*3 + kw] (src/mat/origin/cpu/conv/conv2d.cpp:546-560, gy2d
// being gy's NCHW buffer read as a row-major [N*OH*OW, OC] matrix exactly as it lies, line 548) is a product with a short
// output (OC x C*9) and a long sum (every pixel of every image). As a matrix product over gathered operands every element
// of col costs an address computation, a bounds check and a 4-byte load of its own, nine times per input float. Here one
// workgroup takes one image at a time: its gy block (P x OC floats, contiguous) and its input with a zero border
// (C x (H+2) x (W+2) floats) go to LDS once, and the 16x16x4 MFMA steps read both operands out of LDS by plain offsets —
// the column (c, kh, kw) is a constant offset per lane, the pixel a running one. A wave owns a 32 x 48 block of gW (two
// by three MFMA tiles) and keeps it in registers across the workgroup's images; each workgroup writes one partial gW, and
// a second launch adds the partials in workgroup order. The bias gradient (the NCHW reading of the same block,
// conv2d.cpp:566-580) is summed from the pieces as they are staged and travels in the same partials.
#include "conv_side.h"
#include "odl_common.h"

#include <map>
#include <mutex>
#include <tuple>

typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace
{
constexpr int kIT = 768;            // threads per workgroup: twelve waves, three per SIMD
constexpr int kWaves = kIT / 64;    // and at most that many 32 x 48 blocks of gW
constexpr int kBlockRows = 32, kBlockCols = 48;

struct ImageGeom
{
    const float *gy, *x;
    float *part;  // part[workgroup][OC*C*9 + OC]
    int N, C, H, W, OC, P, cols;
    int pr, pc, ldg;  // floats between the padded input's rows and channels and between the gy2d rows in LDS
    int blocks_c, blocks;
    int E;           // floats per partial
    int tile_pitch;  // floats between gW's rows when its blocks meet in LDS
    odl::FastDiv by_oc, by_p, by_w, by_cols;
};

// (time stamps of a workgroup's phases for a test harness that includes this file with ODL_IMAGE_DBG defined; nothing otherwise)
#ifdef ODL_IMAGE_DBG
__device__ unsigned long long g_image_dbg[256 * 16];
#define ODL_IMAGE_STAMP(i) do { if (threadIdx.x == 0 && blockIdx.x < 256) g_image_dbg[blockIdx.x * 16 + (i)] = wall_clock64(); } while (0)
#else
#define ODL_IMAGE_STAMP(i) do { } while (0)
#endif

__global__ __launch_bounds__(kIT) void conv_image_wgrad_kernel(const ImageGeom g)
{
    extern __shared__ float lds[];
    const int P = g.P, W = g.W, OC = g.OC, ldg = g.ldg;
    float *gs = lds;               // [P][ldg]
    float *xs = gs + P * ldg;      // [C][pc]: (H+2) rows of pr floats each, zero border
    float *ps = xs + g.C * g.pc;   // [OC*P/4] sums of the staged 16-byte pieces (the bias gradient reads them)
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int j = lane & 15, kq = lane >> 4;

    ODL_IMAGE_STAMP(0);

    // this wave's block of gW: rows rb*32 .., columns cb*48 ..; a lane's column of B in each of the three tiles
    const bool worker = wave < g.blocks;
    const int rb = worker ? wave / g.blocks_c : 0, cb = worker ? wave % g.blocks_c : 0;
    int colbase[3];
#pragma unroll
    for (int ct = 0; ct < 3; ++ct)
    {
        int col = cb * kBlockCols + ct * 16 + j;
        col = col < g.cols ? col : g.cols - 1;  // (columns past the end compute a copy that is not stored)
        const int c = col / 9, tap = col - c * 9, kh = tap / 3, kw = tap - kh * 3;
        colbase[ct] = c * g.pc + kh * g.pr + kw;
    }
    f32x4 acc[2][3];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int ct = 0; ct < 3; ++ct)
            acc[rt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    // the bias gradient: thread t stands for channel t / gb_share and takes every gb_share-th piece sum from its own on
    const int gb_share = kIT / OC, gb_ch = t / gb_share, gb_q = t - gb_ch * gb_share;
    float bacc = 0.f;

    for (int n = blockIdx.x; n < g.N; n += gridDim.x)
    {
        // ---- staging: the loads of the gy block's and the input's first pieces are in flight together (one trip to memory
        // for a 14 x 14 image with 64 and 32 channels), then the barrier after which LDS may be overwritten
        const float *blk = g.gy + (int64_t)n * OC * P, *xi = g.x + (int64_t)n * g.C * P;
        const int quads = OC * P / 4, xquads = g.C * P / 4;
        constexpr int U = 5, XU = 3;
        auto store_gy = [&](int e4, const f32x4 &v) {
            const unsigned e = 4u * (unsigned)e4, p = odl::fastdiv(e, g.by_oc), c0 = e - p * (unsigned)OC;
            *reinterpret_cast<f32x4 *>(gs + p * ldg + c0) = v;
            ps[e4] = (v[0] + v[1]) + (v[2] + v[3]);
        };
        // four floats of one channel of the input (P % 4 == 0), each to its place inside the border
        auto store_x = [&](int i4, const f32x4 &v) {
            const unsigned i = 4u * (unsigned)i4, c = odl::fastdiv(i, g.by_p), r = i - c * (unsigned)P;
            unsigned h = odl::fastdiv(r, g.by_w), w = r - h * (unsigned)W;
            float *d = xs + c * g.pc + g.pr + 1;
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                d[h * g.pr + w] = v[q];
                if (++w == (unsigned)W)
                    w = 0, ++h;
            }
        };
        {
            f32x4 v[U], xv[XU];
#pragma unroll
            for (int u = 0; u < U; ++u)
            {
                const int e4 = t + u * kIT;
                v[u] = *reinterpret_cast<const f32x4 *>(blk + 4 * (e4 < quads ? e4 : t));  // (quads >= kIT)
            }
#pragma unroll
            for (int u = 0; u < XU; ++u)
            {
                const int i4 = t + u * kIT;
                xv[u] = *reinterpret_cast<const f32x4 *>(xi + 4 * (i4 < xquads ? i4 : 0));
            }
            if (n == (int)blockIdx.x)  // the border is written once: the images overwrite the inside only
                for (int i = t; i < g.C * g.pc; i += kIT)
                    xs[i] = 0.f;
            __syncthreads();  // the previous image has been read (the border is in place)
            ODL_IMAGE_STAMP(1);
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (t + u * kIT < quads)
                    store_gy(t + u * kIT, v[u]);
#pragma unroll
            for (int u = 0; u < XU; ++u)
                if (t + u * kIT < xquads)
                    store_x(t + u * kIT, xv[u]);
        }
        for (int e0 = t + U * kIT; e0 < quads; e0 += U * kIT)  // (larger images: the rest)
        {
            f32x4 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u)
            {
                const int e4 = e0 + u * kIT;
                v[u] = *reinterpret_cast<const f32x4 *>(blk + 4 * (e4 < quads ? e4 : e0));
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (e0 + u * kIT < quads)
                    store_gy(e0 + u * kIT, v[u]);
        }
        for (int i4 = t + XU * kIT; i4 < xquads; i4 += kIT)
            store_x(i4, *reinterpret_cast<const f32x4 *>(xi + 4 * i4));
        ODL_IMAGE_STAMP(2);
        __syncthreads();
        ODL_IMAGE_STAMP(3);

        if (worker)
        {
            // pixel p = 4*step + kq of the image, row oh and column ow: po = oh*pr + ow is its offset in the padded input.
            // The operands of a step are fetched while the MFMAs of the step before run: two sets of registers take turns,
            // and nothing in the loop branches. (The fetch after the last step reads LDS past the rows in use — inside the
            // workgroup's allocation, never used.)
            int ow = kq, po = kq;
            const float *ap = gs + kq * ldg + rb * kBlockRows + j;
            const int steps = P / 4, wrap_add = 4 + g.pr - W;
            float fa[2][2], fb[2][3];
#define ODL_IMAGE_FETCH(S)                                                                             \
    {                                                                                                  \
        fa[S][0] = ap[0], fa[S][1] = ap[16];                                                           \
        fb[S][0] = xs[colbase[0] + po], fb[S][1] = xs[colbase[1] + po], fb[S][2] = xs[colbase[2] + po]; \
        ap += 4 * ldg;                                                                                 \
        ow += 4;                                                                                       \
        const bool wrap = ow >= W; /* (W >= 4: at most one row further) */                             \
        ow -= wrap ? W : 0;                                                                            \
        po += wrap ? wrap_add : 4;                                                                     \
    }
#define ODL_IMAGE_MFMAS(S)                                                                             \
    {                                                                                                  \
        acc[0][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[S][0], fb[S][0], acc[0][0], 0, 0, 0);     \
        acc[1][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[S][1], fb[S][0], acc[1][0], 0, 0, 0);     \
        acc[0][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[S][0], fb[S][1], acc[0][1], 0, 0, 0);     \
        acc[1][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[S][1], fb[S][1], acc[1][1], 0, 0, 0);     \
        acc[0][2] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[S][0], fb[S][2], acc[0][2], 0, 0, 0);     \
        acc[1][2] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[S][1], fb[S][2], acc[1][2], 0, 0, 0);     \
    }
            ODL_IMAGE_FETCH(0)
            for (int s = 0; s + 2 <= steps; s += 2)
            {
                ODL_IMAGE_FETCH(1)
                __builtin_amdgcn_sched_barrier(0);
                ODL_IMAGE_MFMAS(0)
                __builtin_amdgcn_sched_barrier(0);
                ODL_IMAGE_FETCH(0)
                __builtin_amdgcn_sched_barrier(0);
                ODL_IMAGE_MFMAS(1)
                __builtin_amdgcn_sched_barrier(0);
            }
            if (steps & 1)
                ODL_IMAGE_MFMAS(0)
#undef ODL_IMAGE_FETCH
#undef ODL_IMAGE_MFMAS
        }
        ODL_IMAGE_STAMP(4);
        if (gb_ch < OC)
            for (int q0 = gb_q; q0 < P / 4; q0 += 4 * gb_share)  // (four reads in flight)
            {
                float b[4];
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    b[u] = ps[gb_ch * (P / 4) + (q0 + u * gb_share < P / 4 ? q0 + u * gb_share : q0)];
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    bacc += q0 + u * gb_share < P / 4 ? b[u] : 0.f;
            }
    }

    ODL_IMAGE_STAMP(5);
    // ---- one partial per workgroup: gW as it lies in gW, then the bias sums. The blocks meet in LDS so that the partial
    // is written in whole 16-byte pieces one after the other (from the registers a wave's store covered four rows by 64
    // bytes, half a cache line each).
    float *out = g.part + (int64_t)blockIdx.x * g.E;
    const int tp = g.tile_pitch;
    float *tile = lds;                 // [OC][tile_pitch]
    float *shares = tile + OC * tp;    // [OC][gb_share]
    __syncthreads();  // the last image has been read
    if (worker)
    {
#pragma unroll
        for (int rt = 0; rt < 2; ++rt)
#pragma unroll
            for (int ct = 0; ct < 3; ++ct)
            {
                const int col = cb * kBlockCols + ct * 16 + j;
                if (col < g.cols)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        tile[(rb * kBlockRows + rt * 16 + 4 * kq + r) * tp + col] = acc[rt][ct][r];
            }
    }
    if (gb_ch < OC)
        shares[t] = bacc;
    __syncthreads();
    const odl::FastDiv by_cols = g.by_cols;
    for (int f4 = t; f4 < OC * g.cols / 4; f4 += kIT)
    {
        unsigned row = odl::fastdiv(4u * (unsigned)f4, by_cols), col = 4u * (unsigned)f4 - row * (unsigned)g.cols;
        f32x4 v;
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            v[q] = tile[row * tp + col];
            if (++col == (unsigned)g.cols)
                col = 0, ++row;
        }
        *reinterpret_cast<f32x4 *>(out + 4 * f4) = v;
    }
    if (t < OC)
    {
        float s = shares[t * gb_share];
        for (int q = 1; q < gb_share; ++q)
            s += shares[t * gb_share + q];
        out[OC * g.cols + t] = s;
    }
    ODL_IMAGE_STAMP(6);
}

// gw, gb = sum over the workgroups' partials in workgroup order: sixteen 16-byte columns per workgroup, 64 threads a
// column that each add every 64th partial from their own on; their sums are added four and then sixteen at a time in
// thread order — the same order on every run. Workgroups past the fold's (n_fold of them) make the filter copy that the
// LDS-patch input gradient stages from (conv_side.h), one launch less when that kernel follows.
__global__ __launch_bounds__(1024) void conv_image_fold_kernel(const float *__restrict__ part, int nparts, int E4, int W4,
                                                                float *gw, float *gb, unsigned n_fold, odl::SidePack pack,
                                                                unsigned n_pack)
{
    __shared__ f32x4 sums[64][16];
    __shared__ f32x4 sums2[16][16];
    if (blockIdx.x >= n_fold)
    {
        odl::side_pack(pack, blockIdx.x - n_fold, n_pack);
        return;
    }
    const int t = threadIdx.x, col = t & 15, sub = t >> 4;
    const int i = blockIdx.x * 16 + col;
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    if (i < E4)
    {
#pragma unroll 4
        for (int z = sub; z < nparts; z += 64)
            s += reinterpret_cast<const f32x4 *>(part)[(int64_t)z * E4 + i];
    }
    sums[sub][col] = s;
    __syncthreads();
    if (t < 256)
        sums2[sub][col] = ((sums[4 * sub][col] + sums[4 * sub + 1][col]) + sums[4 * sub + 2][col]) + sums[4 * sub + 3][col];
    __syncthreads();
    if (t < 16 && i < E4)
    {
        f32x4 v = sums2[0][col];
        for (int q = 1; q < 16; ++q)
            v += sums2[q][col];
        float *o = i < W4 ? (gw ? gw + 4 * (int64_t)i : nullptr) : (gb ? gb + 4 * (int64_t)(i - W4) : nullptr);
        if (o)
            o[0] = v[0], o[1] = v[1], o[2] = v[2], o[3] = v[3];
    }
}

// The pitches of the padded input in LDS: the 64 lanes of a B read differ in column (c, kh, kw) and pixel, and the
// 32 banks should see each of them at most twice (the least 64 lanes can do). Searched once per image shape.
struct Pitches
{
    int pr, pc;
};

Pitches find_pitches(int C, int H, int W)
{
    static std::mutex mu;
    static std::map<std::tuple<int, int, int>, Pitches> known;
    const auto key = std::make_tuple(C, H, W);
    std::lock_guard<std::mutex> hold(mu);
    const auto it = known.find(key);
    if (it != known.end())
        return it->second;
    const int cols = C * 9, P = H * W;
    const int tiles = (cols + 15) / 16, steps = std::min(P / 4, 2 * W);
    Pitches best{W + 2, (H + 2) * (W + 2)};
    long best_cost = -1;
    for (int pr = W + 2; pr <= W + 5; ++pr)
        for (int pc = (H + 2) * pr; pc <= (H + 2) * pr + 32; ++pc)
        {
            long cost = 0;
            for (int ct = 0; ct < tiles; ++ct)
                for (int s = 0; s < steps; ++s)
                {
                    int hits[32] = {0}, worst = 0;
                    for (int l = 0; l < 64; ++l)
                    {
                        const int col = std::min(ct * 16 + l % 16, cols - 1), p = 4 * s + l / 16;
                        const int c = col / 9, tap = col % 9;
                        const int a = c * pc + (tap / 3) * pr + tap % 3 + (p / W) * pr + p % W;
                        worst = std::max(worst, ++hits[a & 31]);
                    }
                    cost += worst;
                }
            if (best_cost < 0 || cost < best_cost)
                best_cost = cost, best = Pitches{pr, pc};
        }
    known[key] = best;
    return best;
}

struct ImagePlan
{
    bool ok;
    int blocks_c, blocks, nwg, ldg, tile_pitch;
    Pitches pitch;
    size_t lds;
};

ImagePlan plan_image(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC)
{
    ImagePlan p{};
    const int64_t P = H * W;
    if (OC % kBlockRows != 0 || OC > kIT || C < 1 || W < 4 || P % 4 != 0 || C * 9 > 4096 || H > 64 || W > 64)
        return p;
    p.blocks_c = (int)odl::ceil_div(C * 9, kBlockCols);
    p.blocks = (int)(OC / kBlockRows) * p.blocks_c;
    // every block needs a wave of its own, and most waves should have one
    if (p.blocks > kWaves || p.blocks < kWaves / 2 || OC * P / 4 < kIT)
        return p;
    // an image per workgroup: too few images leave most of the chip idle
    const int cus = odl::device_cus();
    if (2 * N < cus || N * OC * P >= (1ll << 40) || N * C * P >= (1ll << 40))
        return p;
    p.nwg = (int)(N < cus ? N : cus);
    p.ldg = (int)OC + 16;  // (16 mod 32: the four pixels of an A read fall into different halves of the banks)
    // the pitch search is only worth its time for a shape that passes the cheap tests
    const int64_t lds_least = (P * p.ldg + C * (H + 2) * (W + 2) + OC * P / 4) * 4;
    if (lds_least > 160 * 1024)
        return p;
    p.pitch = find_pitches((int)C, (int)H, (int)W);
    // gW's rows in LDS at the end: a pitch of 4 mod 8 floats puts the four rows of an accumulator store into different
    // halves of the banks
    p.tile_pitch = (int)(C * 9 + 7) / 8 * 8 + 4;
    const size_t staged = (size_t)(P * p.ldg + C * p.pitch.pc + OC * P / 4), gathered = (size_t)(OC * p.tile_pitch + kIT);
    p.lds = (staged > gathered ? staged : gathered) * sizeof(float);
    p.ok = p.lds <= 160 * 1024;
    return p;
}

hipError_t allow_lds()
{
    static const hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(&conv_image_wgrad_kernel),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    return rc;
}
}  // namespace

namespace odl
{
bool conv_image_wgrad_ok(const float *gy, const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                         int SH, int SW, int PH, int PW)
{
    if (!(KH == 3 && KW == 3 && SH == 1 && SW == 1 && PH == 1 && PW == 1))
        return false;
    if (((reinterpret_cast<uintptr_t>(gy) | reinterpret_cast<uintptr_t>(x)) & 15) != 0)
        return false;
    return plan_image(N, C, H, W, OC).ok;
}

size_t conv_image_wgrad_workspace(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC)
{
    const ImagePlan p = plan_image(N, C, H, W, OC);
    return p.ok ? (size_t)p.nwg * (size_t)(OC * C * 9 + OC) * sizeof(float) : 0;
}

// gw and gb may each be null (the partials are computed either way). pack: a filter copy for the input gradient to be made
// by n_pack more workgroups of the second launch, or null.
int conv_image_wgrad(const float *gy, const float *x, float *gw, float *gb, int64_t N, int64_t C, int64_t H, int64_t W,
                     int64_t OC, void *workspace, size_t workspace_bytes, hipStream_t st, const SidePack *pack, unsigned n_pack)
{
    const ImagePlan p = plan_image(N, C, H, W, OC);
    if (!p.ok)
        return fail(ODL_ERR_RUNTIME, "conv2d_backward: the image-resident weight gradient does not take this shape");
    const size_t need = (size_t)p.nwg * (size_t)(OC * C * 9 + OC) * sizeof(float);
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= need && reinterpret_cast<uintptr_t>(workspace) % 16 == 0,
                "conv2d_backward: a 16-byte aligned workspace of %zu bytes required, got %zu", need, workspace_bytes);
    ImageGeom g{};
    g.gy = gy, g.x = x, g.part = static_cast<float *>(workspace);
    g.N = (int)N, g.C = (int)C, g.H = (int)H, g.W = (int)W, g.OC = (int)OC, g.P = (int)(H * W), g.cols = (int)(C * 9);
    g.pr = p.pitch.pr, g.pc = p.pitch.pc, g.ldg = p.ldg;
    g.blocks_c = p.blocks_c, g.blocks = p.blocks;
    g.E = (int)(OC * C * 9 + OC);
    g.tile_pitch = p.tile_pitch, g.by_cols = make_fastdiv((unsigned)(C * 9));
    g.by_oc = make_fastdiv((unsigned)OC), g.by_p = make_fastdiv((unsigned)g.P), g.by_w = make_fastdiv((unsigned)W);
    ODL_HIP_CHECK(allow_lds());
    hipLaunchKernelGGL(conv_image_wgrad_kernel, dim3(p.nwg), dim3(kIT), p.lds, st, g);
    ODL_LAUNCH_CHECK();
    if (gw || gb || pack)
    {
        const int E4 = g.E / 4;
        const unsigned n_fold = (gw || gb) ? (unsigned)ceil_div(E4, 16) : 0u;
        if (!pack)
            n_pack = 0;
        hipLaunchKernelGGL(conv_image_fold_kernel, dim3(n_fold + n_pack), dim3(1024), 0, st, g.part, p.nwg, E4,
                           (int)(OC * C * 9 / 4), gw, gb, n_fold, pack ? *pack : SidePack{}, n_pack);
        ODL_LAUNCH_CHECK();
    }
    return ODL_OK;
}
}  // namespace odl
