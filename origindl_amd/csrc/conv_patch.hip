// 3x3, stride 1, padding 1 convolution on the matrix cores (v_mfma_f32_32x32x2_f32) with the input patch held in LDS.
//
// The implicit-GEMM kernels gather one [16 k, 128 pixel] operand tile per 16 values of K, so every input element
// travels from L2 to LDS once per filter tap. Here a workgroup stages, per slab of 16 input channels, the image rows
// its 128 output pixels touch (plus one halo row above and below and one zero column left and right) once, and the
// nine taps read that patch at shifted LDS addresses: nine times fewer loads and one barrier pair per 144 values of K.
//
// One kernel serves two products of a 3x3/s1/p1 layer (src/operators/conv/conv2d.cpp:458-560 in the reference):
//   forward         y[n,oc,h,w]  = b[oc] + sum_{c,t} x[n,c,h+dy,w+dx] * w[oc,c,t]                (source read as NCHW)
//   input gradient  gx[n,c,h,w]  = sum_{oc,t} gy2d[pix(n,h+dy,w+dx)][oc] * w[oc,c,8-t]
// where gy2d is the gradient buffer read as a row-major [N*OH*OW, OC] matrix exactly as it lies, the reference's
// reading (conv2d.cpp:548) — for this kernel a channel-minor source.
#include "conv_side.h"
#include "odl_common.h"

#include <atomic>

namespace
{
// least number of workgroups for which this kernel is chosen; negative = one per compute unit of the device
std::atomic<int64_t> g_min_wgs{-1};

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int V>
struct ActTag  // the activation as a compile-time value for a generic lambda
{
    static constexpr int value = V;
};

constexpr int kThreads = 256;
constexpr int kPixTile = 128;    // output pixels per workgroup, consecutive in (n, h, w) order
constexpr int kSlab = 16;        // input channels per staging step
constexpr int kPosPerThread = 2; // patch positions (row, column) one thread stages
constexpr int kLdp = kSlab + 4;  // floats per patch position in LDS: 16-byte aligned, an odd number of 16-byte units
constexpr int kLda = 9 * kSlab + 4;  // floats per filter row in LDS, likewise
constexpr size_t kLdsCap = 80 * 1024;  // two workgroups per compute unit

struct PatchGeom
{
    const float *src, *wp, *bias;
    float *dst;
    int Cin, M, Mpad, NH, H, W, HW;  // NH = N*H image rows in the batch
    int PW, plane;                   // patch width W + 2 and positions per patch (rows * PW)
    int pixels, mtiles, act;
    odl::FastDiv by_w, by_h, by_hw, by_pw;
    // Tail split. The launch runs in rounds of as many workgroups as the chip holds; when the last round would be a
    // handful of tiles, those tiles (numbers tail_first..) are cut into tail_pieces runs of channel slabs instead —
    // workgroups main_blocks.. — which write their raw accumulators to tail_ws, one [BM][128] block per (tile, piece);
    // conv_patch_tail_kernel adds the pieces in order and finishes the tile.
    int main_blocks, tail_first, tail_pieces, slabs_per_piece;
    float *tail_ws;
    int xcds;  // consecutive workgroup ids are dealt round-robin over this many XCDs, each with an L2 of its own
};

// wp[(m*nslab + slab)*144 + tap*16 + cc]: the zero-padded filter copy the kernel stages with 16-byte copies
__global__ void conv_patch_pack_kernel(const odl::SidePack p)
{
    odl::side_pack(p, blockIdx.x, gridDim.x);
}

template <int BM, bool CH_MINOR>
__global__ __launch_bounds__(kThreads) void conv_patch_kernel(const PatchGeom g)
{
    constexpr int KS = 9 * kSlab;
    constexpr int WM = BM >= 64 ? 2 : 1, WN = 4 / WM;
    constexpr int TM = BM / WM, TN = kPixTile / WN;
    constexpr int RB = TM / 32, CB = TN / 32;
    extern __shared__ float lds[];
    float *As = lds;              // [BM][kLda]
    float *Bs = lds + BM * kLda;  // [plane + 3][kLdp]; the last three positions stay zero
    float *bias_s = Bs + (g.plane + 3) * kLdp;  // [BM]: the bias of the tile's rows (zeros without one)

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, l32 = lane & 31, lh = lane >> 5;
    int tile = blockIdx.x, piece = -1;
    if (g.tail_pieces > 0 && (int)blockIdx.x >= g.main_blocks)
    {
        const int u = (int)blockIdx.x - g.main_blocks;
        tile = g.tail_first + u / g.tail_pieces;
        piece = u % g.tail_pieces;
    }
    else
    {
        // a contiguous band of tiles per XCD: the output-channel tiles of one pixel tile read the same patch, and the
        // next pixel tile shares two of its rows, so they should meet in one L2
        const unsigned total = (unsigned)g.main_blocks, nx = (unsigned)g.xcds;
        const unsigned loc = blockIdx.x / nx, xcd = blockIdx.x - loc * nx;
        const unsigned full = total / nx, rem = total - full * nx;
        tile = (int)(xcd * full + (xcd < rem ? xcd : rem) + loc);
    }
    const int mt = tile % g.mtiles, nt = tile / g.mtiles;
    const int m0 = mt * BM, p0 = nt * kPixTile;
    const int wm = (wave % WM) * TM, wn = (wave / WM) * TN;
    const int gr0 = (int)odl::fastdiv((unsigned)p0, g.by_w);  // first image row (of the whole batch) of the tile

    // ---- where this thread's patch positions come from: patch row r is batch row gr0 - 1 + r
    int src_off[kPosPerThread];
#pragma unroll
    for (int i = 0; i < kPosPerThread; ++i)
    {
        const int pos = t + i * kThreads;
        const int r = (int)odl::fastdiv((unsigned)pos, g.by_pw), col = pos - r * g.PW;
        const int gr = gr0 - 1 + r;
        const bool ok = pos < g.plane && col >= 1 && col <= g.W && gr >= 0 && gr < g.NH;
        int off = -1;
        if (ok)
        {
            if (CH_MINOR)
                off = (gr * g.W + col - 1) * g.Cin;
            else
            {
                const int n = (int)odl::fastdiv((unsigned)gr, g.by_h), h = gr - n * g.H;
                off = (n * g.Cin * g.H + h) * g.W + col - 1;
            }
        }
        src_off[i] = off;
    }
    if (t < 3 * kLdp)
        Bs[g.plane * kLdp + t] = 0.f;
    // The bias of the tile's rows waits in LDS from here on (the first barrier of the slab loop publishes it): fetched
    // after the last slab it cost every workgroup a trip to memory before its first store — 4.3 us of a 28 us
    // workgroup by in-kernel timestamps — and held in registers it took the 64-row kernel past 256 registers.
    const bool has_bias = g.bias != nullptr && piece < 0;
    if (t < BM)
        bias_s[t] = (has_bias && m0 + t < g.M) ? g.bias[m0 + t] : 0.f;

    // ---- where this lane's output pixels sit in the patch, one base per tap row; a tap row that falls outside the
    // pixel's own image points at the zero positions instead
    int base[CB][3];
#pragma unroll
    for (int j = 0; j < CB; ++j)
    {
        int p = p0 + wn + j * 32 + l32;
        p = p < g.pixels ? p : g.pixels - 1;
        const int grow = (int)odl::fastdiv((unsigned)p, g.by_w), w = p - grow * g.W;
        const int n = (int)odl::fastdiv((unsigned)grow, g.by_h), h = grow - n * g.H;
        // the position left of the pixel, so that the three taps of a row sit at offsets 0, 1 and 2 positions
        const int left = (grow - gr0 + 1) * g.PW + w;
        const int zero = g.plane;
        base[j][0] = (h > 0 ? left - g.PW : zero) * kLdp + 4 * lh;
        base[j][1] = left * kLdp + 4 * lh;
        base[j][2] = (h < g.H - 1 ? left + g.PW : zero) * kLdp + 4 * lh;
    }

    f32x16 acc[RB][CB];
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int j = 0; j < CB; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0.f;

    const int nslab = g.Cin / kSlab;
    const int ch_stride = CH_MINOR ? 1 : g.HW;
    const int s_beg = piece < 0 ? 0 : piece * g.slabs_per_piece;
    const int s_end = piece < 0 ? nslab : (s_beg + g.slabs_per_piece < nslab ? s_beg + g.slabs_per_piece : nslab);

    // one slab travels global memory -> registers -> LDS; the loads of slab s + 1 are issued before the matrix
    // instructions of slab s and land while those run
    constexpr int A_VECS = KS * BM / 4, A_PER_T = (A_VECS + kThreads - 1) / kThreads;
    f32x4 ra[A_PER_T];
    float rb[kPosPerThread][kSlab];
    auto load_slab = [&](int s)
    {
        const float *wsrc = g.wp + ((int64_t)m0 * nslab + s) * KS;
#pragma unroll
        for (int q = 0; q < A_PER_T; ++q)
        {
            const int e = t + q * kThreads;
            if (A_VECS % kThreads == 0 || e < A_VECS)
            {
                const int m = e / (KS / 4), k4 = e % (KS / 4);
                ra[q] = *reinterpret_cast<const f32x4 *>(wsrc + (int64_t)m * nslab * KS + k4 * 4);
            }
        }
#pragma unroll
        for (int i = 0; i < kPosPerThread; ++i)
        {
            if (src_off[i] < 0)
            {
#pragma unroll
                for (int cc = 0; cc < kSlab; ++cc)
                    rb[i][cc] = 0.f;
            }
            else if (CH_MINOR)
            {
                const f32x4 *in = reinterpret_cast<const f32x4 *>(g.src + src_off[i] + s * kSlab);
#pragma unroll
                for (int q = 0; q < kSlab / 4; ++q)
                {
                    const f32x4 v = in[q];
                    rb[i][q * 4 + 0] = v[0], rb[i][q * 4 + 1] = v[1], rb[i][q * 4 + 2] = v[2], rb[i][q * 4 + 3] = v[3];
                }
            }
            else
            {
                const float *in = g.src + src_off[i] + (int64_t)s * kSlab * ch_stride;
#pragma unroll
                for (int cc = 0; cc < kSlab; ++cc)
                    rb[i][cc] = in[(int64_t)cc * ch_stride];
            }
        }
    };
    auto store_slab = [&]()
    {
#pragma unroll
        for (int q = 0; q < A_PER_T; ++q)
        {
            const int e = t + q * kThreads;
            if (A_VECS % kThreads == 0 || e < A_VECS)
            {
                const int m = e / (KS / 4), k4 = e % (KS / 4);
                *reinterpret_cast<f32x4 *>(As + m * kLda + k4 * 4) = ra[q];
            }
        }
#pragma unroll
        for (int i = 0; i < kPosPerThread; ++i)
        {
            const int pos = t + i * kThreads;
            if (pos < g.plane)
            {
#pragma unroll
                for (int q = 0; q < kSlab / 4; ++q)
                {
                    f32x4 v;
                    v[0] = rb[i][q * 4 + 0], v[1] = rb[i][q * 4 + 1], v[2] = rb[i][q * 4 + 2], v[3] = rb[i][q * 4 + 3];
                    *reinterpret_cast<f32x4 *>(Bs + pos * kLdp + q * 4) = v;
                }
            }
        }
    };

    load_slab(s_beg);
    for (int s = s_beg; s < s_end; ++s)
    {
        __syncthreads();  // the previous slab has been read
        store_slab();
        __syncthreads();
        if (s + 1 < s_end)
            load_slab(s + 1);

        // ---- 144 values of K: nine taps x two groups of eight channels. One 16-byte read per operand block brings four
        // channels; instruction e of a group takes channel e from lanes 0-31 and channel 4 + e from lanes 32-63. The
        // operands of group q + 1 are read while the instructions of group q run.
        constexpr int NG = 9 * (kSlab / 8);
        f32x4 a[2][RB], b[2][CB];
        auto read_group = [&](int q, int buf)
        {
            const int tap = q / (kSlab / 8), g8 = q % (kSlab / 8);
            const int dyi = tap / 3, dxi = tap % 3;
#pragma unroll
            for (int i = 0; i < RB; ++i)
                a[buf][i] =
                    *reinterpret_cast<const f32x4 *>(As + (wm + i * 32 + l32) * kLda + tap * kSlab + g8 * 8 + 4 * lh);
#pragma unroll
            for (int j = 0; j < CB; ++j)
                b[buf][j] = *reinterpret_cast<const f32x4 *>(Bs + base[j][dyi] + dxi * kLdp + g8 * 8);
        };
        read_group(0, 0);
#pragma unroll
        for (int q = 0; q < NG; ++q)
        {
            if (q + 1 < NG)
                read_group(q + 1, (q + 1) & 1);
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int i = 0; i < RB; ++i)
#pragma unroll
                    for (int j = 0; j < CB; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[q & 1][i][e], b[q & 1][j][e], acc[i][j], 0, 0, 0);
            // issue order for the instruction scheduler: the next group's LDS reads go between this group's first
            // matrix instructions instead of after its last
            if (q + 1 < NG)
            {
#pragma unroll
                for (int r = 0; r < RB + CB; ++r)
                {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one matrix instruction
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
                }
                __builtin_amdgcn_sched_group_barrier(0x008, 4 * RB * CB - (RB + CB), 0);
            }
            else
                __builtin_amdgcn_sched_group_barrier(0x008, 4 * RB * CB, 0);
        }
    }

    // ---- accumulator register r of lane (l32, lh) holds row 8*(r/4) + 4*lh + r%4, column l32
    if (piece >= 0)
    {
        // a piece of a tail tile: the raw sums, tile-local (rows or pixels past the end hold whatever the padding gave)
        float *out = g.tail_ws + ((int64_t)(tile - g.tail_first) * g.tail_pieces + piece) * (BM * kPixTile);
#pragma unroll
        for (int j = 0; j < CB; ++j)
#pragma unroll
            for (int i = 0; i < RB; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    out[(wm + i * 32 + 8 * (r / 4) + 4 * lh + (r % 4)) * kPixTile + wn + j * 32 + l32] = acc[i][j][r];
        return;
    }
    float bv[RB][16];
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            const f32x4 b4 = *reinterpret_cast<const f32x4 *>(bias_s + wm + i * 32 + 8 * q + 4 * lh);
            bv[i][4 * q + 0] = b4[0], bv[i][4 * q + 1] = b4[1], bv[i][4 * q + 2] = b4[2], bv[i][4 * q + 3] = b4[3];
        }
    auto store_all = [&](auto act_tag) {
        constexpr int ACT = decltype(act_tag)::value;
#pragma unroll
        for (int j = 0; j < CB; ++j)
        {
            const int p = p0 + wn + j * 32 + l32;
            if (p >= g.pixels)
                continue;
            const int n = (int)odl::fastdiv((unsigned)p, g.by_hw), hw = p - n * g.HW;
#pragma unroll
            for (int i = 0; i < RB; ++i)
            {
                const int row0 = m0 + wm + i * 32 + 4 * lh;
                const int rows_left = g.M - row0;
                float *out = g.dst + ((int64_t)n * g.M + row0) * g.HW + hw;
#pragma unroll
                for (int r = 0; r < 16; ++r)
                {
                    const int dr = 8 * (r / 4) + (r % 4);
                    if (dr >= rows_left)
                        continue;
                    float v = acc[i][j][r];
                    if (has_bias)
                        v = v + bv[i][r];
                    out[(int64_t)dr * g.HW] = odl::apply_act(v, ACT);
                }
            }
        }
    };
    if (g.act == 1)
        store_all(ActTag<1>{});
    else if (g.act == 2)
        store_all(ActTag<2>{});
    else
        store_all(ActTag<0>{});
}

// Adds the pieces of each tail tile in piece order and stores the tile the way the main kernel does (bias, activation,
// NCHW). One thread per output element, lanes along the pixels.
__global__ __launch_bounds__(kThreads) void conv_patch_tail_kernel(const PatchGeom g, int BM)
{
    const int per_tile = BM * kPixTile;
    const int idx = blockIdx.x * kThreads + threadIdx.x;
    const int ti = idx / per_tile, e = idx - ti * per_tile;
    const int tile = g.tail_first + ti;
    if (tile >= g.mtiles * (int)((g.pixels + kPixTile - 1) / kPixTile))
        return;
    const int row_l = e / kPixTile, px = e - row_l * kPixTile;
    const int mt = tile % g.mtiles, nt = tile / g.mtiles;
    const int row = mt * BM + row_l, p = nt * kPixTile + px;
    if (row >= g.M || p >= g.pixels)
        return;
    const float *src = g.tail_ws + (int64_t)ti * g.tail_pieces * per_tile + e;
    float v = src[0];
    for (int z = 1; z < g.tail_pieces; ++z)
        v += src[(int64_t)z * per_tile];
    if (g.bias)
        v = v + g.bias[row];
    const int n = (int)odl::fastdiv((unsigned)p, g.by_hw), hw = p - n * g.HW;
    g.dst[((int64_t)n * g.M + row) * g.HW + hw] = odl::apply_act(v, g.act);
}

inline int patch_rows(int64_t W)
{
    return (int)((W - 1 + kPixTile - 1) / W) + 1 + 2;
}

inline int tile_bm(int64_t M)
{
    return M <= 32 ? 32 : 64;
}

inline size_t lds_bytes(int bm, int plane)
{
    return ((size_t)bm * kLda + (size_t)(plane + 3) * kLdp + (size_t)bm) * sizeof(float);  // filters, patch, the tile's bias
}

// more dynamic LDS than the default limit of 64 KB, asked for once per kernel
template <int BM, bool CH_MINOR>
hipError_t allow_lds_of()
{
    static const hipError_t rc =
        hipFuncSetAttribute(reinterpret_cast<const void *>(&conv_patch_kernel<BM, CH_MINOR>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsCap);
    return rc;
}

hipError_t allow_lds(int bm, bool ch_minor)
{
    if (bm == 32)
        return ch_minor ? allow_lds_of<32, true>() : allow_lds_of<32, false>();
    return ch_minor ? allow_lds_of<64, true>() : allow_lds_of<64, false>();
}

bool shape_ok(const float *src, int64_t N, int64_t Cin, int64_t H, int64_t W, int64_t M, int KH, int KW, int SH, int SW,
              int PH, int PW)
{
    if (!(KH == 3 && KW == 3 && SH == 1 && SW == 1 && PH == 1 && PW == 1))
        return false;
    if (Cin < kSlab || Cin % kSlab != 0 || M < 1 || reinterpret_cast<uintptr_t>(src) % 16 != 0)
        return false;
    const int64_t plane = (int64_t)patch_rows(W) * (W + 2);
    if (plane > kPosPerThread * kThreads || lds_bytes(tile_bm(M), (int)plane) > kLdsCap)
        return false;
    // fewer workgroups than compute units: the implicit kernels, which slice K, do better
    // (odl_hip_set_conv_patch_min_workgroups replaces the threshold, so that small shapes can be sent through this kernel)
    const int64_t min_wgs = g_min_wgs.load(std::memory_order_relaxed);
    if (odl::ceil_div(N * H * W, kPixTile) * odl::ceil_div(M, tile_bm(M)) < (min_wgs < 0 ? odl::device_cus() : min_wgs))
        return false;
    // 32-bit element offsets inside the kernel
    return N * Cin * H * W < (1ll << 31) && N * M * H * W < (1ll << 40) && N * H * W < (1ll << 31) - kPixTile &&
           Cin * 9 * (M + 64) < (1ll << 31);
}

size_t packed_bytes(int64_t Cin, int64_t M)
{
    const int bm = tile_bm(M);
    const int64_t mpad = odl::ceil_div(M, bm) * bm;
    return (((size_t)Cin * 9 * mpad * sizeof(float)) + 255) & ~(size_t)255;
}

// the channel-minor kernel runs a 33..64-row product of many pixel tiles as two 32-row tiles
bool use_halves(int64_t pixels, int64_t M, bool ch_minor)
{
    return ch_minor && tile_bm(M) == 64 && M <= 64 && odl::ceil_div(pixels, kPixTile) >= 512;
}

// Workgroups of a variant that one compute unit holds at once: what the runtime reports for the kernel (registers and
// LDS together), or, on a machine without a device — where only the workspace-size queries run — the same figure from
// the kernels' register counts (96 / 156 / 138 / 198 of 512 per SIMD) and the LDS size.
int wgs_per_cu(int bm, bool ch_minor, size_t lds)
{
    int n = 0;
    const void *fn = bm == 32 ? (ch_minor ? reinterpret_cast<const void *>(&conv_patch_kernel<32, true>)
                                          : reinterpret_cast<const void *>(&conv_patch_kernel<32, false>))
                              : (ch_minor ? reinterpret_cast<const void *>(&conv_patch_kernel<64, true>)
                                          : reinterpret_cast<const void *>(&conv_patch_kernel<64, false>));
    (void)allow_lds(bm, ch_minor);
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, fn, kThreads, lds) == hipSuccess && n > 0)
        return n;
    (void)hipGetLastError();
    const int by_regs = bm == 32 ? (ch_minor ? 5 : 3) : (ch_minor ? 3 : 2);
    const int by_lds = (int)((160 * 1024) / (lds > 0 ? lds : 1));
    n = by_regs < by_lds ? by_regs : by_lds;
    return n > 0 ? n : 1;
}

struct TailPlan
{
    int tiles = 0, pieces = 0, slabs_per_piece = 0;
    size_t bytes = 0;
};

// A launch runs in rounds of `slots` workgroups. When the last round would hold at most half of that, its tiles are
// cut into runs of channel slabs so that the round is short.
TailPlan plan_tail(int64_t n_wg, int nslab, int bm, bool ch_minor, size_t lds)
{
    TailPlan p;
    const int64_t slots = (int64_t)wgs_per_cu(bm, ch_minor, lds) * odl::device_cus();
    const int64_t r = n_wg % slots;
    if (n_wg <= slots || r == 0 || r > slots / 2 || nslab < 2)
        return p;
    int64_t pieces = slots / r;
    if (pieces > nslab)
        pieces = nslab;
    if (pieces > 8)
        pieces = 8;
    if (pieces < 2)
        return p;
    p.slabs_per_piece = (int)odl::ceil_div(nslab, pieces);
    p.pieces = (int)odl::ceil_div(nslab, p.slabs_per_piece);
    p.tiles = (int)r;
    p.bytes = (size_t)p.tiles * p.pieces * bm * kPixTile * sizeof(float);
    return p;
}

TailPlan plan_tail_for(int64_t N, int64_t Cin, int64_t H, int64_t W, int64_t M, bool ch_minor)
{
    const int bm_pad = tile_bm(M);
    const int bm = use_halves(N * H * W, M, ch_minor) ? 32 : bm_pad;
    const int64_t mtiles = odl::ceil_div(M, bm_pad) * bm_pad / bm;
    const int plane = patch_rows(W) * ((int)W + 2);
    return plan_tail(odl::ceil_div(N * H * W, kPixTile) * mtiles, (int)(Cin / kSlab), bm, ch_minor, lds_bytes(bm, plane));
}

// packed: the filter copy at the head of the workspace has been made already (by the caller's own launch of side_pack)
int launch(const float *src, const float *w, const float *bias, float *dst, int64_t N, int64_t Cin, int64_t H, int64_t W,
           int64_t M, bool ch_minor, int act, void *workspace, size_t workspace_bytes, hipStream_t st, const char *who,
           bool packed = false)
{
    const size_t need = packed_bytes(Cin, M);
    if (!workspace || workspace_bytes < need || reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
        return odl::fail(ODL_ERR_INVALID_ARG, "%s: needs a 16-byte aligned workspace of %zu bytes, got %zu", who, need,
                         workspace_bytes);
    // The filter copy is padded to tile_bm(M) rows. The channel-minor kernel runs a 33..64-row product of many pixel
    // tiles as two 32-row tiles: twice the workgroups at half the length leave a shorter tail when the last
    // workgroups of the launch drain (64 rows x 784 pixel tiles: 170 -> 162 us).
    const int bm_pad = tile_bm(M);
    const bool halves = use_halves(N * H * W, M, ch_minor);
    const int bm = halves ? 32 : bm_pad;
    PatchGeom g{};
    g.src = src, g.bias = bias, g.dst = dst;
    g.Cin = (int)Cin, g.M = (int)M, g.Mpad = (int)(odl::ceil_div(M, bm_pad) * bm_pad);
    g.NH = (int)(N * H), g.H = (int)H, g.W = (int)W, g.HW = (int)(H * W);
    g.PW = (int)W + 2, g.plane = patch_rows(W) * g.PW;
    g.pixels = (int)(N * H * W), g.mtiles = g.Mpad / bm, g.act = act;
    g.by_w = odl::make_fastdiv((unsigned)W), g.by_h = odl::make_fastdiv((unsigned)H);
    g.by_hw = odl::make_fastdiv((unsigned)(H * W)), g.by_pw = odl::make_fastdiv((unsigned)g.PW);
    float *wp = static_cast<float *>(workspace);
    g.wp = wp;
    if (!packed)
    {
        const int total = g.Cin * 9 * g.Mpad;
        hipLaunchKernelGGL(conv_patch_pack_kernel, dim3((unsigned)odl::ceil_div(total, 256)), dim3(256), 0, st,
                           odl::SidePack{w, wp, g.Cin, g.M, g.Mpad, ch_minor ? 1 : 0});
        ODL_LAUNCH_CHECK();
    }
    const size_t lds = lds_bytes(bm, g.plane);
    ODL_HIP_CHECK(allow_lds(bm, ch_minor));
    // the tiles of a short last round go out as runs of channel slabs (when the workspace has room for their sums)
    const int64_t n_wg = odl::ceil_div(g.pixels, kPixTile) * g.mtiles;
    const TailPlan tp = plan_tail(n_wg, g.Cin / kSlab, bm, ch_minor, lds);
    g.xcds = odl::chip().xcds;
    g.main_blocks = (int)n_wg, g.tail_first = (int)n_wg, g.tail_pieces = 0, g.slabs_per_piece = 0, g.tail_ws = nullptr;
    if (tp.pieces > 0 && workspace_bytes >= need + tp.bytes)
    {
        g.tail_first = (int)(n_wg - tp.tiles), g.main_blocks = g.tail_first;
        g.tail_pieces = tp.pieces, g.slabs_per_piece = tp.slabs_per_piece;
        g.tail_ws = reinterpret_cast<float *>(static_cast<char *>(workspace) + need);
    }
    const dim3 grid((unsigned)(g.main_blocks + (g.tail_pieces > 0 ? tp.tiles * tp.pieces : 0)));
    if (bm == 32)
    {
        if (ch_minor)
            hipLaunchKernelGGL((conv_patch_kernel<32, true>), grid, dim3(kThreads), lds, st, g);
        else
            hipLaunchKernelGGL((conv_patch_kernel<32, false>), grid, dim3(kThreads), lds, st, g);
    }
    else
    {
        if (ch_minor)
            hipLaunchKernelGGL((conv_patch_kernel<64, true>), grid, dim3(kThreads), lds, st, g);
        else
            hipLaunchKernelGGL((conv_patch_kernel<64, false>), grid, dim3(kThreads), lds, st, g);
    }
    ODL_LAUNCH_CHECK();
    if (g.tail_pieces > 0)
    {
        const int64_t threads = (int64_t)tp.tiles * bm * kPixTile;
        hipLaunchKernelGGL(conv_patch_tail_kernel, dim3((unsigned)odl::ceil_div(threads, kThreads)), dim3(kThreads), 0, st, g,
                           bm);
        ODL_LAUNCH_CHECK();
    }
    return ODL_OK;
}
}  // namespace

namespace odl
{
bool conv_patch_forward_ok(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH,
                           int SW, int PH, int PW)
{
    // Measured on the 3x3 layers of the benchmark networks, this kernel is the faster forward whenever it fills the chip:
    // few input channels (K < 576: the implicit-GEMM kernel's fixed cost per workgroup dominates there), short image
    // rows (64 -> 128 channels at 14x14: 96 against 109 us), and — since the tiles of a short last round are cut into
    // runs of channel slabs — long rows too (64 -> 128 channels at 56x56: 165 against 176 us).
    return shape_ok(x, N, C, H, W, OC, KH, KW, SH, SW, PH, PW);
}

size_t conv_patch_forward_workspace(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC)
{
    return packed_bytes(C, OC) + plan_tail_for(N, C, H, W, OC, false).bytes;
}

int conv_patch_forward(const float *x, const float *w, const float *b, float *y, int64_t N, int64_t C, int64_t H,
                       int64_t W, int64_t OC, int act, void *workspace, size_t workspace_bytes, hipStream_t st)
{
    return launch(x, w, b, y, N, C, H, W, OC, false, act, workspace, workspace_bytes, st, "conv2d");
}

bool conv_patch_dgrad_ok(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH,
                         int SW, int PH, int PW)
{
    return shape_ok(gy, N, OC, H, W, C, KH, KW, SH, SW, PH, PW);
}

size_t conv_patch_dgrad_workspace(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC)
{
    return packed_bytes(OC, C) + plan_tail_for(N, OC, H, W, C, true).bytes;
}

int conv_patch_dgrad(const float *gy, const float *w, float *gx, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
                     void *workspace, size_t workspace_bytes, hipStream_t st, bool packed)
{
    return launch(gy, w, nullptr, gx, N, OC, H, W, C, true, 0, workspace, workspace_bytes, st, "conv2d_backward", packed);
}

// the filter copy conv_patch_dgrad stages from, as a job for a launch of the caller's (then `packed` above)
SidePack conv_patch_dgrad_pack(const float *w, int64_t C, int64_t OC, void *workspace)
{
    const int bm_pad = tile_bm(C);
    return SidePack{w, static_cast<float *>(workspace), (int)OC, (int)C, (int)(ceil_div(C, bm_pad) * bm_pad), 1};
}
}  // namespace odl

extern "C" int odl_hip_set_conv_patch_min_workgroups(int64_t min_workgroups)
{
    g_min_wgs.store(min_workgroups < 0 ? -1 : min_workgroups, std::memory_order_relaxed);
    return ODL_OK;
}
