// Weight gradient of a 3x3 / padding 1 convolution (stride 1 or 2) on the matrix cores (v_mfma_f32_32x32x2_f32), walking
// the output image a few rows at a time:
//
//   gW[oc][c][kh][kw] = sum_m gy2d[m][oc] * x[n(m)][c][S*oh(m) + kh - 1][S*ow(m) + kw - 1]
//
// where gy2d is the upstream gradient's NCHW buffer read as a row-major [N*OH*OW, OC] matrix exactly as it lies (the
// reference's reading, src/mat/origin/cpu/conv/conv2d.cpp:548-562) and m = (n, oh, ow) counts output pixels.
//
// The product is [OC] x [C*9] with a reduction as long as the batch has output pixels, so almost all of the parallelism
// has to come from cutting the reduction, and every cut costs one partial copy of gW. The implicit-GEMM kernel gathers
// its col operand element by element (16 pixels x 128 (c,tap) rows per slab, 4-byte loads) and needs some 150 cuts of
// 128x128 tiles to keep its loads hidden. Here a workgroup owns a 128 (oc) x 192 (three taps of one filter row x 64
// channels) tile and walks a long run of output rows, one slab of R rows (R*OW = 32..64 pixels) at a time:
//   * the slab's gy2d rows are one contiguous piece of memory: they go straight into LDS (buffer_load ... lds), two
//     slabs deep, and are read back as the A operand with lanes along oc;
//   * the slab's input rows (for the tile's filter row: one input row per output row) are staged once, 64 channels x R
//     rows with a zero column left and right, and the three taps of the filter row read them at addresses shifted by
//     one element - every input element is fetched once per filter row, not once per tap and slab;
//   * eight waves, each 32 oc x 96 columns (three 32x32 blocks): 16 four-byte LDS reads feed 12 matrix instructions, and
//     a slab is 4.5 us of matrix work between two barriers.
// About one workgroup per compute unit; the partial tiles are summed in slice order by a second small kernel
// (deterministic, no float atomics).
#include "conv_side.h"
#include "odl_common.h"

namespace
{
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kNT = 256;
constexpr int kOcTile = 64, kCTile = 64, kCols = 3 * kCTile;
constexpr int kGyRows = 64;                   // rows of a gy2d stage in LDS (a slab has at most this many pixels)
constexpr int kPatchFloats = kCTile * 129;    // the staged input rows: 64 channels x at most 129 floats each
constexpr unsigned kOutside = 0x80000000u;    // beyond every buffer descriptor's size: the load delivers zeros
constexpr int kXV = 8;                        // 16-byte pieces of input one thread stages per slab, at most

struct WgradGeom
{
    const float *x, *gy;
    float *part;  // [slices][tiles][64 oc][192 columns]
    int C, H, W, OC, OH, OW, N;
    int R, KP;          // output rows and output pixels per slab (KP = R*OW, a multiple of 8)
    int slabs;          // ceil(N*OH / R)
    int tiles_oc, tiles_c, tiles;  // tiles = tiles_oc * 3 * tiles_c
    int slices, slabs_per_slice;
    int pitch_r, pitch_c;  // floats per staged input row (W + 2) and per channel (R * pitch_r made odd)
    int rq, cgroup;        // 16-byte pieces of one channel's rows in a slab (R * W/4), and channels staged per pass (256 / rq)
    int xcds;
    unsigned gy_bytes;     // size of the gy buffer
    odl::FastDiv by_oh, by_ow, by_rq, by_q;
};

__device__ inline void load_to_lds_16(i32x4 rsrc, unsigned lds_byte_address, unsigned lane_offset)
{
    asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(lds_byte_address), "v"(lane_offset), "s"(rsrc)
                 : "memory", "m0");
}

#ifdef ODL_WGRAD_DBG
__device__ unsigned long long g_wgrad_dbg[512 * 128];
#define ODL_WGRAD_STAMP(i) do { if (threadIdx.x == 0 && (i) < 128) g_wgrad_dbg[blockIdx.x * 128 + (i)] = wall_clock64(); } while (0)
#else
#define ODL_WGRAD_STAMP(i) do { } while (0)
#endif

template <int N>
__device__ inline void wait_vmcnt()
{
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// STEPS = KP / 8 eight-wide K steps per slab; S = stride. Two workgroups of four waves share a compute unit (65 KB of
// LDS each): the barriers and the patch refill of one are covered by the matrix instructions of the other.
template <int STEPS, int S>
__global__ __launch_bounds__(kNT, 2) void conv_wgrad_rows_kernel(const WgradGeom g)
{
    __shared__ __attribute__((aligned(16))) float gy_s[2][kGyRows * kOcTile];
    __shared__ __attribute__((aligned(16))) float patch[kPatchFloats];
    constexpr int GY_U = kGyRows * kOcTile / 4 / kNT;  // 16-byte pieces of a gy stage per thread: 4

    ODL_WGRAD_STAMP(0);
    const int t = threadIdx.x, lane = t & 63, l32 = lane & 31, lh = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int rb = wave & 1, half = wave >> 1;  // the wave's 32 oc rows and its 96 of the tile's 192 columns

    // workgroup -> (slice, tile): a contiguous band of workgroups per XCD, the tiles of one slice next to each other
    // (they read the same gy2d rows and the same input rows, which then meet in one L2)
    int slice, tile;
    {
        const unsigned total = (unsigned)(g.slices * g.tiles), nx = (unsigned)g.xcds;
        const unsigned loc = blockIdx.x / nx, xcd = blockIdx.x - loc * nx;
        const unsigned full = total / nx, rem = total - full * nx;
        const unsigned v = xcd * full + (xcd < rem ? xcd : rem) + loc;
        slice = (int)(v / (unsigned)g.tiles), tile = (int)(v - (unsigned)slice * (unsigned)g.tiles);
    }
    const int rt = tile % g.tiles_oc, rest = tile / g.tiles_oc;
    const int kh = rest % 3, cb = rest / 3;
    const int slab0 = slice * g.slabs_per_slice;
    int nslab = g.slabs - slab0;
    nslab = nslab < g.slabs_per_slice ? nslab : g.slabs_per_slice;
    nslab = __builtin_amdgcn_readfirstlane(nslab);

    // ---- gy2d: a slab's rows, 64 oc of each, straight into LDS. Piece f of the stage = (row f / 16, 16 bytes f % 16).
    i32x4 rgy;
    {
        const uint64_t p = reinterpret_cast<uint64_t>(g.gy);
        rgy[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)p);
        rgy[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(p >> 32));
        rgy[2] = (int)g.gy_bytes;
        rgy[3] = 0x00020000;
    }
    const unsigned gy_lds = (unsigned)(uintptr_t)(__attribute__((address_space(3))) float *)&gy_s[0][0];
    unsigned gy_off[GY_U];  // byte offset of this thread's pieces inside slab 0 of the batch (kOutside: past the slab)
#pragma unroll
    for (int u = 0; u < GY_U; ++u)
    {
        const int f = t + u * kNT, row = f >> 4, piece = f & 15;
        gy_off[u] = row < g.KP ? (unsigned)((row * g.OC + rt * kOcTile + piece * 4) * 4) : kOutside;
    }
    const unsigned gy_step = (unsigned)(g.KP * g.OC * 4);  // bytes from one slab to the next
    auto issue_gy = [&](int stage, int slab) {
#pragma unroll
        for (int u = 0; u < GY_U; ++u)
        {
            // (rows past the end of the batch lie past the buffer's size and arrive as zeros)
            const unsigned off = gy_off[u] == kOutside ? kOutside : gy_off[u] + (unsigned)slab * gy_step;
            load_to_lds_16(rgy, gy_lds + (unsigned)((stage * kGyRows * kOcTile + (u * kNT + wave * 64) * 4) * 4), off);
        }
    };

    // ---- the input rows of a slab. A thread owns one 16-byte piece (slab row r, piece q of the image row) of every
    // cgroup-th channel from its first one on: all its pieces share the image, the row and the place in the row, and
    // differ by a constant stride in memory and in the patch. The row steps by R output rows per slab.
    const unsigned ch0 = odl::fastdiv((unsigned)t, g.by_rq), rq = (unsigned)t - ch0 * (unsigned)g.rq;
    const unsigned xr_r = odl::fastdiv(rq, g.by_q), xr_q = rq - xr_r * (unsigned)(g.W / 4);
    const bool x_thread = (int)ch0 < g.cgroup;
    const int x_dst = (int)ch0 * g.pitch_c + (int)xr_r * g.pitch_r + 1 + 4 * (int)xr_q;
    const int x_base = ((cb * kCTile + (int)ch0) * g.H) * g.W + 4 * (int)xr_q;
    const int x_dst_step = g.cgroup * g.pitch_c, x_src_step = g.cgroup * g.H * g.W;
    int x_n, x_oh;
    {
        const unsigned orow = (unsigned)(slab0 * g.R) + xr_r;  // the piece's output row in the first slab of this slice
        const unsigned n = odl::fastdiv(orow, g.by_oh);
        x_n = (int)n, x_oh = (int)(orow - n * (unsigned)g.OH);
    }
    f32x4 xr[kXV];
    bool xr_ok = false;
    const int chw = g.C * g.H * g.W;
    // (No branch around the loads: a piece outside the image reads the tensor's first bytes instead and is zeroed when
    // stored. Channels past the tile's 64 are likewise read from a valid place and never stored.)
    auto load_x = [&]() {
        const int ih = S * x_oh + kh - 1;
        xr_ok = x_thread && x_n < g.N && ih >= 0 && ih < g.H;
        const int off = xr_ok ? x_n * chw + ih * g.W + x_base : 0;
#pragma unroll
        for (int u = 0; u < kXV; ++u)
        {
            const bool on = xr_ok && (int)ch0 + u * g.cgroup < kCTile;
            xr[u] = *reinterpret_cast<const f32x4 *>(g.x + (on ? off + u * x_src_step : 0));
        }
        x_oh += g.R;
        if (x_oh >= g.OH)
            x_oh -= g.OH, x_n += 1;
    };
    auto store_x = [&]() {
#pragma unroll
        for (int u = 0; u < kXV; ++u)
            if (x_thread && (int)ch0 + u * g.cgroup < kCTile)
            {
                float *d = patch + x_dst + u * x_dst_step;
                d[0] = xr_ok ? xr[u][0] : 0.f, d[1] = xr_ok ? xr[u][1] : 0.f, d[2] = xr_ok ? xr[u][2] : 0.f,
                d[3] = xr_ok ? xr[u][3] : 0.f;
            }
    };

    // the patch starts out as zeros: its first and last column of every row are never written again
    for (int i = t; i < kPatchFloats; i += kNT)
        patch[i] = 0.f;

    // ---- fragment addresses. A: gy_s[k][32*rb + l32], k = 8*st + 4*lh + s. B: the lane's channel of each of the wave's
    // three blocks, at the slab pixel k's place in the patch: patch[(cc0 + l32)*pitch_c + r(k)*pitch_r + S*ow(k) + kw]
    const float *a_lane = &gy_s[0][0] + (4 * lh) * kOcTile + rb * 32 + l32;
    int b_k[STEPS][4];  // float offset of pixel k in a channel's rows
#pragma unroll
    for (int st = 0; st < STEPS; ++st)
#pragma unroll
        for (int s = 0; s < 4; ++s)
        {
            const unsigned k = (unsigned)(8 * st + 4 * lh + s);
            const unsigned r = odl::fastdiv(k, g.by_ow);
            b_k[st][s] = (int)r * g.pitch_r + S * (int)(k - r * (unsigned)g.OW) + l32 * g.pitch_c;
        }
    int b_blk[3];  // block jb of the wave: tap kw = b / 2 and channels 32*(b % 2).. of the tile, b = 3*half + jb
#pragma unroll
    for (int jb = 0; jb < 3; ++jb)
    {
        const int b = 3 * half + jb;
        b_blk[jb] = __builtin_amdgcn_readfirstlane((b & 1) * 32 * g.pitch_c + (b >> 1));
    }

    f32x16 acc[3];
#pragma unroll
    for (int j = 0; j < 3; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            acc[j][r] = 0.f;

    auto read_frags = [&](const float *as, int st, float (&a)[4], float (&b)[3][4]) {
#pragma unroll
        for (int s = 0; s < 4; ++s)
            a[s] = as[(8 * st + s) * kOcTile];
#pragma unroll
        for (int j = 0; j < 3; ++j)
#pragma unroll
            for (int s = 0; s < 4; ++s)
                b[j][s] = patch[b_k[st][s] + b_blk[j]];
    };

    ODL_WGRAD_STAMP(1);
    // Slab i: gy stage i % 2, and the one patch. Before the first barrier of its iteration a thread has waited for its
    // own gy pieces of the slab (queued an iteration ago); the barrier also says that everybody has read slab i-1, so the
    // patch can be overwritten with slab i's rows (in registers since an iteration ago) and the other gy stage refilled.
    if (nslab > 0)
    {
        issue_gy(0, slab0);
        load_x();
    }
    for (int i = 0; i < nslab; ++i)
    {
        wait_vmcnt<0>();
        __syncthreads();
        ODL_WGRAD_STAMP(2 + 3 * i);
        store_x();
        if (i + 1 < nslab)
        {
            issue_gy((i + 1) & 1, slab0 + i + 1);
            load_x();
        }
        __syncthreads();  // the patch is written, everybody's share of the gy stage has landed
        ODL_WGRAD_STAMP(3 + 3 * i);
        const float *as = a_lane + (i & 1) * (kGyRows * kOcTile);
        float fa[2][4], fb[2][3][4];
        read_frags(as, 0, fa[0], fb[0]);
#pragma unroll
        for (int st = 0; st < STEPS; ++st)
        {
            const int cur = st & 1, nxt = cur ^ 1;
            // the next step's fragments are read while this step's matrix instructions run
            if (st + 1 < STEPS)
                read_frags(as, st + 1, fa[nxt], fb[nxt]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int j = 0; j < 3; ++j)
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cur][s], fb[cur][j][s], acc[j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        ODL_WGRAD_STAMP(4 + 3 * i);
    }
    wait_vmcnt<0>();  // nothing of this workgroup may still be on its way into LDS when the LDS is handed on

    // accumulator register r of lane (l32, lh) holds row 8*(r/4) + 4*lh + r%4 and the lane's column of the block. The
    // partial tile is stored as it is computed, [64 oc][192 columns] (lanes along the columns: whole 128-byte lines);
    // the fold kernel moves the sums to their places in gW.
    float *out = g.part + ((int64_t)slice * g.tiles + tile) * (kOcTile * kCols);
#pragma unroll
    for (int jb = 0; jb < 3; ++jb)
    {
        float *o = out + (rb * 32 + 4 * lh) * kCols + (3 * half + jb) * 32 + l32;
#pragma unroll
        for (int r = 0; r < 16; ++r)
            o[(8 * (r / 4) + (r % 4)) * kCols] = acc[jb][r];
    }
    ODL_WGRAD_STAMP(127);
}

// gW = part[0] + part[1] + ... in slice order (conv_side.h)
__global__ __launch_bounds__(1024) void wgrad_fold_kernel(const odl::SideFold f)
{
    __shared__ f32x4 sums[1024];
    odl::side_fold(f, blockIdx.x, sums);
}

struct RowsPlan
{
    bool ok;
    int R, KP, slices, slabs_per_slice, slabs, tiles;
};

RowsPlan plan_rows(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW,
                   int64_t OH, int64_t OW)
{
    RowsPlan p{};
    if (KH != 3 || KW != 3 || PH != 1 || PW != 1 || SH != SW || (SH != 1 && SH != 2) || C % kCTile != 0 || OC % kOcTile != 0 ||
        W % 4 != 0 || OW < 1 || OW > 64)
        return p;
    // the most output rows per slab whose pixels are a multiple of eight, 32 to 64 of them
    int R = 0;
    for (int r = 1; r * OW <= 64; ++r)
        if ((r * OW) % 8 == 0)
            R = r;
    // (a thread stages one 16-byte piece of a row for up to kXV channels, kNT / (R * W/4) channels per pass)
    if (R == 0 || R > OH || R * OW < 32 || ((R * (W + 2)) | 1) > 129 || R * (W / 4) > kNT ||
        (kNT / (R * (W / 4))) * kXV < kCTile)
        return p;
    const int64_t rows = N * OH, M = rows * OW;
    if (M * OC * 4 >= (1ll << 31) || N * C * H * W * 4 >= (1ll << 31) || rows >= (1ll << 30))
        return p;
    p.R = R, p.KP = R * (int)OW;
    p.slabs = (int)odl::ceil_div(rows, R);
    p.tiles = (int)(OC / kOcTile) * 3 * (int)(C / kCTile);
    // about two workgroups per compute unit, every slice at least four slabs long
    int slices = 2 * odl::device_cus() / p.tiles;
    if (slices > p.slabs / 4)
        slices = p.slabs / 4;
    if (slices < 1)
        return p;
    p.slabs_per_slice = (int)odl::ceil_div(p.slabs, slices);
    p.slices = (int)odl::ceil_div(p.slabs, p.slabs_per_slice);
    // worth it from about a GFLOP on, and when the slices fill at least half the chip
    p.ok = 2 * M * C * 9 * OC >= (1ll << 30) && (int64_t)p.slices * p.tiles >= odl::device_cus();
    return p;
}
}  // namespace

namespace odl
{
bool conv_wgrad_rows_ok(const float *gy, const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH,
                        int KW, int SH, int SW, int PH, int PW, int64_t OH, int64_t OW)
{
    return ((reinterpret_cast<uintptr_t>(gy) | reinterpret_cast<uintptr_t>(x)) & 15) == 0 &&
           plan_rows(N, C, H, W, OC, KH, KW, SH, SW, PH, PW, OH, OW).ok;
}

size_t conv_wgrad_rows_workspace(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW,
                                 int PH, int PW, int64_t OH, int64_t OW)
{
    const RowsPlan p = plan_rows(N, C, H, W, OC, KH, KW, SH, SW, PH, PW, OH, OW);
    return p.ok ? (size_t)p.slices * OC * C * 9 * sizeof(float) : 0;
}

// fold == nullptr: the partial tiles are summed into gw by a launch of this function's own. Otherwise *fold receives that
// job and the caller runs it (side_fold) together with other small jobs.
int conv_wgrad_rows(const float *gy, const float *x, float *gw, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
                    int S, int64_t OH, int64_t OW, void *workspace, size_t workspace_bytes, hipStream_t st, SideFold *fold)
{
    const RowsPlan p = plan_rows(N, C, H, W, OC, 3, 3, S, S, 1, 1, OH, OW);
    if (!p.ok)
        return fail(ODL_ERR_RUNTIME, "conv2d_backward: the row-walking weight gradient does not take this shape");
    const size_t need = (size_t)p.slices * OC * C * 9 * sizeof(float);
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= need && reinterpret_cast<uintptr_t>(workspace) % 16 == 0,
                "conv2d_backward: a 16-byte aligned workspace of %zu bytes required, got %zu", need, workspace_bytes);
    WgradGeom g{};
    g.x = x, g.gy = gy, g.part = static_cast<float *>(workspace);
    g.C = (int)C, g.H = (int)H, g.W = (int)W, g.OC = (int)OC, g.OH = (int)OH, g.OW = (int)OW;
    g.N = (int)N, g.R = p.R, g.KP = p.KP, g.slabs = p.slabs;
    g.tiles_oc = (int)(OC / kOcTile), g.tiles_c = (int)(C / kCTile), g.tiles = p.tiles;
    g.slices = p.slices, g.slabs_per_slice = p.slabs_per_slice;
    g.pitch_r = (int)W + 2, g.pitch_c = (p.R * ((int)W + 2)) | 1;
    g.rq = p.R * (int)(W / 4), g.cgroup = kNT / g.rq;
    g.xcds = chip().xcds;
    g.gy_bytes = (unsigned)(N * OH * OW * OC * 4);
    g.by_oh = make_fastdiv((unsigned)OH), g.by_ow = make_fastdiv((unsigned)OW);
    g.by_rq = make_fastdiv((unsigned)g.rq), g.by_q = make_fastdiv((unsigned)(W / 4));
    const dim3 grid((unsigned)(p.slices * p.tiles)), block(kNT);
    const int steps = p.KP / 8;
#define ODL_WGRAD_CASE(ST)                                                                      \
    if (steps == ST)                                                                            \
    {                                                                                           \
        if (S == 1)                                                                             \
            hipLaunchKernelGGL((conv_wgrad_rows_kernel<ST, 1>), grid, block, 0, st, g);         \
        else                                                                                    \
            hipLaunchKernelGGL((conv_wgrad_rows_kernel<ST, 2>), grid, block, 0, st, g);         \
    }
    ODL_WGRAD_CASE(4)
    ODL_WGRAD_CASE(5)
    ODL_WGRAD_CASE(6)
    ODL_WGRAD_CASE(7)
    ODL_WGRAD_CASE(8)
#undef ODL_WGRAD_CASE
    ODL_LAUNCH_CHECK();
    const SideFold f{g.part, gw, p.slices, (int)(OC * C * 9 / 4), g.tiles_oc, (int)(C * 9)};
    if (fold)
    {
        *fold = f;
        return ODL_OK;
    }
    hipLaunchKernelGGL(wgrad_fold_kernel, dim3((unsigned)ceil_div(f.n4, 256)), dim3(1024), 0, st, f);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}
}  // namespace odl
