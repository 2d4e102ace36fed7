// FP32 GEMM on v_mfma_f32_32x32x2_f32 whose operands travel from global memory into LDS without passing through
// registers (buffer_load ... lds, 16 bytes per lane), four K slabs deep.
//
// Why. With operands staged through registers, every K slab costs the wait for its loads plus the LDS stores in front
// of the barrier, and the staging instructions compete with the matrix instructions for issue slots. A workgroup that is
// alone on its compute unit idles the matrix pipe through all of that (1024x1024x4096: 99 us with staging, 72 us with the
// staging taken out as an experiment, 73 us here); on launches of many tiles the difference is 82 -> 88 % of the matrix
// peak at 4096^3. Here a slab's loads are queued three slabs ahead and land in LDS on their own; a wave only waits for
// loads that were queued three barriers ago, then reads its fragments and issues its matrix instructions.
//
//   * 512 threads: KSETS sets of waves share one tile (2 sets of four waves on square tiles, 4 sets of two waves on the
//     64x32 tile); of the 8-wide K steps of a slab each set multiplies every KSETS-th one, and the other sets'
//     accumulators join the first's through LDS before the epilogue, added in set order.
//   * LDS holds the operand tiles exactly as the loads deliver them: lane i of a wave's load lands at base + 16*i.
//       K-contiguous operand (A of A.B, B of A.B^T): tile [rows][BK], a row's 16-byte pieces permuted by
//         piece ^ swizzle(row) — chosen on the global side, so that the 8 rows one ds_read_b128 phase touches fall into
//         8 different bank groups although the rows are not padded;
//       row-contiguous operand (A of A^T.B, B of A.B): tile [BK][cols], read back with ds_read_b32, lanes along cols.
//   * Rows, columns and K positions outside the matrix: the lane's offset is set past the buffer's size and the load
//     delivers zeros, so ragged edges need no separate code.
//   * Instances: 128x128x16 at two workgroups per compute unit (many tiles; a short last round as K pieces), 128x128x32,
//     64x64x32 and 64x32x64 at one (few tiles), 64x64x32 at two (batches of small products: 1x1 convolutions).
#include "gemm_dma.h"
#include "odl_common.h"
#include "reduce_small.h"

namespace
{
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kNT     = 512;
constexpr int kEpiBiasCol = 1, kEpiBiasRow = 2;
template <int V>
struct IntTag  // a compile-time integer passed to a generic lambda
{
    static constexpr int value = V;
};
// calls f(IntTag<bias kind>, IntTag<activation>) for the launch's epilogue: bias kind 0 none (and no activation), 1 by
// column, 2 by row; the activation 0 none, 1 relu, 2 silu
template <typename F>
__device__ inline void with_epilogue_kind(int bias_kind, int act, F &&f)
{
    if (bias_kind == 0)
        f(IntTag<0>{}, IntTag<0>{});
    else if (bias_kind == 1)
    {
        if (act == 1)
            f(IntTag<1>{}, IntTag<1>{});
        else if (act == 2)
            f(IntTag<1>{}, IntTag<2>{});
        else
            f(IntTag<1>{}, IntTag<0>{});
    }
    else
    {
        if (act == 1)
            f(IntTag<2>{}, IntTag<1>{});
        else if (act == 2)
            f(IntTag<2>{}, IntTag<2>{});
        else
            f(IntTag<2>{}, IntTag<0>{});
    }
}
constexpr unsigned kOutside = 0x80000000u;  // beyond the 2^31 - 1 bytes every buffer descriptor here declares

// What the workgroup -> tile mapping divides by, as multiply-and-shift constants worked out by the launcher: done with
// the machine's integer division (a reciprocal on the vector unit and a trip back to the scalar one, six times) the
// mapping was a fifth of the 1 us a workgroup spends before its first load, which a 13 us product notices.
struct DmaTileMap
{
    odl::FastDiv by_xcds, by_nt, by_gsz, by_gm_last;
    unsigned xcds, xcd_full, xcd_rem;  // XCDs, workgroups every XCD gets, and how many XCDs get one more
};

// tiles in groups of 8 tile-rows; inside a group down the rows first
__device__ inline void tile_coords(unsigned t, int tiles_m, int tiles_n, const DmaTileMap &map, int &tm, int &tn)
{
    const unsigned gsz = 8u * (unsigned)tiles_n;
    const unsigned grp = odl::fastdiv(t, map.by_gsz), in_g = t - grp * gsz;
    const int first_m = (int)grp * 8;
    if (tiles_m - first_m >= 8)
        tm = first_m + (int)(in_g & 7u), tn = (int)(in_g >> 3);
    else
    {
        const unsigned gm = (unsigned)(tiles_m - first_m), q = odl::fastdiv(in_g, map.by_gm_last);
        tm = first_m + (int)(in_g - q * gm), tn = (int)q;
    }
}

typedef int i32x4 __attribute__((ext_vector_type(4)));

// One 16-byte load per lane from a buffer into LDS: lane i's data lands at lds_byte_address + 16*i. Written as an
// instruction rather than through the compiler's builtin: the compiler cannot tell which stage a queued load writes
// and would wait for ALL queued loads before every LDS read, which is exactly the wait this kernel exists to avoid.
// The waits are placed by hand (wait_vmcnt below). The LDS address travels in M0, which nothing else here uses.
__device__ inline void load_to_lds_16(i32x4 rsrc, unsigned lds_byte_address, unsigned lane_offset)
{
    asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(lds_byte_address), "v"(lane_offset), "s"(rsrc)
                 : "memory", "m0");
}

__device__ inline i32x4 buffer_of(const float *base)
{
    const uint64_t p = reinterpret_cast<uint64_t>(base);
    i32x4 r;
    // (the address is the same in every lane; readfirstlane tells the compiler so, and the descriptor stays in SGPRs)
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)p);
    r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(p >> 32));  // stride 0: a raw buffer
    r[2] = 0x7fffffff;                                          // bytes; offsets at or past it deliver zeros
    r[3] = 0x00020000;
    return r;
}

// s_waitcnt that only waits for the vector-memory counter to drop to n (gfx9 encoding: vmcnt in bits 3:0 and 15:14)
template <int N>
__device__ inline void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// which 16-byte slot of its LDS row a K-contiguous row's piece goes to: piece ^ swizzle(row). Eight consecutive rows,
// read 16 bytes each at the same piece, must fall into eight different bank groups: rows that share a 128-byte line of
// LDS (8/PIECES of them) get the same value, consecutive lines different ones.
template <int PIECES>
__device__ inline int swizzle(int row)
{
    return PIECES >= 8 ? (row & (PIECES - 1)) : ((row / (8 / PIECES)) & (PIECES - 1));
}

// KSETS wave sets share a tile: the eight waves are WAVES_N columns x (8 / KSETS / WAVES_N) rows of wave tiles, times
// KSETS sets that each multiply every KSETS-th 8-wide K step (2 sets for square tiles; 4 sets on a 64x32 tile, whose
// two 32x32 blocks could not occupy eight waves otherwise).
// The whole product of one workgroup. `bid` is the workgroup's number inside its product (a launch may hold two
// products, below); As / Bs are the LDS stages, kStages x BM*BK and kStages x BN*BK floats.
template <int BM, int BN, int BK, bool TA, bool TB, int KSETS, int kStages>
__device__ __forceinline__ void sgemm_dma_body(const odl::DmaGemmArgs &g, const DmaTileMap &map, const unsigned bid,
                                               float *const As0, float *const Bs0)
{
    constexpr bool A_KMAJOR = !TA, B_KMAJOR = TB;
    constexpr int PIECES = BK / 4;                       // 16-byte pieces in a K-contiguous row of a slab
    constexpr int A_U = BM * BK / 4 / kNT, B_U = BN * BK / 4 / kNT;  // loads per thread and slab
    static_assert((BM * BK / 4) % kNT == 0 && (BN * BK / 4) % kNT == 0 && (PIECES & (PIECES - 1)) == 0, "tile shape");
    constexpr int PER_SLAB = A_U + B_U;
    // Row-contiguous B on a 128-wide tile: a wave takes the whole tile width, and lane l32 of its four column blocks owns
    // the four ADJACENT columns 4*l32 .. 4*l32+3 (block j = column 4*l32 + j). One 16-byte LDS read of a K row then feeds
    // the four blocks' matrix instructions of one K pair, where the plain layout (block j = columns 32*j + l32) needs a
    // 4-byte read per block and K value; the output leaves in 16-byte stores as well.
    constexpr bool QUADB = !B_KMAJOR && BN == 128 && BM == 128 && KSETS == 2;
    constexpr int WAVES_N = QUADB ? 1 : (KSETS == 2 ? 2 : 1), WAVES_M = 8 / KSETS / WAVES_N;
    constexpr int RB = BM / WAVES_M / 32, CB = BN / WAVES_N / 32;  // 32x32 blocks per wave
    constexpr int STEPS = BK / 8 / KSETS;                          // 8-wide K steps per wave and slab
    static_assert(RB >= 1 && CB >= 1 && STEPS >= 1 && RB * WAVES_M * 32 == BM && CB * WAVES_N * 32 == BN, "wave layout");
    auto As = [&](int stage) { return As0 + stage * (BM * BK); };
    auto Bs = [&](int stage) { return Bs0 + stage * (BN * BK); };
    static_assert(kStages * BM * BK >= (KSETS - 1) * (8 / KSETS) * 16 * 64, "the A buffers hold one accumulator block of every wave of the other sets");

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave8 = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr int TILE_WAVES = 8 / KSETS;
    const int wave = wave8 % TILE_WAVES, kset = wave8 / TILE_WAVES;
    const int l32 = lane & 31, lh = lane >> 5;
    const int wm = (wave / WAVES_N) * (BM / WAVES_M), wn = (wave % WAVES_N) * (BN / WAVES_N);

    // workgroup -> (K slice, tile): a contiguous band of workgroups per XCD, tiles in groups of 8 tile-rows
    int tm, tn, kz = 0, bz = 0;
    int64_t kbeg, kend;
    float *tail_out = nullptr;
    {
        const unsigned nt = (unsigned)(g.tiles_m * g.tiles_n);
        unsigned t;
        if (g.tail_splits > 0 && (int)bid >= g.main_blocks)
        {
            // pieces of the tail tiles keep the hardware's round-robin order: they are short and should spread over all XCDs
            const int u = (int)bid - g.main_blocks;
            const int ti = u / g.tail_splits, piece = u - ti * g.tail_splits;
            t = (unsigned)(g.tail_first + ti);
            kbeg = (int64_t)piece * g.tail_kps;
            kend = (kbeg + g.tail_kps < g.K) ? kbeg + g.tail_kps : g.K;
            tail_out = g.tail_ws + (int64_t)u * (BM * BN);
        }
        else
        {
            const unsigned nx = map.xcds;
            const unsigned loc = odl::fastdiv(bid, map.by_xcds), xcd = bid - loc * nx;
            unsigned v = xcd * map.xcd_full + (xcd < map.xcd_rem ? xcd : map.xcd_rem) + loc;
            if (g.batch > 1)
            {
                bz = (int)odl::fastdiv(v, map.by_nt);  // one K slice per product when there are several
                v -= (unsigned)bz * nt;
            }
            kz = (int)odl::fastdiv(v, map.by_nt);
            t = v - (unsigned)kz * nt;
            kbeg = (int64_t)kz * g.k_per_split;
            kend = (kbeg + g.k_per_split < g.K) ? kbeg + g.k_per_split : g.K;
        }
        tile_coords(t, g.tiles_m, g.tiles_n, map, tm, tn);
    }
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    const int nkt = __builtin_amdgcn_readfirstlane((int)((kend - kbeg + BK - 1) / BK));
    const int klen = (int)(kend - kbeg);

    // buffer descriptors based at this workgroup's corner of each operand; every lane offset is relative to it
    const float *abase = g.A + (int64_t)bz * g.a_batch + (A_KMAJOR ? m0 * g.lda + kbeg : kbeg * g.lda + m0);
    const float *bbase = g.B + (int64_t)bz * g.b_batch + (B_KMAJOR ? n0 * g.ldb + kbeg : kbeg * g.ldb + n0);
    const i32x4 ra = buffer_of(abase), rb = buffer_of(bbase);
    const unsigned as_lds = (unsigned)(uintptr_t)(__attribute__((address_space(3))) float *)As0;
    const unsigned bs_lds = (unsigned)(uintptr_t)(__attribute__((address_space(3))) float *)Bs0;

    // per load of this thread: byte offset inside slab 0, the K position it covers inside a slab, and whether its row
    // (or column quad) is inside the matrix
    unsigned a_off[A_U], b_off[B_U];
    int a_k[A_U], b_k[B_U];
    bool a_in[A_U], b_in[B_U];
#pragma unroll
    for (int u = 0; u < A_U; ++u)
    {
        const int f = tid + u * kNT;
        if (A_KMAJOR)
        {
            const int row = f / PIECES, piece = (f % PIECES) ^ swizzle<PIECES>(row);
            a_off[u] = (unsigned)((row * g.lda + 4 * piece) * 4), a_k[u] = 4 * piece, a_in[u] = m0 + row < g.M;
        }
        else
        {
            const int k = f / (BM / 4), c4 = f % (BM / 4);
            a_off[u] = (unsigned)((k * g.lda + 4 * c4) * 4), a_k[u] = k, a_in[u] = m0 + 4 * c4 < g.M;
        }
    }
#pragma unroll
    for (int u = 0; u < B_U; ++u)
    {
        const int f = tid + u * kNT;
        if (B_KMAJOR)
        {
            const int row = f / PIECES, piece = (f % PIECES) ^ swizzle<PIECES>(row);
            b_off[u] = (unsigned)((row * g.ldb + 4 * piece) * 4), b_k[u] = 4 * piece, b_in[u] = n0 + row < g.N;
        }
        else
        {
            const int k = f / (BN / 4), c4 = f % (BN / 4);
            b_off[u] = (unsigned)((k * g.ldb + 4 * c4) * 4), b_k[u] = k, b_in[u] = n0 + 4 * c4 < g.N;
        }
    }
    const unsigned a_step = (unsigned)((A_KMAJOR ? (int64_t)BK : (int64_t)BK * g.lda) * 4);
    const unsigned b_step = (unsigned)((B_KMAJOR ? (int64_t)BK : (int64_t)BK * g.ldb) * 4);

    // queue the loads of slab kt into a stage (slabs past the end deliver zeros into a stage nobody reads: the count of
    // loads in flight stays the same for every slab, which is what the waits below rely on)
    auto issue = [&](int stage, int kt) {
        const int k0 = kt * BK;
#pragma unroll
        for (int u = 0; u < A_U; ++u)
        {
            const bool ok = a_in[u] && k0 + a_k[u] < klen;
            load_to_lds_16(ra, as_lds + (unsigned)((stage * BM * BK + (u * kNT + wave8 * 64) * 4) * 4),
                           ok ? a_off[u] + (unsigned)kt * a_step : kOutside);
        }
#pragma unroll
        for (int u = 0; u < B_U; ++u)
        {
            const bool ok = b_in[u] && k0 + b_k[u] < klen;
            load_to_lds_16(rb, bs_lds + (unsigned)((stage * BN * BK + (u * kNT + wave8 * 64) * 4) * 4),
                           ok ? b_off[u] + (unsigned)kt * b_step : kOutside);
        }
    };

    f32x16 acc[RB][CB];
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int j = 0; j < CB; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0.f;

    // one 8-wide K step of this wave's set: its fragments from LDS (four K values per lane and block), then its matrix
    // instructions
    auto read_frags = [&](const float *as, const float *bs, int st, float (&a)[RB][4], float (&b)[CB][4]) {
        const int ks = KSETS * st + kset;
#pragma unroll
        for (int i = 0; i < RB; ++i)
        {
            const int r = wm + i * 32 + l32;
            if (A_KMAJOR)
            {
                const f32x4 v = *reinterpret_cast<const f32x4 *>(as + (r * PIECES + ((2 * ks + lh) ^ swizzle<PIECES>(r))) * 4);
                a[i][0] = v[0], a[i][1] = v[1], a[i][2] = v[2], a[i][3] = v[3];
            }
            else
            {
#pragma unroll
                for (int s = 0; s < 4; ++s)
                    a[i][s] = as[(ks * 8 + 4 * lh + s) * BM + r];
            }
        }
#pragma unroll
        for (int j = 0; j < CB; ++j)
        {
            const int c = wn + j * 32 + l32;
            if (B_KMAJOR)
            {
                const f32x4 v = *reinterpret_cast<const f32x4 *>(bs + (c * PIECES + ((2 * ks + lh) ^ swizzle<PIECES>(c))) * 4);
                b[j][0] = v[0], b[j][1] = v[1], b[j][2] = v[2], b[j][3] = v[3];
            }
            else if (!QUADB)
            {
#pragma unroll
                for (int s = 0; s < 4; ++s)
                    b[j][s] = bs[(ks * 8 + 4 * lh + s) * BN + c];
            }
        }
        if (QUADB)
        {
#pragma unroll
            for (int s = 0; s < 4; ++s)
            {
                const f32x4 v = *reinterpret_cast<const f32x4 *>(bs + (ks * 8 + 4 * lh + s) * BN + 4 * l32);
#pragma unroll
                for (int j = 0; j < CB; ++j)
                    b[j][s] = v[j % 4];
            }
        }
    };
    auto mfma_part = [&](const float (&a)[RB][4], const float (&b)[CB][4], int s0, int s1) {
#pragma unroll
        for (int s = s0; s < s1; ++s)
#pragma unroll
            for (int i = 0; i < RB; ++i)
#pragma unroll
                for (int j = 0; j < CB; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][s], b[j][s], acc[i][j], 0, 0, 0);
    };

    // Slabs 0..2 are on their way before the loop.
#pragma unroll
    for (int s = 0; s < kStages - 1; ++s)
        issue(s, s);
    float fa[2][RB][4], fb[2][CB][4];
    // Both operands K-contiguous (two 16-byte LDS reads per block and step): the fragments of the next K step are read
    // while the matrix instructions of the current one run — the first half of a step's instructions is issued, then (when
    // the next step opens a new slab) the wait for that slab, the barrier and the queueing of the slab four ahead, then the
    // reads of the next fragments, then the second half, so neither the barrier nor the LDS latency leaves the matrix pipe
    // idle (4096^3 dA = dC.B^T: 994 -> 955 us). With a row-contiguous operand the same order measured slower than reading
    // right after the barrier (4-byte reads: NN 1005 -> 1047 us, TN 992 -> 1026 us) or no faster (B in 16-byte quads: the
    // second fragment set takes the kernel past 128 registers and with that to one workgroup per compute unit; held to
    // 128 registers it runs 969 against 972 us): those keep the plain order.
    // (On the 64-row tiles, whose waves hold one block each, the order also pays with a row-contiguous B — 1024^3 22.0
    // -> 21.3 us, 6272x256x1152 41.2 -> 40.2 us against the plain order on one box — but not with a row-contiguous A.)
    constexpr bool PIPE = A_KMAJOR && (B_KMAJOR || BM <= 64);
    if constexpr (PIPE)
    {
        if (nkt > 0)
        {
            wait_vmcnt<(kStages - 2) * PER_SLAB>();
            __syncthreads();
            issue(kStages - 1, kStages - 1);
            read_frags(As(0), Bs(0), 0, fa[0], fb[0]);
        }
        // all K steps of slab j, which lies in stage s; `more`: a slab follows it
        auto slab = [&](int s, int j, bool more) {
#pragma unroll
            for (int st = 0; st < STEPS; ++st)
            {
                const int cur = (s * STEPS + st) & 1, nxt = cur ^ 1;  // kStages * STEPS is even: the parity carries over
                // (the scheduling fences keep the order written here: left alone, the compiler sinks the reads below
                // all sixteen matrix instructions and waits for them at once)
                mfma_part(fa[cur], fb[cur], 0, 2);
                __builtin_amdgcn_sched_barrier(0);
                if (st + 1 < STEPS)
                    read_frags(As(s), Bs(s), st + 1, fa[nxt], fb[nxt]);
                else
                {
                    if (more)
                    {
                        wait_vmcnt<(kStages - 2) * PER_SLAB>();  // this thread's loads of slab j+1 have landed
                        __syncthreads();                         // ... and everybody else's; slab j has been read by all
                        issue(s, j + kStages);
                    }
                    // (read without a condition: after the last slab the values are never used, and a read inside a
                    // branch would have to be waited for at the branch's end)
                    read_frags(As((s + 1) % kStages), Bs((s + 1) % kStages), 0, fa[nxt], fb[nxt]);
                }
                __builtin_amdgcn_sched_barrier(0);
                mfma_part(fa[cur], fb[cur], 2, 4);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        // rounds of four slabs that all have a successor run as straight-line code; the last one to four test as they go
        int kt = 0;
        for (; kt + kStages < nkt; kt += kStages)
        {
#pragma unroll
            for (int s = 0; s < kStages; ++s)
                slab(s, kt + s, true);
        }
#pragma unroll
        for (int s = 0; s < kStages; ++s)
            if (kt + s < nkt)
                slab(s, kt + s, kt + s + 1 < nkt);
    }
    else
    {
        // in the loop, slab kt's loads were queued three barriers ago
        for (int kt = 0; kt < nkt; kt += kStages)
        {
#pragma unroll
            for (int s = 0; s < kStages; ++s)
            {
                if (kt + s < nkt)
                {
                    wait_vmcnt<(kStages - 2) * PER_SLAB>();  // this thread's loads of slab kt+s have landed
                    __syncthreads();                         // ... and everybody else's; slab kt+s-1 has been read by all
                    issue((s + kStages - 1) % kStages, kt + s + kStages - 1);
#pragma unroll
                    for (int st = 0; st < STEPS; ++st)
                    {
                        read_frags(As(s), Bs(s), st, fa[0], fb[0]);
                        mfma_part(fa[0], fb[0], 0, 4);
                    }
                }
            }
        }
    }
    wait_vmcnt<0>();  // the zero-filled slabs past the end are still landing in the stages
    __syncthreads();

    // the other wave sets hand their accumulators to the first, one 32x32 block of each wave at a time; the first adds
    // them in set order
    {
        float *xch = As0 + (wave * 16) * 64 + lane;
        constexpr int SET_STRIDE = TILE_WAVES * 16 * 64;
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
            for (int j = 0; j < CB; ++j)
            {
                if (kset > 0)
                {
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        xch[(kset - 1) * SET_STRIDE + r * 64] = acc[i][j][r];
                }
                __syncthreads();
                if (kset == 0)
                {
#pragma unroll
                    for (int z = 0; z < KSETS - 1; ++z)
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            acc[i][j][r] += xch[z * SET_STRIDE + r * 64];
                }
                __syncthreads();
            }
        if (kset > 0)
            return;
    }

    // accumulator register r of lane (l32, lh) holds row 8*(r/4) + 4*lh + r%4 and the lane's column of block j
    if constexpr (QUADB)
    {
        // the lane's four blocks are four adjacent columns: one 16-byte store per row where the row's base allows
        const int64_t col0 = n0 + 4 * l32;
        float *Cout = tail_out ? tail_out : g.C + (int64_t)kz * g.c_split_stride + (int64_t)bz * g.c_batch;
        const int64_t ld = tail_out ? BN : g.ldc, cbase = tail_out ? 4 * l32 : col0;
        const int64_t rbase = tail_out ? 0 : m0;
        const bool whole = (reinterpret_cast<uintptr_t>(Cout) & 15) == 0 && (tail_out || (col0 + 3 < g.N && g.ldc % 4 == 0));
        // (the kind of epilogue decided once per launch, as for the plain layout below)
        auto store_rows = [&](auto bias_tag, auto act_tag) {
            constexpr int BIAS = decltype(bias_tag)::value, ACT = decltype(act_tag)::value;
            float bcol[4] = {0.f, 0.f, 0.f, 0.f};
            if (BIAS == 1)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    bcol[e] = col0 + e < g.N ? g.bias[col0 + e] : 0.f;
            const bool row_bias = BIAS == 2 && g.bias != nullptr;
#pragma unroll
            for (int i = 0; i < RB; ++i)
            {
                const int64_t row0 = rbase + wm + i * 32 + 4 * lh;
                const int rows_left = tail_out ? 32 : (int)(g.M - row0 < 32 ? g.M - row0 : 32);
                float *out = Cout + row0 * ld + cbase;
#pragma unroll
                for (int r = 0; r < 16; ++r)
                {
                    const int dr = 8 * (r / 4) + (r % 4);
                    if (dr >= rows_left)
                        continue;
                    f32x4 v = {acc[i][0][r], acc[i][1][r], acc[i][2][r], acc[i][3][r]};
                    if (BIAS == 1)
                    {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            v[e] = odl::apply_act(v[e] + bcol[e], ACT);
                    }
                    else if (BIAS == 2)
                    {
                        const float br = row_bias ? g.bias[row0 + dr] : 0.f;
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            v[e] = odl::apply_act(row_bias ? v[e] + br : v[e], ACT);
                    }
                    if (whole)
                        *reinterpret_cast<f32x4 *>(out + (int64_t)dr * ld) = v;
                    else
                    {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (tail_out || col0 + e < g.N)
                                out[(int64_t)dr * ld + e] = v[e];
                    }
                }
            }
        };
        const int bias_kind = tail_out ? 0 : (g.epi == kEpiBiasCol && g.bias != nullptr) ? 1 : (g.epi == kEpiBiasRow ? 2 : 0);
        with_epilogue_kind(bias_kind, g.act, store_rows);
        return;
    }
    if (tail_out)
    {
        // K piece of a tail tile: the whole BM x BN partial, tile-local (rows or columns past the matrix hold zeros)
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
            for (int j = 0; j < CB; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    tail_out[(wm + i * 32 + 8 * (r / 4) + 4 * lh + (r % 4)) * BN + wn + j * 32 + l32] = acc[i][j][r];
        return;
    }
    float *Cout = g.C + (int64_t)kz * g.c_split_stride + (int64_t)bz * g.c_batch;
    // The kind of epilogue is the same for the whole launch: it is decided once, outside the sixteen-element loops, whose
    // bodies are then an addition, the activation as a constant, and a store (with the tests inside, a 64x32 tile spent
    // 1.7 us of a 13 us product here). BIAS: 0 none (a column bias that is absent also means no activation), 1 by
    // column, 2 by row (an absent row bias still applies the activation). With c_p > 0 the product's columns are
    // (image, position) pairs of an NCHW tensor of M channels: rows are then c_p elements apart, the bias goes by row.
    auto store_blocks = [&](auto bias_tag, auto act_tag) {
        constexpr int BIAS = decltype(bias_tag)::value, ACT = decltype(act_tag)::value;
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
            for (int j = 0; j < CB; ++j)
            {
                const int64_t col = n0 + wn + j * 32 + l32;
                if (col >= g.N)
                    continue;
                const int64_t row0 = m0 + wm + i * 32 + 4 * lh;
                const int rows_left = (int)(g.M - row0 < 32 ? g.M - row0 : 32);  // rows from row0 on inside the matrix
                int64_t stride = g.ldc;
                float *out = Cout + row0 * g.ldc + col;
                if (g.c_p > 0)
                {
                    const int64_t img = (int64_t)((unsigned)col / (unsigned)g.c_p), pos = col - img * g.c_p;
                    stride = g.c_p, out = Cout + (img * g.M + row0) * g.c_p + pos;
                }
                const float bcol = BIAS == 1 ? g.bias[col] : 0.f;
                const bool row_bias = BIAS == 2 && g.bias != nullptr;
#pragma unroll
                for (int r = 0; r < 16; ++r)
                {
                    const int dr = 8 * (r / 4) + (r % 4);
                    if (dr >= rows_left)
                        continue;
                    float v = acc[i][j][r];
                    if (BIAS == 1)
                        v = odl::apply_act(v + bcol, ACT);
                    else if (BIAS == 2)
                        v = odl::apply_act(row_bias ? v + g.bias[row0 + dr] : v, ACT);
                    out[(int64_t)dr * stride] = v;
                }
            }
    };
    const int bias_kind = g.c_p > 0 ? 2 : (g.epi == kEpiBiasCol && g.bias != nullptr) ? 1 : (g.epi == kEpiBiasRow ? 2 : 0);
    with_epilogue_kind(bias_kind, g.act, store_blocks);
}

template <int BM, int BN, int BK, bool TA, bool TB, int WGS_PER_CU, int KSETS = 2, int kStages = 4>
// (The second launch bound counts waves per SIMD, of which a workgroup of 512 threads brings two: WGS_PER_CU there only
// keeps the register budget generous — the kernels use under 128 registers and fit two workgroups per compute unit
// anyway. Bounds of 2 * WGS_PER_CU changed the compiler's schedule for the worse: 2048^3 dA = dC.B^T 133 -> 142 us.)
__global__ __launch_bounds__(kNT, WGS_PER_CU) void sgemm_dma_kernel(const odl::DmaGemmArgs g, const DmaTileMap map)
{
    __shared__ __attribute__((aligned(16))) float As[kStages * BM * BK];
    __shared__ __attribute__((aligned(16))) float Bs[kStages * BN * BK];
    sgemm_dma_body<BM, BN, BK, TA, TB, KSETS, kStages>(g, map, blockIdx.x, As, Bs);
}

// Two independent products in one launch: workgroups [0, first) run product 0 = X.Y^T, the others product 1 = X^T.Y —
// the two gradients of a matrix product (gx = gy.w^T, gw = x^T.gy), each on its own tile shape. Two workgroups, one of
// each product as a rule, share a compute unit: the prologue, barriers and epilogue of one are covered by the matrix
// instructions of the other, and the second launch's start-up is gone. Same tile code as the single launches, so the
// same bits.
template <int BM0, int BN0, int BK0, int KSETS0, int ST0, int BM1, int BN1, int BK1, int KSETS1, int ST1>
__global__ __launch_bounds__(kNT, 2) void sgemm_dma_pair_kernel(const odl::DmaGemmArgs g0, const DmaTileMap map0,
                                                                const odl::DmaGemmArgs g1, const DmaTileMap map1,
                                                                const unsigned first, const unsigned first_padded,
                                                                const unsigned n1, const odl::ColSumJob sums)
{
    constexpr int F0 = ST0 * (BM0 + BN0) * BK0, F1 = ST1 * (BM1 + BN1) * BK1;
    static_assert(F0 * 4 <= 80 * 1024 && F1 * 4 <= 80 * 1024, "two workgroups must fit the LDS of a compute unit");
    __shared__ __attribute__((aligned(16))) float stages[F0 > F1 ? F0 : F1];
    const unsigned bid = blockIdx.x;
    if (bid < first)
        sgemm_dma_body<BM0, BN0, BK0, false, true, KSETS0, ST0>(g0, map0, bid, stages, stages + ST0 * BM0 * BK0);
    else if (bid >= first_padded)  // (the gap keeps product 1's workgroup numbers congruent to the XCD they run on)
    {
        if (bid - first_padded < n1)
            sgemm_dma_body<BM1, BN1, BK1, true, false, KSETS1, ST1>(g1, map1, bid - first_padded, stages, stages + ST1 * BM1 * BK1);
        else
        {
            // the column sum that rides along (the first 256 threads run reduce_small.h's two halves: the bits of the
            // launch of its own)
            const unsigned bx = bid - first_padded - n1, tid = threadIdx.x;
            if (sums.quads)
            {
                auto &sh = *reinterpret_cast<typename odl::ColSumSmall<4, 8>::Sums *>(stages);
                if (tid < 256)
                    odl::ColSumSmall<4, 8>::accumulate(sums.src, sums.axis, sums.inner, bx, 0, tid, sh);
                __syncthreads();
                if (tid < 256)
                    odl::ColSumSmall<4, 8>::finish(sums.dst, sums.inner, bx, 0, tid, sh);
            }
            else
            {
                auto &sh = *reinterpret_cast<typename odl::ColSumSmall<1, 16>::Sums *>(stages);
                if (tid < 256)
                    odl::ColSumSmall<1, 16>::accumulate(sums.src, sums.axis, sums.inner, bx, 0, tid, sh);
                __syncthreads();
                if (tid < 256)
                    odl::ColSumSmall<1, 16>::finish(sums.dst, sums.inner, bx, 0, tid, sh);
            }
        }
    }
}
}  // namespace

namespace odl
{
bool sgemm_dma_fits(bool ta, bool tb, const DmaGemmArgs &g)
{
    const bool aligned = ((reinterpret_cast<uintptr_t>(g.A) | reinterpret_cast<uintptr_t>(g.B)) % 16 == 0) &&
                         g.lda % 4 == 0 && g.ldb % 4 == 0 && (ta ? g.M : g.K) % 4 == 0 && (tb ? g.K : g.N) % 4 == 0 &&
                         (g.splits == 1 || g.k_per_split % 32 == 0) && (g.tail_splits == 0 || g.tail_kps % 16 == 0);
    // lane offsets are 32-bit and must stay below 2^31: the rows of a tile, or the K range of a slice, times the row length
    const int64_t a_span = (ta ? g.k_per_split + 64 : 128) * g.lda * 4, b_span = (tb ? 128 : g.k_per_split + 64) * g.ldb * 4;
    return aligned && a_span < (1ll << 31) && b_span < (1ll << 31) && g.M > 0 && g.N > 0 && g.K > 0;
}

static DmaTileMap tile_map_of(const DmaGemmArgs &g)
{
    DmaTileMap map;
    const int64_t nt = (int64_t)g.tiles_m * g.tiles_n;
    const unsigned total = (unsigned)(g.tail_splits > 0 ? g.main_blocks : nt * g.splits * (g.batch > 1 ? g.batch : 1));
    const unsigned nx = (unsigned)(g.xcds > 0 ? g.xcds : 1);
    map.by_xcds = make_fastdiv(nx), map.by_nt = make_fastdiv((unsigned)nt);
    map.by_gsz = make_fastdiv(8u * (unsigned)g.tiles_n);
    map.by_gm_last = make_fastdiv((unsigned)(g.tiles_m % 8 ? g.tiles_m % 8 : 8));
    map.xcds = nx, map.xcd_full = total / nx, map.xcd_rem = total % nx;
    return map;
}

int sgemm_dma_pair_launch(int tile0, const DmaGemmArgs &g0, int tile1, const DmaGemmArgs &g1, hipStream_t st,
                          const ColSumJob *sums)
{
    if (g0.splits != 1 || g1.splits != 1 || g0.tail_splits > 0 || g1.tail_splits > 0 || g0.batch > 1 || g1.batch > 1 ||
        g0.c_p > 0 || g1.c_p > 0)
        return fail(ODL_ERR_RUNTIME, "sgemm: a pair launch takes two whole, unbatched products");
    const unsigned n0 = (unsigned)(g0.tiles_m * g0.tiles_n), n1 = (unsigned)(g1.tiles_m * g1.tiles_n);
    const unsigned nx = (unsigned)(g0.xcds > 0 ? g0.xcds : 1), n0p = (n0 + nx - 1) / nx * nx;
    const DmaTileMap m0 = tile_map_of(g0), m1 = tile_map_of(g1);
    const ColSumJob job = sums ? *sums : ColSumJob{};
    const dim3 grid(n0p + n1 + job.blocks), block(kNT);
    // per class: tile rows, tile columns, slab width, wave sets, stages (two workgroups of 64 to 72 KB per compute unit)
#define ODL_PAIR_64 64, 64, 32, 2, 4
#define ODL_PAIR_32 64, 32, 64, 4, 3
#define ODL_PAIR_128 128, 128, 16, 2, 4
#define ODL_PAIR_CASE(T0, C0, T1, C1)                                                                                   \
    if (tile0 == T0 && tile1 == T1)                                                                                     \
    {                                                                                                                   \
        hipLaunchKernelGGL((sgemm_dma_pair_kernel<C0, C1>), grid, block, 0, st, g0, m0, g1, m1, n0, n0p, n1, job);      \
        return ODL_OK;                                                                                                  \
    }
    ODL_PAIR_CASE(64, ODL_PAIR_64, 64, ODL_PAIR_64)
    ODL_PAIR_CASE(64, ODL_PAIR_64, 32, ODL_PAIR_32)
    ODL_PAIR_CASE(32, ODL_PAIR_32, 64, ODL_PAIR_64)
    ODL_PAIR_CASE(32, ODL_PAIR_32, 32, ODL_PAIR_32)
    ODL_PAIR_CASE(128, ODL_PAIR_128, 128, ODL_PAIR_128)
#undef ODL_PAIR_CASE
#undef ODL_PAIR_64
#undef ODL_PAIR_32
#undef ODL_PAIR_128
    return fail(ODL_ERR_RUNTIME, "sgemm: no pair kernel for tile classes %d and %d", tile0, tile1);
}

int sgemm_dma_launch(int tile, bool ta, bool tb, const DmaGemmArgs &g, hipStream_t st)
{
    if (g.c_p > 0 && !(tile == 64 || tile == 65 || tile == 32))
        return fail(ODL_ERR_RUNTIME, "sgemm: the NCHW output exists for the 64-wide tiles only");
    const int64_t nt = (int64_t)g.tiles_m * g.tiles_n;
    const dim3 grid((unsigned)(g.tail_splits > 0 ? g.main_blocks + (nt - g.tail_first) * g.tail_splits
                                                 : nt * g.splits * (g.batch > 1 ? g.batch : 1))),
        block(kNT);
    const DmaTileMap map = tile_map_of(g);
#define ODL_DMA_CASE(TA, TB)                                                                          \
    if (ta == TA && tb == TB)                                                                         \
    {                                                                                                 \
        if (tile == 64)                                                                               \
            hipLaunchKernelGGL((sgemm_dma_kernel<64, 64, 32, TA, TB, 1, 2, 4>), grid, block, 0, st, g, map); \
        else if (tile == 65)                                                                          \
            hipLaunchKernelGGL((sgemm_dma_kernel<64, 64, 32, TA, TB, 2>), grid, block, 0, st, g, map);     \
        else if (tile == 32)                                                                          \
            hipLaunchKernelGGL((sgemm_dma_kernel<64, 32, 64, TA, TB, 1, 4, 4>), grid, block, 0, st, g, map); \
        else if (tile == 128)                                                                         \
            hipLaunchKernelGGL((sgemm_dma_kernel<128, 128, 32, TA, TB, 1>), grid, block, 0, st, g, map);   \
        else                                                                                          \
            hipLaunchKernelGGL((sgemm_dma_kernel<128, 128, 16, TA, TB, 2>), grid, block, 0, st, g, map);   \
        return ODL_OK;                                                                                \
    }
    ODL_DMA_CASE(false, false)
    ODL_DMA_CASE(false, true)
    ODL_DMA_CASE(true, false)
    ODL_DMA_CASE(true, true)
#undef ODL_DMA_CASE
    return ODL_ERR_RUNTIME;
}

bool conv1x1_dma_ok(const float *x, const float *w, int64_t N, int64_t C, int64_t HW, int64_t OC)
{
    return N >= 1 && N < 65536 && C >= 4 && C % 4 == 0 && HW >= 4 && HW % 4 == 0 && OC >= 1 &&
           ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) % 16 == 0) &&
           (C + 64) * HW * 4 < (1ll << 31) && 128 * C * 4 < (1ll << 31) &&
           ceil_div(OC, 64) * ceil_div(HW, 32) * N < (1ll << 31);
}

int conv1x1_dma(const float *x, const float *w, const float *b, float *y, int64_t N, int64_t C, int64_t HW, int64_t OC,
                int act, hipStream_t st)
{
    DmaGemmArgs g{};
    g.A = w, g.B = x, g.bias = b, g.C = y;
    g.M = OC, g.N = HW, g.K = C, g.lda = C, g.ldb = HW, g.ldc = HW;
    g.splits = 1, g.k_per_split = ceil_div(C, 64) * 64, g.c_split_stride = 0;
    g.epi = 2, g.act = act, g.xcds = chip().xcds;
    g.tail_splits = 0, g.main_blocks = 0, g.tail_kps = 0, g.tail_ws = nullptr;
    g.batch = (int)N, g.a_batch = 0, g.b_batch = C * HW, g.c_batch = OC * HW;
    // 64x64 tiles when they occupy the chip (two workgroups per compute unit once there are more than the chip holds
    // singly), 64x32 tiles for the small images
    const int64_t t64 = ceil_div(OC, 64) * ceil_div(HW, 64) * N, cus = device_cus();
    int tile = t64 >= cus / 2 ? (t64 > cus + cus / 4 ? 65 : 64) : 32;
    g.tiles_m = (int)ceil_div(OC, 64), g.tiles_n = (int)ceil_div(HW, tile == 32 ? 32 : 64);
    g.tail_first = g.tiles_m * g.tiles_n;
    return sgemm_dma_launch(tile, false, false, g, st);
}
}  // namespace odl
