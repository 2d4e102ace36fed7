// FP32 GEMM for gfx950 on the matrix cores (v_mfma_f32_32x32x2_f32), hand-written.
//
// C[M,N] = op(A)[M,K] . op(B)[K,N], row-major, all four transpose combinations, so that the backward
// products dA = dC.B^T (NT) and dB = A^T.dC (TN) read their operands in place — the reference materialises
// both transposes first (src/operators/math/mat_mul.cpp:171-174).
//
// Shape of the kernel (wave64, 256 threads = 4 waves in a 2x2 grid):
//   * workgroup tile BM x BN x BK, wave tile (BM/2) x (BN/2) made of 32x32 MFMA blocks whose accumulators
//     stay in registers for the whole K loop;
//   * each operand tile is staged through LDS in the layout its global layout suggests, so the global->LDS
//     copy is always a 16-byte load and a 16-byte store with no transposition:
//       K-contiguous in memory  -> LDS [row][BK+4]  (fragment = one ds_read_b128 per lane),
//       row-contiguous in memory -> LDS [k][rows+4] (fragment = four conflict-free ds_read_b32);
//     both layouts give lane (i = lane%32, h = lane/32) the four values k = 4h..4h+3 of its row, and MFMA
//     step s multiplies the k = {s, 4+s} pair — the K order inside a tile is permuted, which a sum allows;
//   * two LDS buffers and register prefetch of the next K slab: one barrier per slab;
//   * workgroup -> tile mapping that keeps each XCD (one L2 each, workgroups are dealt round-robin over the
//     8 XCDs) on a contiguous band of tiles, walked in groups of 8 tile-rows so A and B panels are reused
//     from that XCD's L2;
//   * split-K (grid.y) writes partial tiles that a second kernel sums in slice order — deterministic.
#include "gemm_dma.h"
#include "odl_common.h"
#include "reduce_small.h"

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace odl
{
// gemm_skinny.hip: products whose output has at most 16 columns (a classifier layer), on the vector ALUs
bool skinny_ok(int64_t M, int64_t N, int64_t K);
int skinny_forward(const float *x, const float *w, const float *bias, float *y, int64_t M, int64_t N, int64_t K, int64_t ldx,
                   int64_t ldw, int64_t ldy, int act, hipStream_t st);
bool skinny_bias_ok(int64_t M, int64_t N);
int skinny_backward(const float *x, const float *w, const float *gy, float *gx, float *gw, float *gb, int64_t M, int64_t K,
                    int64_t N, hipStream_t st);
}  // namespace odl

namespace
{
constexpr int kThreads = 256;

inline bool aligned16(const void *p)
{
    return reinterpret_cast<uintptr_t>(p) % 16 == 0;
}
constexpr int kGroupM  = 8;

enum : int
{
    EPI_PLAIN     = 0,  // C[row*ldc + col]
    EPI_BIAS_COL  = 1,  // + bias[col]
    EPI_NCHW_ROWB = 2,  // conv forward: row = oc, col = n*P + p -> y[(n*OC + oc)*P + p] (+ bias[oc])
};

// Where the B operand comes from. Besides a plain matrix it can be gathered on the fly from an NCHW image
// (the im2col matrix is then never materialised) or from the upstream gradient of a convolution.
enum : int
{
    SB_PLAIN       = 0,
    SB_CONV_FWD    = 1,  // B(row = output pixel m, k = (c,kh,kw)) = x[n, c, oh*SH-PH+kh, ow*SW-PW+kw]      (forward)
    SB_CONV_WGRAD  = 2,  // B(k = output pixel m, row = (c,kh,kw)) = same element                            (weight grad)
    SB_CONV_DGRAD  = 3,  // B(row = input pixel q, k = (kh,kw,oc)) = gy2d[(n, h+PH-kh, w+PW-kw), oc], stride 1 (input grad)
    SB_CONV_FWD_TAP = 4,  // the forward operand with K ordered (kh,kw,c), C a multiple of 16: a slab of 16 k is one tap
};

using odl::FastDiv;
using odl::fastdiv;
using odl::make_fastdiv;

struct ConvSrc
{
    int C, H, W, OH, OW, OC;
    int KH, KW, SH, SW, PH, PW;
    FastDiv by_ow, by_oh;  // output pixel number -> (n, oh, ow)
    FastDiv by_w, by_h;    // input pixel number -> (n, h, w)
    FastDiv by_cslabs;     // K slab number -> (tap, channel slab) for the tap-ordered forward gather (C / 16 slabs a tap)
};

struct GemmArgs
{
    const float *A;
    const float *B;
    float *C;
    const float *bias;
    int64_t M, N, K;
    int64_t lda, ldb, ldc;
    int64_t k_per_split;     // K range of one grid.y slice (multiple of BK)
    int64_t c_split_stride;  // elements between the partial outputs of consecutive slices (0 = none)
    int64_t P;               // EPI_NCHW_ROWB: OH*OW
    int act;                 // EPI_NCHW_ROWB, EPI_BIAS_COL: activation applied after the bias (0 none, 1 relu, 2 silu)
    int tiles_m, tiles_n;
    int splits;              // K slices (grid = tiles_m * tiles_n * splits workgroups)
    int xcds;                // XCDs of the device: consecutive workgroup ids are dealt round-robin over them
    // Tail split (splits == 1 only): when the tile count is a little over a multiple of the CU count, the last
    // `nt - tail_first` tiles would run alone after everything else. They are cut into tail_splits K pieces
    // each — workgroups main_blocks.. — which write tile-local partials to tail_ws; tail_fixup_kernel sums them.
    int main_blocks, tail_first, tail_splits;
    int64_t tail_kps;
    float *tail_ws;
};

using odl::apply_act;

template <int V>
struct ActTag  // the activation as a compile-time value for a generic lambda
{
    static constexpr int value = V;
};

__device__ __host__ inline void tile_coords(int t, int tiles_m, int tiles_n, int &tm, int &tn)
{
    const int gsz = 8 * tiles_n;  // groups of 8 tile-rows
    const int grp = t / gsz, in_g = t % gsz;
    const int first_m = grp * 8;
    const int gm = (tiles_m - first_m) < 8 ? (tiles_m - first_m) : 8;
    tm = first_m + in_g % gm;
    tn = in_g / gm;
}

// WS = 2: the workgroup has a second set of four waves on the same tile. Both sets stage the operands together; of the
// 8-wide K steps of a slab each set multiplies every other one, and the second set's accumulators join the first's
// through LDS before the epilogue. For products with at most one workgroup per compute unit: a lone set of four waves
// (one per SIMD) leaves the matrix pipe idle whenever it waits for LDS, memory or the barrier; the second set fills
// those gaps without changing the tile shape.
template <int BM, int BN, int BK, bool TA, bool TB, bool VEC, int EPI, int SB = SB_PLAIN, int CK = 0, int WS = 1, bool PF2 = false>
__global__ __launch_bounds__(kThreads * WS, (WS == 1 && BM * BN >= 128 * 128 && VEC && SB != SB_CONV_WGRAD ? (PF2 ? 3 : 4) : 1)) void sgemm_mfma_kernel(GemmArgs g, ConvSrc cv)
{
    constexpr int NT = kThreads * WS;
    static_assert(WS == 1 || (WS == 2 && SB == SB_PLAIN && VEC && (BK / 8) % 2 == 0), "the second wave set: plain operands only");
    // A tile: !TA -> memory is [M][K] (K-contiguous) -> LDS K-major; TA -> memory [K][M] -> LDS row-major.
    // B tile: !TB -> memory is [K][N] (row-contiguous) -> LDS row-major; TB -> memory [N][K] -> LDS K-major.
    // A gathered B is laid out in LDS the way its gather runs: the forward gather has lanes along the pixels
    // (rows of B) -> row-major; the weight-grad gather has lanes along the pixels (K of B) and the input-grad
    // gather reads 16 bytes along oc (K of B) -> K-major.
    constexpr bool A_KMAJOR = !TA;
    constexpr bool B_KMAJOR = (SB == SB_PLAIN) ? TB : (SB != SB_CONV_FWD && SB != SB_CONV_FWD_TAP);
    static_assert(SB != SB_CONV_FWD_TAP || CK > 0, "the tap-ordered gather keeps its bounds as a per-lane tap mask");
    static_assert(SB == SB_PLAIN || BN == 128, "the gather mappings assume 128 B rows per tile");
    constexpr int LDA_S     = A_KMAJOR ? (BK + 4) : (BM + 4);
    constexpr int LDB_S     = B_KMAJOR ? (BK + 4) : (BN + 4);
    constexpr int A_SIZE    = A_KMAJOR ? BM * LDA_S : BK * LDA_S;
    constexpr int B_SIZE    = B_KMAJOR ? BN * LDB_S : BK * LDB_S;
    constexpr int WM = BM / 2, WN = BN / 2;  // wave tile
    constexpr int RB = WM / 32, CB = WN / 32;
    constexpr int A_PER_T = BM * BK / NT;  // floats staged per thread
    constexpr int B_PER_T = BN * BK / NT;
    static_assert(BK % 8 == 0 && A_PER_T % 4 == 0 && B_PER_T % 4 == 0, "tile shape");

    __shared__ __attribute__((aligned(16))) float As[2][A_SIZE];
    __shared__ __attribute__((aligned(16))) float Bs[2][B_SIZE];
    // (the second wave set's accumulators pass through the A buffers at the end)
    static_assert(WS == 1 || 2 * A_SIZE >= 4 * 16 * 64, "the A buffers hold one accumulator block of four waves");

    const int tid  = threadIdx.x;
    const int lane = tid & 63, wave = WS > 1 ? ((tid >> 6) & 3) : (tid >> 6), kset = WS > 1 ? (tid >> 8) : 0;  // kset: which wave set (0 when WS == 1)
    const int l32 = lane & 31, lh = lane >> 5;
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;

    // ---- workgroup -> (K slice, tile). The grid is one-dimensional (tiles x slices). Workgroups are dealt
    // round-robin over the 8 XCDs, so the id is first unfolded into a contiguous band per XCD; inside a band the
    // tiles of one K slice are adjacent (they read the same K range of A and B, which then sits in that XCD's L2),
    // and tiles are walked in groups of kGroupM tile-rows.
    int tm, tn, kz = 0;
    int64_t kbeg, kend;
    float *tail_out = nullptr;
    {
        const int nt = g.tiles_m * g.tiles_n;
        int t;
        if (g.tail_splits > 0 && (int)blockIdx.x >= g.main_blocks)
        {
            // tail pieces keep the hardware's round-robin order: they are short and should spread over all XCDs
            const int u = (int)blockIdx.x - g.main_blocks;
            const int ti = u / g.tail_splits, piece = u - ti * g.tail_splits;
            t = g.tail_first + ti;
            kbeg = (int64_t)piece * g.tail_kps;
            kend = (kbeg + g.tail_kps < g.K) ? kbeg + g.tail_kps : g.K;
            tail_out = g.tail_ws + (int64_t)u * (BM * BN);
        }
        else
        {
            // (the workgroup count of a launch is below 2^31: 32-bit arithmetic)
            const unsigned total = g.tail_splits > 0 ? (unsigned)g.main_blocks : (unsigned)nt * (unsigned)g.splits;
            const unsigned bid = blockIdx.x, nx = (unsigned)g.xcds;
            const unsigned loc = bid / nx, xcd = bid - loc * nx;
            const unsigned full = total / nx, rem = total - full * nx;
            const unsigned v = xcd * full + (xcd < rem ? xcd : rem) + loc;
            kz = (int)(v / (unsigned)nt);
            t = (int)(v - (unsigned)kz * (unsigned)nt);
            kbeg = (int64_t)kz * g.k_per_split;
            kend = (kbeg + g.k_per_split < g.K) ? kbeg + g.k_per_split : g.K;
        }
        tile_coords(t, g.tiles_m, g.tiles_n, tm, tn);
    }
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    const int nkt = (int)((kend - kbeg + BK - 1) / BK);

    float ra[A_PER_T], rb_main[B_PER_T];

    auto load_tile = [&](const float *__restrict__ src, int64_t ld, bool kmajor, int64_t row0, int64_t rows,
                         int64_t k0, int brows, float *regs, int per_t) {
        // kmajor: memory [rows][K]; else memory [K][rows]. `brows` = BM or BN.
        if (VEC)
        {
            for (int u = 0; u < per_t / 4; ++u)
            {
                const int f = tid + u * NT;
                int64_t r, k;
                if (kmajor)
                {
                    r = row0 + f / (BK / 4);
                    k = k0 + 4 * (f % (BK / 4));
                }
                else
                {
                    k = k0 + f / (brows / 4);
                    r = row0 + 4 * (f % (brows / 4));
                }
                f32x4 v = {0.f, 0.f, 0.f, 0.f};
                if (r < rows && k < kend)
                    v = *reinterpret_cast<const f32x4 *>(src + (kmajor ? r * ld + k : k * ld + r));
                regs[4 * u + 0] = v[0];
                regs[4 * u + 1] = v[1];
                regs[4 * u + 2] = v[2];
                regs[4 * u + 3] = v[3];
            }
        }
        else
        {
            for (int u = 0; u < per_t; ++u)
            {
                const int e = tid + u * NT;
                int64_t r, k;
                if (kmajor)
                {
                    r = row0 + e / BK;
                    k = k0 + e % BK;
                }
                else
                {
                    k = k0 + e / brows;
                    r = row0 + e % brows;
                }
                regs[u] = (r < rows && k < kend) ? src[kmajor ? r * ld + k : k * ld + r] : 0.f;
            }
        }
    };

    auto store_tile = [&](float *lds, int lds_ld, bool kmajor, int brows, const float *regs, int per_t) {
        if (VEC)
        {
            for (int u = 0; u < per_t / 4; ++u)
            {
                const int f = tid + u * NT;
                int off;
                if (kmajor)
                    off = (f / (BK / 4)) * lds_ld + 4 * (f % (BK / 4));
                else
                    off = (f / (brows / 4)) * lds_ld + 4 * (f % (brows / 4));
                f32x4 v = {regs[4 * u], regs[4 * u + 1], regs[4 * u + 2], regs[4 * u + 3]};
                *reinterpret_cast<f32x4 *>(lds + off) = v;
            }
        }
        else
        {
            for (int u = 0; u < per_t; ++u)
            {
                const int e = tid + u * NT;
                const int off = kmajor ? (e / BK) * lds_ld + e % BK : (e / brows) * lds_ld + e % brows;
                lds[off] = regs[u];
            }
        }
    };

    // ---- gathered B operands: per-thread state that does not change along K
    const int KH = CK > 0 ? CK : cv.KH, KW = CK > 0 ? CK : cv.KW;
    const int KHW = KH * KW;
    [[maybe_unused]] const float *fw_base = nullptr;  // forward: &x[n, 0, oh*SH-PH, ow*SW-PW] of this thread's pixel
    [[maybe_unused]] int fw_hb = 0, fw_wb = 0;
    [[maybe_unused]] bool fw_live = false;
    [[maybe_unused]] unsigned fw_mask = 0;
    [[maybe_unused]] unsigned fw_voff = 0;  // tap-ordered forward: byte offset of x[n, 0, oh*SH, ow*SW]
    [[maybe_unused]] int wg_off[B_PER_T];  // weight grad: this thread's 8 (c,kh,kw) as offsets into an image ...
    [[maybe_unused]] int wg_kh[CK > 0 ? 1 : B_PER_T], wg_kw[CK > 0 ? 1 : B_PER_T];  // ... and as taps (any kernel size)
    [[maybe_unused]] unsigned wg_taps = 0;  // ... or as eight 4-bit tap numbers kh*KW+kw (3x3, 1x1; 15 = no such row)
    [[maybe_unused]] int dg_n[2], dg_h[2], dg_w[2];                        // input grad: this thread's 2 pixels
    [[maybe_unused]] bool dg_live[2];
    if constexpr (SB == SB_CONV_FWD || SB == SB_CONV_FWD_TAP)
    {
        const int64_t m = n0 + (tid & (BN - 1));
        fw_live = m < g.N;
        const unsigned mm = fw_live ? (unsigned)m : 0u;  // the pixel count is below 2^31
        const unsigned q = fastdiv(mm, cv.by_ow);
        const int64_t n = fastdiv(q, cv.by_oh);
        const int ow = (int)(mm - q * (unsigned)cv.OW), oh = (int)(q - (unsigned)n * (unsigned)cv.OH);
        fw_hb = oh * cv.SH - cv.PH, fw_wb = ow * cv.SW - cv.PW;
        fw_base = g.B + n * cv.C * cv.H * cv.W + (int64_t)fw_hb * cv.W + fw_wb;  // dereferenced only when in bounds
        fw_voff = (unsigned)(((n * cv.C * cv.H + oh * cv.SH) * cv.W + ow * cv.SW) * 4);  // the image is under 4 GiB
        if constexpr (CK > 0)
        {
            // bit kh*KW+kw: that tap of this thread's pixel lies inside the image
            for (int kh = 0; kh < CK; ++kh)
                for (int kw = 0; kw < CK; ++kw)
                    if (fw_live && (unsigned)(fw_hb + kh) < (unsigned)cv.H && (unsigned)(fw_wb + kw) < (unsigned)cv.W)
                        fw_mask |= 1u << (kh * CK + kw);
        }
    }
    if constexpr (SB == SB_CONV_WGRAD)
    {
#pragma unroll
        for (int u = 0; u < B_PER_T; ++u)
        {
            const int64_t ck = n0 + (tid >> 4) + 16 * u;
            const bool ok = ck < g.N;
            const int cki = ok ? (int)ck : 0;
            const int c = cki / KHW, r = cki - c * KHW;
            const int kh = r / KW, kw = r - kh * KW;
            wg_off[u] = (c * cv.H + kh) * cv.W + kw;
            if constexpr (CK > 0)
                wg_taps |= (ok ? (unsigned)r : 15u) << (4 * u);
            else
            {
                wg_kh[u] = ok ? kh : (1 << 20);  // an out-of-range row fails every bounds check
                wg_kw[u] = kw;
            }
        }
    }
    if constexpr (SB == SB_CONV_DGRAD)
    {
#pragma unroll
        for (int u = 0; u < 2; ++u)
        {
            const int64_t q = n0 + (tid >> 2) + 64 * u;
            dg_live[u] = q < g.N;
            const unsigned qq = dg_live[u] ? (unsigned)q : 0u;  // the pixel count is below 2^31
            const unsigned row = fastdiv(qq, cv.by_w), img = fastdiv(row, cv.by_h);
            dg_w[u] = (int)(qq - row * (unsigned)cv.W);
            dg_h[u] = (int)(row - img * (unsigned)cv.H);
            dg_n[u] = (int)img;
        }
    }

    auto load_b = [&](int64_t k0, float *rb_) {
        if constexpr (SB == SB_PLAIN)
        {
            load_tile(g.B, g.ldb, B_KMAJOR, n0, g.N, k0, BN, rb_, B_PER_T);
        }
        else if constexpr (SB == SB_CONV_FWD)
        {
            // element u of this thread: row = tid % 128 (its pixel), k = k0 + tid/128 + 2u  (wave-uniform)
            const int ksub = __builtin_amdgcn_readfirstlane(tid >> 7);
#pragma unroll
            for (int u = 0; u < B_PER_T; ++u)
            {
                const int k = (int)k0 + ksub + 2 * u;
                const int c = k / KHW, r = k - c * KHW;
                const int kh = r / KW, kw = r - kh * KW;
                bool ok;
                if constexpr (CK > 0)
                    ok = ((fw_mask >> r) & 1u) != 0 && k < kend;
                else
                {
                    const int h = fw_hb + kh, w = fw_wb + kw;
                    ok = fw_live && k < kend && (unsigned)h < (unsigned)cv.H && (unsigned)w < (unsigned)cv.W;
                }
                rb_[u] = ok ? fw_base[(c * cv.H + kh) * cv.W + kw] : 0.f;
            }
        }
        else if constexpr (SB == SB_CONV_FWD_TAP)
        {
            // element u: row = tid % 128 (its pixel), k = k0 + tid/128 + 2u. The slab k0..k0+15 is one tap (kh,kw)
            // and 16 consecutive channels, so the bounds test is one bit of the lane's tap mask for the whole slab
            // and every address is a block-uniform base (channel plane + tap, minus the padding) plus the lane's
            // constant pixel offset.
            const int ksub = __builtin_amdgcn_readfirstlane(tid >> 7);
            const int slab = __builtin_amdgcn_readfirstlane((int)(k0 / BK));
            const int tap = (int)fastdiv((unsigned)slab, cv.by_cslabs), c0 = (slab - tap * (cv.C / BK)) * BK + ksub;
            const int kh = tap / CK, kw = tap - kh * CK;
            const int64_t plane = (int64_t)cv.H * cv.W;
            const char *sb = reinterpret_cast<const char *>(g.B) +
                             (c0 * plane + (int64_t)(kh - cv.PH) * cv.W + (kw - cv.PW)) * (int64_t)sizeof(float);
#pragma unroll
            for (int u = 0; u < B_PER_T; ++u)
                rb_[u] = 0.f;
            if (((fw_mask >> tap) & 1u) != 0)
            {
#pragma unroll
                for (int u = 0; u < B_PER_T; ++u)
                    rb_[u] = *reinterpret_cast<const float *>(sb + (int64_t)u * 2 * plane * (int64_t)sizeof(float) + fw_voff);
            }
        }
        else if constexpr (SB == SB_CONV_WGRAD)
        {
            // element u: k = k0 + tid % 16 (its pixel for this slab), row = tid/16 + 16u
            // (the pixel count is below 2^31, so the pixel number and its decomposition stay in 32 bits)
            const unsigned m = (unsigned)k0 + (unsigned)(tid & 15);
            const bool live = m < (unsigned)kend;
            const unsigned mm = live ? m : 0u;
            const unsigned q = fastdiv(mm, cv.by_ow), n = fastdiv(q, cv.by_oh);
            const int ow = (int)(mm - q * (unsigned)cv.OW), oh = (int)(q - n * (unsigned)cv.OH);
            const int hb = oh * cv.SH - cv.PH, wb = ow * cv.SW - cv.PW;
            const float *base = g.B + (int64_t)n * (cv.C * cv.H * cv.W) + (hb * cv.W + wb);
            if constexpr (CK > 0)
            {
                // bit kh*CK+kw of pm: that tap of this slab's pixel lies inside the image
                unsigned colm = 0, pm = 0;
#pragma unroll
                for (int kw = 0; kw < CK; ++kw)
                    colm |= ((unsigned)(wb + kw) < (unsigned)cv.W ? 1u : 0u) << kw;
#pragma unroll
                for (int kh = 0; kh < CK; ++kh)
                    pm |= ((unsigned)(hb + kh) < (unsigned)cv.H ? colm : 0u) << (kh * CK);
                pm = live ? pm : 0u;
#pragma unroll
                for (int u = 0; u < B_PER_T; ++u)
                {
                    const bool ok = ((pm >> ((wg_taps >> (4 * u)) & 15u)) & 1u) != 0;
                    rb_[u] = ok ? base[wg_off[u]] : 0.f;
                }
            }
            else
            {
#pragma unroll
                for (int u = 0; u < B_PER_T; ++u)
                {
                    const int h = hb + wg_kh[u], w = wb + wg_kw[u];
                    const bool ok = live && (unsigned)h < (unsigned)cv.H && (unsigned)w < (unsigned)cv.W;
                    rb_[u] = ok ? base[wg_off[u]] : 0.f;
                }
            }
        }
        else
        {
            // float4 u: row = tid/4 + 64u (its pixel), k = k0 + 4*(tid%4) .. +3 = four consecutive oc of one tap.
            // K runs as (oc slab of 16, tap, oc within the slab): the KH*KW taps of one 64-byte slab follow each
            // other, and neighbouring pixels' taps re-read the same gy rows, so those reads hit in cache.
            const int slab = (int)(k0 / BK);  // block-uniform
            const int ocs = slab / KHW, tap = slab - ocs * KHW;
            const int oc0 = ocs * BK + 4 * (tid & 3);
            const int kh = tap / KW, kw = tap - kh * KW;
#pragma unroll
            for (int u = 0; u < 2; ++u)
            {
                const int oh = dg_h[u] + cv.PH - kh, ow = dg_w[u] + cv.PW - kw;
                const bool ok = dg_live[u] && k0 < kend && (unsigned)oh < (unsigned)cv.OH && (unsigned)ow < (unsigned)cv.OW;
                f32x4 v = {0.f, 0.f, 0.f, 0.f};
                if (ok)
                    v = *reinterpret_cast<const f32x4 *>(g.B + (((int64_t)dg_n[u] * cv.OH + oh) * cv.OW + ow) * cv.OC + oc0);
                rb_[4 * u] = v[0], rb_[4 * u + 1] = v[1], rb_[4 * u + 2] = v[2], rb_[4 * u + 3] = v[3];
            }
        }
    };

    auto store_b = [&](float *lds, const float *rb_) {
        if constexpr (SB == SB_PLAIN)
        {
            store_tile(lds, LDB_S, B_KMAJOR, BN, rb_, B_PER_T);
        }
        else if constexpr (SB == SB_CONV_FWD || SB == SB_CONV_FWD_TAP)
        {
            const int ksub = tid >> 7;
#pragma unroll
            for (int u = 0; u < B_PER_T; ++u)
                lds[(ksub + 2 * u) * LDB_S + (tid & (BN - 1))] = rb_[u];
        }
        else if constexpr (SB == SB_CONV_WGRAD)
        {
#pragma unroll
            for (int u = 0; u < B_PER_T; ++u)
                lds[((tid >> 4) + 16 * u) * LDB_S + (tid & 15)] = rb_[u];
        }
        else
        {
#pragma unroll
            for (int u = 0; u < 2; ++u)
            {
                f32x4 v = {rb_[4 * u], rb_[4 * u + 1], rb_[4 * u + 2], rb_[4 * u + 3]};
                *reinterpret_cast<f32x4 *>(lds + ((tid >> 2) + 64 * u) * LDB_S + 4 * (tid & 3)) = v;
            }
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

    if (nkt > 0)
    {
        load_tile(g.A, g.lda, A_KMAJOR, m0, g.M, kbeg, BM, ra, A_PER_T);
        load_b(kbeg, rb_main);
        store_tile(As[0], LDA_S, A_KMAJOR, BM, ra, A_PER_T);
        store_b(Bs[0], rb_main);
    }
    __syncthreads();

    // the matrix instructions of one K slab out of LDS
    auto mma = [&](const float *as, const float *bs) {
#pragma unroll
        for (int ks0 = 0; ks0 < BK / 8; ks0 += WS)
        {
            const int ks = ks0 + (WS > 1 ? kset : 0);
            float a[RB][4], b[CB][4];
#pragma unroll
            for (int i = 0; i < RB; ++i)
            {
                if (A_KMAJOR)
                {
                    const f32x4 v =
                        *reinterpret_cast<const f32x4 *>(as + (wm + i * 32 + l32) * LDA_S + ks * 8 + 4 * lh);
                    a[i][0] = v[0], a[i][1] = v[1], a[i][2] = v[2], a[i][3] = v[3];
                }
                else
                {
#pragma unroll
                    for (int s = 0; s < 4; ++s)
                        a[i][s] = as[(ks * 8 + 4 * lh + s) * LDA_S + wm + i * 32 + l32];
                }
            }
#pragma unroll
            for (int j = 0; j < CB; ++j)
            {
                if (B_KMAJOR)
                {
                    const f32x4 v =
                        *reinterpret_cast<const f32x4 *>(bs + (wn + j * 32 + l32) * LDB_S + ks * 8 + 4 * lh);
                    b[j][0] = v[0], b[j][1] = v[1], b[j][2] = v[2], b[j][3] = v[3];
                }
                else
                {
#pragma unroll
                    for (int s = 0; s < 4; ++s)
                        b[j][s] = bs[(ks * 8 + 4 * lh + s) * LDB_S + wn + j * 32 + l32];
                }
            }
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int i = 0; i < RB; ++i)
#pragma unroll
                    for (int j = 0; j < CB; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][s], b[j][s], acc[i][j], 0, 0, 0);
        }
    };

    if constexpr (WS > 1 || PF2)
    {
        // One workgroup per compute unit has nobody to cover its memory latency, and a K slab's worth of matrix
        // instructions (0.85 us) is shorter than a load's round trip: operands are fetched TWO slabs ahead into two
        // register sets, so that each load has two slab times to land before it is stored to LDS. The gathered
        // convolution operands, whose loads wait longer still, can ask for the same (PF2).
        float ra2[A_PER_T], rb2[B_PER_T];
        if (nkt > 1)
        {
            load_tile(g.A, g.lda, A_KMAJOR, m0, g.M, kbeg + BK, BM, ra2, A_PER_T);
            load_b(kbeg + BK, rb2);
        }
        for (int kt = 0; kt < nkt; kt += 2)
        {
            if (kt + 2 < nkt)
            {
                const int64_t k0 = kbeg + (int64_t)(kt + 2) * BK;
                load_tile(g.A, g.lda, A_KMAJOR, m0, g.M, k0, BM, ra, A_PER_T);
                load_b(k0, rb_main);
            }
            mma(As[0], Bs[0]);
            if (kt + 1 < nkt)
            {
                store_tile(As[1], LDA_S, A_KMAJOR, BM, ra2, A_PER_T);
                store_b(Bs[1], rb2);
            }
            __syncthreads();
            if (kt + 1 >= nkt)
                break;
            if (kt + 3 < nkt)
            {
                const int64_t k0 = kbeg + (int64_t)(kt + 3) * BK;
                load_tile(g.A, g.lda, A_KMAJOR, m0, g.M, k0, BM, ra2, A_PER_T);
                load_b(k0, rb2);
            }
            mma(As[1], Bs[1]);
            if (kt + 2 < nkt)
            {
                store_tile(As[0], LDA_S, A_KMAJOR, BM, ra, A_PER_T);
                store_b(Bs[0], rb_main);
            }
            __syncthreads();
        }
    }
    else
    {
        for (int kt = 0; kt < nkt; ++kt)
        {
            const int cur = kt & 1;
            if (kt + 1 < nkt)
            {
                const int64_t k0 = kbeg + (int64_t)(kt + 1) * BK;
                load_tile(g.A, g.lda, A_KMAJOR, m0, g.M, k0, BM, ra, A_PER_T);
                load_b(k0, rb_main);
            }
            mma(As[cur], Bs[cur]);
            if (kt + 1 < nkt)
            {
                store_tile(As[cur ^ 1], LDA_S, A_KMAJOR, BM, ra, A_PER_T);
                store_b(Bs[cur ^ 1], rb_main);
            }
            __syncthreads();
        }
    }

    if constexpr (WS > 1)
    {
        // the second wave set hands its accumulators to the first, one 32x32 block of each wave at a time
        float *xch = &As[0][0] + (wave * 16) * 64 + lane;
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
            for (int j = 0; j < CB; ++j)
            {
                if (kset == 1)
                {
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        xch[r * 64] = acc[i][j][r];
                }
                __syncthreads();
                if (kset == 0)
                {
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        acc[i][j][r] += xch[r * 64];
                }
                __syncthreads();
            }
        if (kset == 1)
            return;
    }
    // ---- epilogue: accumulator register r of lane (l32, lh) holds row 8*(r/4) + 4*lh + r%4, column l32
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
    float *Cout = g.C + (int64_t)kz * g.c_split_stride;
    // The activation is a constant inside the store loops, the addresses are a base per block plus a row stride, and
    // the bias values of a block's rows are fetched together before its first store.
    auto store_blocks = [&](auto act_tag) {
        constexpr int ACT = decltype(act_tag)::value;
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
            for (int j = 0; j < CB; ++j)
            {
                const int64_t col = n0 + wn + j * 32 + l32;
                if (col >= g.N)
                    continue;
                const int64_t row0 = m0 + wm + i * 32 + 4 * lh;
                const int rows_left = (int)(g.M - row0 < 32 ? g.M - row0 : 32);
                float bcol = 0.f;
                if (EPI == EPI_BIAS_COL && g.bias)
                    bcol = g.bias[col];
                float *out = Cout + row0 * g.ldc + col;
                int64_t stride = g.ldc;
                float brow[16];
                if (EPI == EPI_NCHW_ROWB)
                {
                    const int64_t n = col / g.P, p = col % g.P;
                    out = Cout + (n * g.M + row0) * g.P + p, stride = g.P;
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                    {
                        const int dr = 8 * (r / 4) + (r % 4);
                        brow[r] = (g.bias && dr < rows_left) ? g.bias[row0 + dr] : 0.f;
                    }
                }
#pragma unroll
                for (int r = 0; r < 16; ++r)
                {
                    const int dr = 8 * (r / 4) + (r % 4);
                    if (dr >= rows_left)
                        continue;
                    float v = acc[i][j][r];
                    if (EPI == EPI_NCHW_ROWB)
                    {
                        if (g.bias)
                            v = v + brow[r];
                        v = apply_act(v, ACT);
                    }
                    else if (EPI == EPI_BIAS_COL)
                        v = apply_act(v + bcol, ACT);
                    out[(int64_t)dr * stride] = v;
                }
            }
    };
    if (EPI == 0 || g.act == 0)
        store_blocks(ActTag<0>{});
    else if (g.act == 1)
        store_blocks(ActTag<1>{});
    else if (g.act == 2)
        store_blocks(ActTag<2>{});
    else
        store_blocks(ActTag<0>{});
}

// out[i] = sum over slices of part[s*stride + i] (+ bias by column). 64 outputs x 16 slice groups per workgroup:
// group g adds slices g, g+16, ..., the group sums meet in LDS and are added in group order — a fixed order.
constexpr int kRedGroups = 16;
__global__ __launch_bounds__(64 * kRedGroups) void splitk_reduce_kernel(const float *__restrict__ part, int splits,
                                                                         int64_t stride, float *out, int64_t M, int64_t N,
                                                                         int64_t ldc, const float *bias, int64_t P, int act)
{
    __shared__ float sh[kRedGroups][64];
    const int lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int64_t i = (int64_t)blockIdx.x * 64 + lane;
    float acc = 0.f;
    if (i < M * N)
    {
#pragma unroll 4
        for (int z = grp; z < splits; z += kRedGroups)
            acc += part[(int64_t)z * stride + i];
    }
    sh[grp][lane] = acc;
    __syncthreads();
    if (grp == 0 && i < M * N)
    {
        float s = sh[0][lane];
#pragma unroll
        for (int k = 1; k < kRedGroups; ++k)
            s += sh[k][lane];
        const int64_t r = i / N, c = i % N;
        if (P > 0)
        {
            // convolution forward: row = output channel (bias by row), column = n*P + p -> y[n][row][p]
            if (bias)
                s = s + bias[r];
            out[((c / P) * M + r) * P + c % P] = apply_act(s, act);
        }
        else
        {
            if (bias)
                s = apply_act(s + bias[c], act);
            out[r * ldc + c] = s;
        }
    }
}

// The same sum for few slices of a large output: one thread per four consecutive outputs, slices added in
// ascending order. Needs N % 4 == 0 (and P % 4 == 0) so that a quad stays inside one row (and one image).
__global__ __launch_bounds__(256) void splitk_reduce_vec_kernel(const float *__restrict__ part, int splits,
                                                                 int64_t stride, float *out, int64_t M, int64_t N,
                                                                 int64_t ldc, const float *bias, int64_t P, int act)
{
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= M * N)
        return;
    f32x4 acc = *reinterpret_cast<const f32x4 *>(part + i);
#pragma unroll 4
    for (int z = 1; z < splits; ++z)
    {
        const f32x4 v = *reinterpret_cast<const f32x4 *>(part + (int64_t)z * stride + i);
        acc[0] += v[0], acc[1] += v[1], acc[2] += v[2], acc[3] += v[3];
    }
    const int64_t r = i / N, c = i % N;
    if (P > 0)
    {
        if (bias)
        {
            const float b = bias[r];
            acc[0] = acc[0] + b, acc[1] = acc[1] + b, acc[2] = acc[2] + b, acc[3] = acc[3] + b;
        }
        acc[0] = apply_act(acc[0], act), acc[1] = apply_act(acc[1], act);
        acc[2] = apply_act(acc[2], act), acc[3] = apply_act(acc[3], act);
        *reinterpret_cast<f32x4 *>(out + ((c / P) * M + r) * P + c % P) = acc;
    }
    else
    {
        if (bias)
        {
            const f32x4 b = *reinterpret_cast<const f32x4 *>(bias + c);
            acc[0] = apply_act(acc[0] + b[0], act), acc[1] = apply_act(acc[1] + b[1], act);
            acc[2] = apply_act(acc[2] + b[2], act), acc[3] = apply_act(acc[3] + b[3], act);
        }
        *reinterpret_cast<f32x4 *>(out + r * ldc + c) = acc;
    }
}

// picks the reduction by shape: many slices of a small output -> slice groups in parallel; few slices of a large
// output -> streaming quads
void launch_splitk_reduce(const float *part, int splits, int64_t stride, float *out, int64_t M, int64_t N, int64_t ldc,
                          const float *bias, int64_t P, hipStream_t st, int act = 0)
{
    const bool quads = splits <= 32 && M * N >= (1 << 16) && N % 4 == 0 && stride % 4 == 0 && ldc % 4 == 0 && P % 4 == 0 &&
                       aligned16(part) && aligned16(out) && (bias == nullptr || P > 0 || aligned16(bias));
    if (quads)
        hipLaunchKernelGGL(splitk_reduce_vec_kernel, dim3((unsigned)odl::ceil_div(M * N, 1024)), dim3(256), 0, st, part,
                           splits, stride, out, M, N, ldc, bias, P, act);
    else
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)odl::ceil_div(M * N, 64)), dim3(64 * kRedGroups), 0, st,
                           part, splits, stride, out, M, N, ldc, bias, P, act);
}

// Sums the K pieces of each tail tile in piece order and stores the tile through the epilogue the main kernel
// would have used. One thread per four consecutive columns of a tile row.
__global__ __launch_bounds__(256) void tail_fixup_kernel(GemmArgs g, int BM, int BN, int epi)
{
    const int per_tile = BM * BN / 4;
    const int idx = blockIdx.x * 256 + threadIdx.x;
    const int ti = idx / per_tile, e = idx - ti * per_tile;
    const int nt = g.tiles_m * g.tiles_n;
    if (g.tail_first + ti >= nt)
        return;
    const int row_l = e / (BN / 4), c4 = e - row_l * (BN / 4);
    const float *p = g.tail_ws + ((int64_t)ti * g.tail_splits * BM + row_l) * BN + 4 * c4;
    f32x4 acc = *reinterpret_cast<const f32x4 *>(p);
#pragma unroll 4
    for (int z = 1; z < g.tail_splits; ++z)
    {
        const f32x4 v = *reinterpret_cast<const f32x4 *>(p + (int64_t)z * BM * BN);
        acc[0] += v[0], acc[1] += v[1], acc[2] += v[2], acc[3] += v[3];
    }
    int tm, tn;
    tile_coords(g.tail_first + ti, g.tiles_m, g.tiles_n, tm, tn);
    const int64_t row = (int64_t)tm * BM + row_l;
    if (row >= g.M)
        return;
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        const int64_t col = (int64_t)tn * BN + 4 * c4 + j;
        if (col >= g.N)
            continue;
        float v = acc[j];
        if (epi == EPI_NCHW_ROWB)
        {
            if (g.bias)
                v = v + g.bias[row];
            g.C[((col / g.P) * g.M + row) * g.P + col % g.P] = apply_act(v, g.act);
        }
        else
        {
            if (epi == EPI_BIAS_COL && g.bias)
                v = apply_act(v + g.bias[col], g.act);
            g.C[row * g.ldc + col] = v;
        }
    }
}

// Whether (and how) to split the last tiles: nt tiles over the chip's CUs (256) run in ceil(nt/256) rounds, and a last round of
// only a few tiles leaves most CUs idle for a whole tile's time. Those few tiles are cut into K pieces instead.
struct TailPlan
{
    int tiles = 0, splits = 0;  // tail tiles and K pieces of each (0: no tail split)
    int64_t kps = 0;
    size_t bytes = 0;
};

TailPlan plan_tail(int64_t nt, int64_t K, int BM, int BN)
{
    TailPlan p;
    const int64_t kt = odl::ceil_div(K, 16);
    const int64_t cus = odl::device_cus();
    const int64_t r = nt % cus;
    if (nt <= cus || nt > cus * 8 || r == 0 || r > cus / 2 || kt < 16)
        return p;
    int64_t s = cus / r;
    if (s > kt / 2)
        s = kt / 2;
    if (s > 32)
        s = 32;
    if (s < 2)
        return p;
    p.kps = odl::ceil_div(kt, s) * 16;
    p.splits = (int)odl::ceil_div(K, p.kps);
    p.tiles = (int)r;
    p.bytes = (size_t)p.tiles * p.splits * BM * BN * sizeof(float);
    return p;
}

// fills the tail fields of g (tiles_m/tiles_n set) when the workspace holds the partials; returns the grid size
unsigned apply_tail(GemmArgs &g, int BM, int BN, void *tail_ws, size_t tail_bytes)
{
    const int64_t nt = (int64_t)g.tiles_m * g.tiles_n;
    g.main_blocks = 0, g.tail_first = (int)nt, g.tail_splits = 0, g.tail_kps = 0, g.tail_ws = nullptr;
    g.xcds = odl::chip().xcds;
    if (g.splits != 1 || tail_ws == nullptr || reinterpret_cast<uintptr_t>(tail_ws) % 16 != 0)
        return (unsigned)(nt * g.splits);
    const TailPlan p = plan_tail(nt, g.K, BM, BN);
    if (p.splits == 0 || tail_bytes < p.bytes)
        return (unsigned)nt;
    g.tail_first = (int)(nt - p.tiles), g.main_blocks = g.tail_first, g.tail_splits = p.splits, g.tail_kps = p.kps;
    g.tail_ws = static_cast<float *>(tail_ws);
    return (unsigned)(g.main_blocks + p.tiles * p.splits);
}

void launch_tail_fixup(const GemmArgs &g, int BM, int BN, int epi, hipStream_t st)
{
    if (g.tail_splits <= 0)
        return;
    const int64_t nt = (int64_t)g.tiles_m * g.tiles_n;
    const int64_t threads = (nt - g.tail_first) * (BM * BN / 4);
    hipLaunchKernelGGL(tail_fixup_kernel, dim3((unsigned)odl::ceil_div(threads, 256)), dim3(256), 0, st, g, BM, BN, epi);
}

// the same product for the variant whose operands go from global memory straight into LDS
odl::DmaGemmArgs dma_args(const GemmArgs &g, int epi)
{
    odl::DmaGemmArgs d{};
    d.A = g.A, d.B = g.B, d.bias = g.bias, d.C = g.C;
    d.M = g.M, d.N = g.N, d.K = g.K, d.lda = g.lda, d.ldb = g.ldb, d.ldc = g.ldc;
    d.tiles_m = g.tiles_m, d.tiles_n = g.tiles_n, d.splits = g.splits;
    d.k_per_split = g.k_per_split, d.c_split_stride = g.c_split_stride;
    d.epi = epi == EPI_BIAS_COL ? 1 : (epi == EPI_NCHW_ROWB ? 2 : 0), d.act = g.act, d.xcds = g.xcds;
    d.c_p = epi == EPI_NCHW_ROWB ? g.P : 0;
    d.main_blocks = g.main_blocks, d.tail_first = g.tail_first, d.tail_splits = g.tail_splits, d.tail_kps = g.tail_kps;
    d.tail_ws = g.tail_ws;
    d.batch = 1, d.a_batch = d.b_batch = d.c_batch = 0;
    return d;
}

// tile counts up to which a launch puts about one workgroup on a compute unit
int64_t lone_workgroup_limit()
{
    const int64_t cus = odl::device_cus();
    return cus + cus / 4;
}

template <int BM, int BN, int BK, int EPI>
int launch_tile(bool ta, bool tb, bool vec, const GemmArgs &g_in, int splits, void *tail_ws, size_t tail_bytes,
                hipStream_t st)
{
    GemmArgs g = g_in;
    g.splits = splits;
    dim3 grid(apply_tail(g, BM, BN, tail_ws, tail_bytes));
    dim3 block(kThreads);
    if constexpr (BM == 128 && BN == 128)
    {
        // at most about one workgroup per compute unit: a second set of four waves on every tile
        if (vec && splits == 1 && g.tail_splits == 0 && (int64_t)g.tiles_m * g.tiles_n <= lone_workgroup_limit())
        {
            if constexpr (EPI != EPI_NCHW_ROWB)
            {
                const odl::DmaGemmArgs d = dma_args(g, EPI);
                if (odl::sgemm_dma_fits(ta, tb, d))
                    return odl::sgemm_dma_launch(128, ta, tb, d, st);
            }
#define ODL_GEMM_TWO_SETS(TA, TB)                                                                                   \
    if (ta == TA && tb == TB)                                                                                       \
    {                                                                                                               \
        hipLaunchKernelGGL((sgemm_mfma_kernel<BM, BN, 32, TA, TB, true, EPI, SB_PLAIN, 0, 2>), grid, dim3(2 * kThreads), \
                           0, st, g, ConvSrc{});                                                                    \
        return ODL_OK;                                                                                              \
    }
            ODL_GEMM_TWO_SETS(false, false)
            ODL_GEMM_TWO_SETS(false, true)
            ODL_GEMM_TWO_SETS(true, false)
            ODL_GEMM_TWO_SETS(true, true)
#undef ODL_GEMM_TWO_SETS
        }
    }
    if constexpr (BM == 128 && BN == 128 && EPI != EPI_NCHW_ROWB)
    {
        // many tiles: operands straight into LDS, two workgroups of eight waves per compute unit (4096^3: 82 -> 88 % of
        // the matrix peak); the K pieces of a split tail are finished by the fix-up kernel as below
        if (vec && splits == 1)
        {
            const odl::DmaGemmArgs d = dma_args(g, EPI);
            if (odl::sgemm_dma_fits(ta, tb, d))
            {
                const int rc = odl::sgemm_dma_launch(129, ta, tb, d, st);
                if (rc == ODL_OK)
                    launch_tail_fixup(g, BM, BN, EPI, st);
                return rc;
            }
        }
    }
#define ODL_GEMM_CASE(TA, TB, V)                                                                      \
    if (ta == TA && tb == TB && vec == V)                                                             \
    {                                                                                                 \
        hipLaunchKernelGGL((sgemm_mfma_kernel<BM, BN, BK, TA, TB, V, EPI>), grid, block, 0, st, g,   \
                           ConvSrc{});                                                                \
        launch_tail_fixup(g, BM, BN, EPI, st);                                                        \
        return ODL_OK;                                                                                \
    }
    ODL_GEMM_CASE(false, false, true)
    ODL_GEMM_CASE(false, true, true)
    ODL_GEMM_CASE(true, false, true)
    ODL_GEMM_CASE(true, true, true)
    ODL_GEMM_CASE(false, false, false)
    ODL_GEMM_CASE(false, true, false)
    ODL_GEMM_CASE(true, false, false)
    ODL_GEMM_CASE(true, true, false)
#undef ODL_GEMM_CASE
    return ODL_ERR_RUNTIME;
}

constexpr int kBK = 16;

// Tile edge for a problem: 128x128 tiles when they can fill the chip (256 CUs), 64x64 tiles for smaller outputs so
// that more workgroups exist.
int pick_tile(int64_t M, int64_t N)
{
    return (odl::ceil_div(M, 128) * odl::ceil_div(N, 128) >= odl::device_cus()) ? 128 : 64;
}

// K slices for problems whose tiles alone cannot fill the chip: aim at ~512 workgroups, at least 4 K slabs each.
int pick_splits(int64_t M, int64_t N, int64_t K, int requested)
{
    if (requested >= 1)
        return requested;
    const int tile      = pick_tile(M, N);
    const int64_t tiles = odl::ceil_div(M, tile) * odl::ceil_div(N, tile);
    const int64_t kt    = odl::ceil_div(K, kBK);
    // (a K of under 256 is a handful of slabs: slicing it saves less than the launch that adds the slices up costs —
    // 256x3136x128, the CNN's hidden layer's input gradient: two slices 7.5 + 4.1 us)
    if (tiles >= odl::device_cus() || kt < 16)
        return 1;
    int64_t s = odl::ceil_div(2 * odl::device_cus(), tiles);
    if (s > kt / 4)
        s = kt / 4;
    if (s > 128)
        s = 128;
    return s < 1 ? 1 : (int)s;
}

// K slices for 64x64 tiles read with 16-byte loads: about one workgroup of eight waves per compute unit, each slice at
// least 8 slabs of 32 long. 0: the product does not suit that variant.
int pick_splits_two_sets(int64_t tiles, int64_t K)
{
    const int64_t cus = odl::device_cus();
    if (tiles > lone_workgroup_limit() || K < 256)
        return 0;
    // cost of s slices in slab times: rounds of workgroups over the compute units, each walking its slabs plus about
    // four slab times of prologue and epilogue, plus the fold's share, which grows with the slices
    const int64_t slabs = odl::ceil_div(K, 32);
    int64_t best = 1, best_cost = 0;
    for (int64_t s = 1; s <= 128 && (s == 1 || K / s >= 256); ++s)
    {
        const int64_t cost = 4 * odl::ceil_div(tiles * s, cus) * (odl::ceil_div(slabs, s) + 4) + s;
        if (s == 1 || cost < best_cost)
            best = s, best_cost = cost;
    }
    // whole slabs per slice, and no empty slice
    return (int)odl::ceil_div(slabs, odl::ceil_div(slabs, best));
}

// A long K walked by few 64x64 tiles (one workgroup per CU, nothing to overlap with): a 32-wide K slab halves the number
// of barrier-and-refill bubbles per tile (1024^3: 34 -> 31 us). 16-byte loads only.
template <int EPI>
int launch_small_tile_wide_slab(bool ta, bool tb, GemmArgs g, int splits, hipStream_t st)
{
    g.splits = splits;
    g.main_blocks = 0, g.tail_first = g.tiles_m * g.tiles_n, g.tail_splits = 0, g.tail_kps = 0, g.tail_ws = nullptr;
    g.xcds = odl::chip().xcds;
    const dim3 grid((unsigned)(g.tiles_m * g.tiles_n * splits)), block(kThreads);
    const bool two_sets = (int64_t)g.tiles_m * g.tiles_n * splits <= lone_workgroup_limit();
    {
        // straight-to-LDS loads: one workgroup per compute unit while the launch is about that size, two beyond it
        // (6272x256x1152: 51 -> 43 us, 3136x512x2304: 98 -> 78 us against the register-staged kernel)
        const odl::DmaGemmArgs d = dma_args(g, EPI);
        if (odl::sgemm_dma_fits(ta, tb, d))
            return odl::sgemm_dma_launch(two_sets ? 64 : 65, ta, tb, d, st);
    }
    if (g.K % 32 != 0)  // the register-staged kernel below walks whole 32-wide slabs only
        return launch_tile<64, 64, kBK, EPI>(ta, tb, true, g, splits, nullptr, 0, st);
#define ODL_WIDE_CASE(TA, TB)                                                                                  \
    if (ta == TA && tb == TB)                                                                                  \
    {                                                                                                          \
        if (two_sets)                                                                                          \
            hipLaunchKernelGGL((sgemm_mfma_kernel<64, 64, 32, TA, TB, true, EPI, SB_PLAIN, 0, 2>), grid,       \
                               dim3(2 * kThreads), 0, st, g, ConvSrc{});                                       \
        else                                                                                                   \
            hipLaunchKernelGGL((sgemm_mfma_kernel<64, 64, 32, TA, TB, true, EPI>), grid, block, 0, st, g, ConvSrc{}); \
        return ODL_OK;                                                                                         \
    }
    ODL_WIDE_CASE(false, false)
    ODL_WIDE_CASE(false, true)
    ODL_WIDE_CASE(true, false)
    ODL_WIDE_CASE(true, true)
#undef ODL_WIDE_CASE
    return ODL_ERR_RUNTIME;
}

template <int EPI>
int launch_any_tile(int tile, bool ta, bool tb, bool vec, const GemmArgs &g, int splits, void *tail_ws,
                    size_t tail_bytes, hipStream_t st)
{
    if (tile == 128)
        return launch_tile<128, 128, kBK, EPI>(ta, tb, vec, g, splits, tail_ws, tail_bytes, st);
    if constexpr (EPI != EPI_NCHW_ROWB)
    {
        if (vec && ((splits == 1 && g.K >= 1024 && g.K % 32 == 0) ||
                    (splits == 1 && g.K >= 128 && (int64_t)g.tiles_m * g.tiles_n > lone_workgroup_limit()) ||
                    splits == pick_splits_two_sets((int64_t)g.tiles_m * g.tiles_n, g.K)))
            return launch_small_tile_wide_slab<EPI>(ta, tb, g, splits, st);
    }
    else if (vec && splits == 1 && g.K >= 128 && g.N < (1ll << 32) && g.P < (1ll << 32))
    {
        // the explicit convolution forward (y^T = W . col^T, stored NCHW): straight-to-LDS loads when the shape allows
        GemmArgs h = g;
        h.splits = 1, h.xcds = odl::chip().xcds;
        h.main_blocks = 0, h.tail_first = h.tiles_m * h.tiles_n, h.tail_splits = 0, h.tail_kps = 0, h.tail_ws = nullptr;
        const odl::DmaGemmArgs d = dma_args(h, EPI);
        if (odl::sgemm_dma_fits(ta, tb, d))
            return odl::sgemm_dma_launch((int64_t)h.tiles_m * h.tiles_n <= lone_workgroup_limit() ? 64 : 65, ta, tb, d, st);
    }
    return launch_tile<64, 64, kBK, EPI>(ta, tb, vec, g, splits, nullptr, 0, st);
}
}  // namespace

namespace odl
{
// Shared by the convolution entry points. epi: 0 plain, 1 bias by column, 2 NCHW store with bias by row.
int sgemm_launch(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                 const float *B, int64_t ldb, float *C, int64_t ldc, const float *bias, int epi, int64_t P,
                 int split_k, void *workspace, size_t workspace_bytes, hipStream_t st, int act = 0)
{
    if (M == 0 || N == 0)
        return ODL_OK;
    ODL_REQUIRE(M > 0 && N > 0 && K >= 0, "sgemm: bad dimensions M=%lld N=%lld K=%lld", (long long)M, (long long)N,
                (long long)K);
    ODL_REQUIRE(A && B && C, "sgemm: null operand");
    ODL_REQUIRE(lda >= (trans_a ? M : K) && ldb >= (trans_b ? K : N) && (epi == EPI_NCHW_ROWB || ldc >= N),
                "sgemm: leading dimension smaller than the row length");
    ODL_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), "sgemm: dimension exceeds 2^31");
    // a classifier layer's handful of output columns: vector-ALU kernel, one launch, no K slices (gemm_skinny.hip)
    if (!trans_a && !trans_b && epi != EPI_NCHW_ROWB && split_k < 1 && odl::skinny_ok(M, N, K))
        return odl::skinny_forward(A, B, epi == EPI_BIAS_COL ? bias : nullptr, C, M, N, K, lda, ldb, ldc,
                                   epi == EPI_BIAS_COL && bias ? act : 0, st);
    GemmArgs g;
    g.A = A, g.B = B, g.C = C, g.bias = bias;
    g.M = M, g.N = N, g.K = K, g.lda = lda, g.ldb = ldb, g.ldc = ldc, g.P = P, g.act = act;
    const int tile = pick_tile(M, N);
    g.tiles_m = (int)ceil_div(M, tile), g.tiles_n = (int)ceil_div(N, tile);
    ODL_REQUIRE((int64_t)g.tiles_m * g.tiles_n < (1ll << 31), "sgemm: too many tiles");

    // 16-byte loads need 16-byte aligned rows: base pointers, leading dimensions and the contiguous extents
    const bool vec = ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) % 16 == 0) && lda % 4 == 0 &&
                     ldb % 4 == 0 && (trans_a ? M : K) % 4 == 0 && (trans_b ? K : N) % 4 == 0;

    // An output of so few 64x64 tiles that K would be cut in two: 64x32 tiles instead, twice as many workgroups walking
    // the whole K — no partial outputs, no second launch to add them (512x1000x784: 15.0 -> 11.5 us).
    if (epi != EPI_NCHW_ROWB && split_k < 1 && tile == 64 && vec &&
        pick_splits_two_sets((int64_t)g.tiles_m * g.tiles_n, K) == 2 && ceil_div(M, 64) * ceil_div(N, 32) <= lone_workgroup_limit())
    {
        GemmArgs h = g;
        h.tiles_n = (int)ceil_div(N, 32), h.splits = 1, h.k_per_split = ceil_div(K, 64) * 64, h.c_split_stride = 0;
        h.xcds = odl::chip().xcds;
        h.main_blocks = 0, h.tail_first = h.tiles_m * h.tiles_n, h.tail_splits = 0, h.tail_kps = 0, h.tail_ws = nullptr;
        const odl::DmaGemmArgs d = dma_args(h, epi);
        if (odl::sgemm_dma_fits(trans_a, trans_b, d))
        {
            const int rc = odl::sgemm_dma_launch(32, trans_a, trans_b, d, st);
            if (rc != ODL_OK)
                return fail(rc, "sgemm: no kernel variant");
            ODL_LAUNCH_CHECK();
            return ODL_OK;
        }
    }
    int splits = (epi == EPI_NCHW_ROWB) ? 1 : pick_splits(M, N, K, split_k);
    if (epi != EPI_NCHW_ROWB && split_k < 1 && tile == 64 && vec)
    {
        const int s2 = pick_splits_two_sets((int64_t)g.tiles_m * g.tiles_n, K);
        if (s2 > 0 && s2 <= splits)  // never more slices than the workspace query promised room for
            splits = s2;
    }
    const int64_t kt = ceil_div(K > 0 ? K : 1, kBK);
    if (splits > kt)
        splits = (int)kt;
    if (splits > 1)
    {
        const size_t need = (size_t)splits * M * N * sizeof(float);
        if (workspace == nullptr || workspace_bytes < need)
        {
            if (split_k > 1)
                return fail(ODL_ERR_INVALID_ARG, "sgemm: split_k=%d needs %zu workspace bytes, got %zu", split_k, need,
                            workspace_bytes);
            splits = 1;  // automatic choice falls back to a single pass
        }
    }
    const bool slab32 = epi != EPI_NCHW_ROWB && tile == 64 && vec && splits > 1 &&
                        splits == pick_splits_two_sets((int64_t)g.tiles_m * g.tiles_n, K);
    g.k_per_split    = slab32 ? ceil_div(ceil_div(K, 32), splits) * 32 : ceil_div(kt, splits) * kBK;
    g.c_split_stride = 0;
    int rc;
    if (splits > 1)
    {
        GemmArgs p = g;
        p.C = static_cast<float *>(workspace), p.ldc = N, p.bias = nullptr, p.c_split_stride = M * N;
        rc = launch_any_tile<EPI_PLAIN>(tile, trans_a, trans_b, vec, p, splits, nullptr, 0, st);
        if (rc != ODL_OK)
            return fail(rc, "sgemm: no kernel variant");
        ODL_LAUNCH_CHECK();
        launch_splitk_reduce(static_cast<const float *>(workspace), splits, M * N, C, M, N, ldc,
                             epi == EPI_BIAS_COL ? bias : nullptr, 0, st, epi == EPI_BIAS_COL && bias ? act : 0);
        ODL_LAUNCH_CHECK();
        return ODL_OK;
    }
    if (epi == EPI_NCHW_ROWB)
        rc = launch_any_tile<EPI_NCHW_ROWB>(tile, trans_a, trans_b, vec, g, 1, workspace, workspace_bytes, st);
    else if (epi == EPI_BIAS_COL && bias)
        rc = launch_any_tile<EPI_BIAS_COL>(tile, trans_a, trans_b, vec, g, 1, workspace, workspace_bytes, st);
    else
        rc = launch_any_tile<EPI_PLAIN>(tile, trans_a, trans_b, vec, g, 1, workspace, workspace_bytes, st);
    if (rc != ODL_OK)
        return fail(rc, "sgemm: no kernel variant");
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

// The two gradients of y = x.w in one launch (gx[M,K] = gy[M,N].w[K,N]^T and gw[K,N] = x[M,K]^T.gy[M,N]) when each of
// them alone would be a single launch of about one workgroup per compute unit on the straight-to-LDS kernel: together
// they put two workgroups on every compute unit. Returns 1 when launched, 0 when the shapes do not suit (the caller then
// launches them one after the other), a negative error code on failure.
namespace
{
// the tile class a product would take as a launch of its own, when that launch is one the pair kernel can stand in for
// (whole K per workgroup, 16-byte loads): 128, 64 or 32; 0 otherwise
int pair_tile_class(bool vec, int64_t M, int64_t N, int64_t K)
{
    if (!vec || K < 128)
        return 0;
    if (pick_tile(M, N) == 128)
        return ceil_div(M, 128) * ceil_div(N, 128) <= lone_workgroup_limit() ? 128 : 0;
    const int64_t tiles = ceil_div(M, 64) * ceil_div(N, 64);
    const int s2 = pick_splits_two_sets(tiles, K);
    if (s2 == 2 && ceil_div(M, 64) * ceil_div(N, 32) <= lone_workgroup_limit())
        return 32;
    if (s2 == 1)  // (which already says: at most about one 64x64 tile per compute unit, K of 256 or more)
        return 64;
    // a K of 128 to 255 on its own is not worth this variant's prologue; next to its partner in one launch it is worth
    // the launch it saves (a hidden layer of 128 units: its input gradient)
    if (K < 256 && tiles <= lone_workgroup_limit())
        return 64;
    return 0;
}

odl::DmaGemmArgs pair_product(int cls, const float *A, int64_t lda, const float *B, int64_t ldb, float *C, int64_t ldc,
                              int64_t M, int64_t N, int64_t K)
{
    odl::DmaGemmArgs d{};
    d.A = A, d.B = B, d.bias = nullptr, d.C = C;
    d.M = M, d.N = N, d.K = K, d.lda = lda, d.ldb = ldb, d.ldc = ldc;
    d.tiles_m = (int)ceil_div(M, cls == 128 ? 128 : 64), d.tiles_n = (int)ceil_div(N, cls == 128 ? 128 : (cls == 32 ? 32 : 64));
    d.splits = 1, d.k_per_split = ceil_div(K, 64) * 64, d.c_split_stride = 0;
    d.epi = 0, d.act = 0, d.xcds = odl::chip().xcds, d.c_p = 0;
    d.main_blocks = 0, d.tail_first = d.tiles_m * d.tiles_n, d.tail_splits = 0, d.tail_kps = 0, d.tail_ws = nullptr;
    d.batch = 1, d.a_batch = d.b_batch = d.c_batch = 0;
    return d;
}
}  // namespace

// gb (may be null): the bias gradient, gy summed over its rows, in the same launch when its size is one the small column
// sum takes (*gb_done tells)
int matmul_backward_pair(const float *x, const float *w, const float *gy, float *gx, float *gw, int64_t M, int64_t K,
                         int64_t N, hipStream_t st, float *gb = nullptr, bool *gb_done = nullptr)
{
    if (gb_done)
        *gb_done = false;
    if (M <= 0 || K <= 0 || N <= 0 || M >= (1ll << 31) || K >= (1ll << 31) || N >= (1ll << 31))
        return 0;
    // 16-byte loads: every row of x [M,K], w [K,N] and gy [M,N] starts on a 16-byte boundary and M is a multiple of four
    // (x^T's rows are read four columns of x at a time)
    const bool vec = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(gy)) % 16 == 0) &&
                     K % 4 == 0 && N % 4 == 0;
    const int c0 = pair_tile_class(vec, M, K, N), c1 = pair_tile_class(vec, K, N, M);
    if (c0 == 0 || c1 == 0 || (c0 == 128) != (c1 == 128))
        return 0;
    const odl::DmaGemmArgs d0 = pair_product(c0, gy, N, w, N, gx, K, M, K, N);  // gx = gy . w^T
    const odl::DmaGemmArgs d1 = pair_product(c1, x, K, gy, N, gw, N, K, N, M);  // gw = x^T . gy
    // all workgroups resident at once, two per compute unit
    if ((int64_t)d0.tiles_m * d0.tiles_n + (int64_t)d1.tiles_m * d1.tiles_n > 2 * (int64_t)odl::device_cus())
        return 0;
    if (!odl::sgemm_dma_fits(false, true, d0) || !odl::sgemm_dma_fits(true, false, d1))
        return 0;
    odl::ColSumJob job{};
    const bool with_sum = gb && gb_done && odl::small_cols(1, M, N);
    if (with_sum)
    {
        job.src = gy, job.dst = gb, job.axis = M, job.inner = N;
        job.quads = (N % 4 == 0 && reinterpret_cast<uintptr_t>(gy) % 16 == 0) ? 1 : 0;
        job.blocks = (unsigned)odl::ceil_div(N, job.quads ? 32 : 16);
    }
    const int rc = odl::sgemm_dma_pair_launch(c0, d0, c1, d1, st, with_sum ? &job : nullptr);
    if (rc != ODL_OK)
        return rc;  // (error codes are negative)
    if (with_sum)
        *gb_done = true;
    return 1;
}

// ------------------------------------------------------------------------------------------------------
// Convolution as implicit GEMM: the same kernel, its B operand gathered from the image / upstream gradient.
namespace
{
bool conv_tile_bm64(int64_t M, int64_t N, int splits)
{
    return M <= 64 || odl::ceil_div(M, 128) * odl::ceil_div(N, 128) * splits < odl::device_cus();
}

// Fetching the gathered operands two K slabs ahead was measured and lost, on full launches (the second register set
// costs the 128x128 kernels their fourth wave per SIMD: C1 forward 175 -> 254 us) and on sparse ones alike (C2 forward,
// one or two workgroups per compute unit: 57 -> 90 us).
constexpr bool kConvPF2 = false;

template <int SB, bool TA, int EPI>
int launch_conv_tile(GemmArgs g, const ConvSrc &cv, int splits, void *tail_ws, size_t tail_bytes, hipStream_t st)
{
    const int ck = (cv.KH == 3 && cv.KW == 3) ? 3 : ((cv.KH == 1 && cv.KW == 1) ? 1 : 0);
    const bool bm64 = conv_tile_bm64(g.M, g.N, splits);
    g.tiles_m = (int)odl::ceil_div(g.M, bm64 ? 64 : 128);
    g.tiles_n = (int)odl::ceil_div(g.N, 128);
    g.splits = splits;
    const dim3 grid(apply_tail(g, bm64 ? 64 : 128, 128, tail_ws, tail_bytes)), block(kThreads);
#define ODL_CONV_CASE(BMV, CKV)                                                                                  \
    if constexpr (SB != SB_CONV_FWD_TAP || CKV > 0)                                                              \
        if (bm64 == (BMV == 64) && ck == CKV)                                                                    \
        {                                                                                                        \
            hipLaunchKernelGGL((sgemm_mfma_kernel<BMV, 128, 16, TA, false, true, EPI, SB, CKV, 1, kConvPF2>), grid,  \
                               block, 0, st, g, cv);                                                             \
            launch_tail_fixup(g, BMV, 128, EPI, st);                                                             \
            return ODL_OK;                                                                                       \
        }
    ODL_CONV_CASE(128, 3)
    ODL_CONV_CASE(128, 1)
    ODL_CONV_CASE(128, 0)
    ODL_CONV_CASE(64, 3)
    ODL_CONV_CASE(64, 1)
    ODL_CONV_CASE(64, 0)
#undef ODL_CONV_CASE
    return ODL_ERR_RUNTIME;
}

// wp[c][((oc/16)*KHW + tap)*16 + oc%16] = w[oc][c][tap]: the K order of the input-grad GEMM (OC % 16 == 0)
__global__ void permute_weight_kernel(const float *__restrict__ w, float *__restrict__ wp, int OC, int C, int KHW)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= (int64_t)OC * C * KHW)
        return;
    const int k = (int)(t % ((int64_t)OC * KHW));
    const int c = (int)(t / ((int64_t)OC * KHW));
    const int lo = k % 16, tap = (k / 16) % KHW, ocs = k / (16 * KHW);
    const int oc = ocs * 16 + lo;
    wp[t] = w[((int64_t)oc * C + c) * KHW + tap];
}

// wp[oc][tap*C + c] = w[oc][c][tap]: the K order of the tap-ordered forward gather
__global__ void permute_weight_tap_kernel(const float *__restrict__ w, float *__restrict__ wp, int C, int KHW, int64_t total)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total)
        return;
    const int K = C * KHW;
    const int64_t oc = t / K;
    const int k = (int)(t - oc * K);
    const int tap = k / C, c = k - tap * C;
    wp[t] = w[oc * K + c * KHW + tap];
}

// K slices for a product whose tiles alone leave most of the chip idle. All workgroups are resident at once (at
// most `slots` of them), so the launch lasts as long as the busiest CU: (workgroups on it) x (K slabs each, plus
// about three slabs' worth of prologue and epilogue). A lone workgroup on a CU has nothing to overlap its memory
// latency with and runs a quarter slower, three or more overlap a little better than two, and every slice adds one
// more pass over the output (tiles x 64 KB) for the reduction that follows. The slice count with the smallest such
// estimate wins.
int pick_conv_splits(int64_t tiles, int64_t kt, int64_t slots, int64_t max_splits)
{
    int best = 1;
    double best_cost = 0;
    const int64_t cus = odl::device_cus();
    for (int64_t s = 1; s <= max_splits && tiles * s <= slots; ++s)
    {
        const int64_t per_cu = odl::ceil_div(tiles * s, cus);
        const double overlap = per_cu == 1 ? 1.25 : (per_cu == 2 ? 1.0 : 0.95);
        const double cost = (double)per_cu * (double)(odl::ceil_div(kt, s) + 3) * overlap + 0.014 * (double)tiles * (double)s;
        if (s == 1 || cost < best_cost)
            best = (int)s, best_cost = cost;
    }
    return best;
}

int wgrad_splits(int64_t OC, int64_t K, int64_t M)
{
    const int64_t tiles = odl::ceil_div(OC, OC <= 64 ? 64 : 128) * odl::ceil_div(K, 128);
    const int64_t kt = odl::ceil_div(M, kBK);
    const int64_t cap = kt / 8 < 256 ? kt / 8 : 256;
    return pick_conv_splits(tiles, kt, (OC <= 64 ? 4 : 3) * (int64_t)odl::device_cus(), cap);
}
}  // namespace

// shapes the gathered-operand kernels accept (everything else takes the explicit im2col path)
bool conv_implicit_forward_ok(const float *w, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                              int64_t OH, int64_t OW)
{
    const int64_t K = C * KH * KW;
    return K % 4 == 0 && aligned16(w) && K < (1 << 30) && C * H * W < (1ll << 30) && N * OH * OW < (1ll << 31) &&
           OC < (1 << 30);
}

bool conv_implicit_wgrad_ok(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                            int64_t OH, int64_t OW)
{
    return OC % 4 == 0 && aligned16(gy) && C * KH * KW < (1 << 30) && C * H * W < (1ll << 30) &&
           N * OH * OW < (1ll << 31);
}

bool conv_implicit_dgrad_ok(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                            int SH, int SW)
{
    return SH == 1 && SW == 1 && OC % 16 == 0 && aligned16(gy) && (int64_t)KH * KW * OC < (1 << 30) &&
           N * H * W < (1ll << 31) && C < (1 << 30);
}

size_t conv_implicit_wgrad_workspace(int64_t N, int64_t C, int64_t OC, int KH, int KW, int64_t OH, int64_t OW)
{
    const int64_t K = C * KH * KW, M = N * OH * OW;
    const int s = wgrad_splits(OC, K, M);
    return s > 1 ? (size_t)s * OC * K * sizeof(float) : 0;
}

static size_t conv_tail_bytes(int64_t M, int64_t N, int64_t K)
{
    const int bm = conv_tile_bm64(M, N, 1) ? 64 : 128;
    return plan_tail(ceil_div(M, bm) * ceil_div(N, 128), K, bm, 128).bytes;
}

static size_t dgrad_wp_bytes(int64_t C, int64_t OC, int KH, int KW)
{
    return (((size_t)C * KH * KW * OC * sizeof(float)) + 255) & ~(size_t)255;
}

// permuted weights, then the tail-split partials of the input-grad GEMM [C, pixels, KH*KW*OC]
size_t conv_implicit_dgrad_workspace(int64_t C, int64_t OC, int KH, int KW, int64_t pixels)
{
    return dgrad_wp_bytes(C, OC, KH, KW) + conv_tail_bytes(C, pixels, (int64_t)KH * KW * OC);
}

static ConvSrc make_src(int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW, int64_t OC, int KH, int KW, int SH,
                        int SW, int PH, int PW)
{
    return ConvSrc{(int)C, (int)H,  (int)W, (int)OH, (int)OW, (int)OC, KH, KW, SH, SW, PH, PW, make_fastdiv((unsigned)OW),
                   make_fastdiv((unsigned)OH), make_fastdiv((unsigned)W), make_fastdiv((unsigned)H), make_fastdiv((unsigned)(C >= kBK ? C / kBK : 1))};
}

// K slices of the forward product when its tiles alone leave most of the chip idle
static int forward_splits(int64_t OC, int64_t M, int64_t K)
{
    const int64_t tiles128 = ceil_div(OC, 128) * ceil_div(M, 128);
    const int64_t tiles = OC <= 64 ? ceil_div(OC, 64) * ceil_div(M, 128) : tiles128;
    const int64_t kt = ceil_div(K, kBK);
    if (tiles128 >= 200 || tiles >= 200 || kt < 8)
        return 1;
    const int64_t cap = kt / 4 < 32 ? kt / 4 : 32;
    return pick_conv_splits(tiles, kt, (OC <= 64 ? 4 : 3) * (int64_t)odl::device_cus(), cap);
}

}  // namespace odl
namespace odl
{
// K slices the gathered forward would cut this product into (1: none)
int conv_implicit_forward_splits(int64_t OC, int64_t M, int64_t K)
{
    return forward_splits(OC, M, K);
}

// The tap-ordered gather: square 1x1 / 3x3 windows over a channel count that fills whole K slabs, image addressed
// with 32-bit byte offsets. A 3x3 window needs the weights re-ordered to [OC][tap][C] first (a 1x1 window's order
// is already that).
static bool forward_tap_ok(int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW)
{
    return KH == KW && (KH == 1 || KH == 3) && C % kBK == 0 && N * C * H * W < (1ll << 30);
}

static size_t forward_wp_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW)
{
    if (!forward_tap_ok(N, C, H, W, KH, KW) || KH == 1)
        return 0;
    return (((size_t)OC * C * KH * KW * sizeof(float)) + 255) & ~(size_t)255;
}

// re-ordered weights (3x3 tap-ordered gather only), then K-slice partials or tail-split partials
size_t conv_implicit_forward_workspace(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                                       int64_t OH, int64_t OW)
{
    const int64_t K = C * KH * KW, M = N * OH * OW;
    const int s = forward_splits(OC, M, K);
    return forward_wp_bytes(N, C, H, W, OC, KH, KW) +
           (s > 1 ? (size_t)s * OC * M * sizeof(float) : conv_tail_bytes(OC, M, K));
}

// y[n][oc][p] = sum_k W2d[oc][k] * x_gathered[(n,p)][k] + b[oc]
// the bytes of the re-ordered filter copy the forward makes for this shape (0: it reads the filter as it lies)
size_t conv_implicit_forward_packed_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW)
{
    return (forward_tap_ok(N, C, H, W, KH, KW) && KH > 1) ? (size_t)OC * C * KH * KW * sizeof(float) : 0;
}

// packed[oc][tap*C + c] = w[oc][c][tap]
int conv_implicit_forward_pack(const float *w, int64_t C, int64_t OC, int KH, int KW, float *packed, hipStream_t st)
{
    const int64_t total = OC * C * KH * KW;
    ODL_REQUIRE(total < (1ll << 31), "conv2d: filter too large");
    hipLaunchKernelGGL(permute_weight_tap_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, st, w, packed, (int)C,
                       KH * KW, total);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int conv_implicit_forward(const float *x, const float *w, const float *b, float *y, int64_t N, int64_t C, int64_t H,
                          int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, int64_t OH, int64_t OW,
                          int act, void *workspace, size_t workspace_bytes, hipStream_t st, const float *packed)
{
    GemmArgs g{};
    g.A = w, g.B = x, g.C = y, g.bias = b, g.act = act;
    g.M = OC, g.N = N * OH * OW, g.K = C * KH * KW;
    g.lda = g.K, g.ldb = 0, g.ldc = 0, g.P = OH * OW;
    g.k_per_split = ceil_div(g.K, kBK) * kBK, g.c_split_stride = 0;
    const ConvSrc cv = make_src(C, H, W, OH, OW, OC, KH, KW, SH, SW, PH, PW);
    bool tap = forward_tap_ok(N, C, H, W, KH, KW);
    if (tap && KH > 1 && packed != nullptr)
        g.A = packed;  // the caller keeps the re-ordered copy (weights that do not change between calls)
    else if (tap && KH > 1)
    {
        const size_t wp_bytes = forward_wp_bytes(N, C, H, W, OC, KH, KW);
        if (workspace != nullptr && workspace_bytes >= wp_bytes)
        {
            float *wp = static_cast<float *>(workspace);
            const int64_t total = OC * g.K;
            hipLaunchKernelGGL(permute_weight_tap_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, st, w, wp,
                               (int)C, KH * KW, total);
            ODL_LAUNCH_CHECK();
            g.A = wp;
            workspace = static_cast<char *>(workspace) + wp_bytes, workspace_bytes -= wp_bytes;
        }
        else
            tap = false;  // a caller without the workspace still gets the (c,kh,kw)-ordered gather
    }
    int splits = forward_splits(OC, g.N, g.K);
    if (splits > 1 && (workspace == nullptr || workspace_bytes < (size_t)splits * OC * g.N * sizeof(float)))
        splits = 1;  // a caller without the workspace still gets the single-pass kernel
    int rc;
    if (splits > 1)
    {
        // K slices into plain [OC, M] partials, then one pass that sums them in order, adds the bias and stores NCHW
        g.k_per_split = ceil_div(ceil_div(g.K, kBK), splits) * kBK;
        splits = (int)ceil_div(g.K, g.k_per_split);
        g.C = static_cast<float *>(workspace), g.bias = nullptr, g.ldc = g.N, g.c_split_stride = OC * g.N;
        rc = tap ? launch_conv_tile<SB_CONV_FWD_TAP, false, EPI_PLAIN>(g, cv, splits, nullptr, 0, st)
                 : launch_conv_tile<SB_CONV_FWD, false, EPI_PLAIN>(g, cv, splits, nullptr, 0, st);
        if (rc != ODL_OK)
            return fail(rc, "conv2d: no kernel variant");
        ODL_LAUNCH_CHECK();
        launch_splitk_reduce(static_cast<const float *>(workspace), splits, OC * g.N, y, OC, g.N, g.N, b, g.P, st, act);
        ODL_LAUNCH_CHECK();
        return ODL_OK;
    }
    rc = tap ? launch_conv_tile<SB_CONV_FWD_TAP, false, EPI_NCHW_ROWB>(g, cv, 1, workspace, workspace_bytes, st)
             : launch_conv_tile<SB_CONV_FWD, false, EPI_NCHW_ROWB>(g, cv, 1, workspace, workspace_bytes, st);
    if (rc != ODL_OK)
        return fail(rc, "conv2d: no kernel variant");
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

// gW[oc][k] = sum_m gy2d[m][oc] * x_gathered[m][k]   (gy2d = gy's buffer as [N*OH*OW, OC])
int conv_implicit_wgrad(const float *gy, const float *x, float *gw, int64_t N, int64_t C, int64_t H, int64_t W,
                        int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, int64_t OH, int64_t OW,
                        void *workspace, size_t workspace_bytes, hipStream_t st)
{
    const int64_t K = C * KH * KW, M = N * OH * OW;
    int splits = wgrad_splits(OC, K, M);
    const size_t need = splits > 1 ? (size_t)splits * OC * K * sizeof(float) : 0;
    if (splits > 1 && (workspace == nullptr || workspace_bytes < need))
        splits = 1;
    GemmArgs g{};
    g.A = gy, g.B = x, g.bias = nullptr;
    g.M = OC, g.N = K, g.K = M;
    g.lda = OC, g.ldb = 0, g.P = 0;
    g.k_per_split = ceil_div(ceil_div(M, kBK), splits) * kBK;
    splits = (int)ceil_div(M, g.k_per_split);
    g.C = splits > 1 ? static_cast<float *>(workspace) : gw;
    g.ldc = K;
    g.c_split_stride = splits > 1 ? OC * K : 0;
    int rc = launch_conv_tile<SB_CONV_WGRAD, true, EPI_PLAIN>(g, make_src(C, H, W, OH, OW, OC, KH, KW, SH, SW, PH, PW),
                                                              splits, nullptr, 0, st);
    if (rc != ODL_OK)
        return fail(rc, "conv2d_backward: no kernel variant");
    ODL_LAUNCH_CHECK();
    if (splits > 1)
    {
        launch_splitk_reduce(static_cast<const float *>(workspace), splits, OC * K, gw, OC, K, K, nullptr, 0, st);
        ODL_LAUNCH_CHECK();
    }
    return ODL_OK;
}

// gx[n][c][h][w] = sum_{kh,kw,oc} W[oc][c][kh][kw] * gy2d[(n, h+PH-kh, w+PW-kw)][oc]   (stride 1)
int conv_implicit_dgrad(const float *gy, const float *w, float *gx, int64_t N, int64_t C, int64_t H, int64_t W,
                        int64_t OC, int KH, int KW, int PH, int PW, int64_t OH, int64_t OW, void *workspace,
                        size_t workspace_bytes, hipStream_t st)
{
    const size_t need = dgrad_wp_bytes(C, OC, KH, KW);  // the tail partials behind it are optional
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= need, "conv2d_backward: workspace of %zu bytes required",
                need);
    float *wp = static_cast<float *>(workspace);
    const int64_t total = OC * C * KH * KW;
    hipLaunchKernelGGL(permute_weight_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, st, w, wp, (int)OC,
                       (int)C, KH * KW);
    ODL_LAUNCH_CHECK();
    GemmArgs g{};
    g.A = wp, g.B = gy, g.C = gx, g.bias = nullptr;
    g.M = C, g.N = N * H * W, g.K = (int64_t)KH * KW * OC;
    g.lda = g.K, g.ldb = 0, g.ldc = 0, g.P = H * W;
    g.k_per_split = g.K, g.c_split_stride = 0;
    int rc = launch_conv_tile<SB_CONV_DGRAD, false, EPI_NCHW_ROWB>(g, make_src(C, H, W, OH, OW, OC, KH, KW, 1, 1, PH, PW),
                                                                   1, static_cast<char *>(workspace) + need,
                                                                   workspace_bytes - need, st);
    if (rc != ODL_OK)
        return fail(rc, "conv2d_backward: no kernel variant");
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

size_t sgemm_workspace(int64_t M, int64_t N, int64_t K, int split_k)
{
    const int s = pick_splits(M, N, K, split_k);
    if (s > 1)
        return (size_t)s * M * N * sizeof(float);
    return pick_tile(M, N) == 128 ? plan_tail(ceil_div(M, 128) * ceil_div(N, 128), K, 128, 128).bytes : 0;
}
}  // namespace odl

extern "C" {

int odl_hip_sgemm(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                  const float *B, int64_t ldb, float *C, int64_t ldc, const float *bias, int split_k, void *workspace,
                  size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    return odl::sgemm_launch(trans_a, trans_b, M, N, K, A, lda, B, ldb, C, ldc, bias, bias ? EPI_BIAS_COL : EPI_PLAIN,
                             0, split_k, workspace, workspace_bytes, odl::as_stream(stream));
}

int odl_hip_linear_act(const float *x, const float *w, const float *b, int64_t M, int64_t N, int64_t K, int activation,
                       float *y, void *workspace, size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(b != nullptr, "linear: null bias");
    ODL_REQUIRE(activation == -1 || activation == 0 || activation == 7,
                "linear: activation must be -1 (none), 0 (relu) or 7 (silu), the unary operator numbers; got %d", activation);
    const int act = activation == 0 ? 1 : (activation == 7 ? 2 : 0);
    return odl::sgemm_launch(0, 0, M, N, K, x, K, w, N, y, N, b, EPI_BIAS_COL, 0, 0, workspace, workspace_bytes,
                             odl::as_stream(stream), act);
}

size_t odl_hip_sgemm_workspace_bytes(int, int, int64_t M, int64_t N, int64_t K, int split_k)
{
    return odl::sgemm_workspace(M, N, K, split_k);
}

size_t odl_hip_matmul_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K, int b_is_batched)
{
    return b_is_batched ? odl::sgemm_workspace(M, N, K, 0) : odl::sgemm_workspace(batch * M, N, K, 0);
}

int odl_hip_matmul(const float *a, const float *b, float *c, int64_t batch, int64_t M, int64_t N, int64_t K,
                   int b_is_batched, void *workspace, size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(batch >= 1, "matmul: batch must be >= 1");
    if (!b_is_batched)  // [batch*M, K] x [K, N]: one GEMM, the batch folds into the rows
        return odl::sgemm_launch(0, 0, batch * M, N, K, a, K, b, N, c, N, nullptr, EPI_PLAIN, 0, 0, workspace,
                                 workspace_bytes, odl::as_stream(stream));
    for (int64_t i = 0; i < batch; ++i)
    {
        int rc = odl::sgemm_launch(0, 0, M, N, K, a + i * M * K, K, b + i * K * N, N, c + i * M * N, N, nullptr,
                                   EPI_PLAIN, 0, 0, workspace, workspace_bytes, odl::as_stream(stream));
        if (rc != ODL_OK)
            return rc;
    }
    return ODL_OK;
}

size_t odl_hip_matmul_backward_workspace_bytes(int64_t M, int64_t K, int64_t N)
{
    const size_t a = odl::sgemm_workspace(M, K, N, 0), b = odl::sgemm_workspace(K, N, M, 0);
    return a > b ? a : b;
}

int odl_hip_matmul_backward(const float *x, const float *w, const float *gy, float *gx, float *gw, int64_t M, int64_t K,
                            int64_t N, void *workspace, size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    hipStream_t st = odl::as_stream(stream);
    if ((gx || gw) && x && w && gy && M > 0 && odl::skinny_ok(M, N, K))
        return odl::skinny_backward(x, w, gy, gx, gw, nullptr, M, K, N, st);  // both gradients of a classifier layer in one launch
    if (gx && gw && x && w && gy)
    {
        const int paired = odl::matmul_backward_pair(x, w, gy, gx, gw, M, K, N, st);
        if (paired < 0)
            return paired;
        if (paired == 1)
        {
            ODL_LAUNCH_CHECK();
            return ODL_OK;
        }
    }
    if (gx)  // gx[M,K] = gy[M,N] . w[K,N]^T
    {
        int rc = odl::sgemm_launch(0, 1, M, K, N, gy, N, w, N, gx, K, nullptr, EPI_PLAIN, 0, 0, workspace,
                                   workspace_bytes, st);
        if (rc != ODL_OK)
            return rc;
    }
    if (gw)  // gw[K,N] = x[M,K]^T . gy[M,N]
    {
        int rc = odl::sgemm_launch(1, 0, K, N, M, x, K, gy, N, gw, N, nullptr, EPI_PLAIN, 0, 0, workspace,
                                   workspace_bytes, st);
        if (rc != ODL_OK)
            return rc;
    }
    return ODL_OK;
}

size_t odl_hip_linear_backward_workspace_bytes(int64_t M, int64_t K, int64_t N)
{
    const size_t a = odl_hip_matmul_backward_workspace_bytes(M, K, N), b = odl_hip_sum_axis_workspace_bytes(1, M, N);
    return a > b ? a : b;
}

int odl_hip_linear_backward(const float *x, const float *w, const float *gy, float *gx, float *gw, float *gb, int64_t M,
                            int64_t K, int64_t N, void *workspace, size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(M >= 0 && K >= 0 && N >= 0, "linear_backward: negative dimension");
    ODL_REQUIRE(gy != nullptr || M * N == 0, "linear_backward: gy is null");
    // a classifier layer: the three gradients in one launch
    if (gb && (gx || gw) && x && w && gy && M > 0 && odl::skinny_ok(M, N, K) && odl::skinny_bias_ok(M, N))
        return odl::skinny_backward(x, w, gy, gx, gw, gb, M, K, N, odl::as_stream(stream));
    if (gb && gx && gw && x && w && gy && M > 0 && !odl::skinny_ok(M, N, K))
    {
        // both matrix gradients as one launch of two products, the column sum as a few more workgroups of it
        bool gb_done = false;
        const int paired = odl::matmul_backward_pair(x, w, gy, gx, gw, M, K, N, odl::as_stream(stream), gb, &gb_done);
        if (paired < 0)
            return paired;
        if (paired == 1)
        {
            ODL_LAUNCH_CHECK();
            if (gb_done)
                return ODL_OK;
            return odl_hip_sum_axis(gy, 1, M, N, gb, workspace, workspace_bytes, stream);
        }
    }
    if (gx || gw)
    {
        const int rc = odl_hip_matmul_backward(x, w, gy, gx, gw, M, K, N, workspace, workspace_bytes, stream);
        if (rc != ODL_OK)
            return rc;
    }
    if (gb)  // (stream order: the workspace is free again)
        return odl_hip_sum_axis(gy, 1, M, N, gb, workspace, workspace_bytes, stream);
    return ODL_OK;
}

int odl_hip_transpose(const float *src, float *dst, int64_t outer, int64_t rows, int64_t cols, void *stream)
{
    ODL_REQUIRE_DEVICE();
    if (outer * rows * cols == 0)
        return ODL_OK;
    ODL_REQUIRE(outer > 0 && rows > 0 && cols > 0, "transpose: bad dimensions");
    return odl::transpose_launch(src, dst, 4, outer, rows, cols, odl::as_stream(stream));
}

}  // extern "C"
