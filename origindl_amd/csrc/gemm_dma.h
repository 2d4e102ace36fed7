// C = A . B for products whose tiles leave about one workgroup per compute unit: operands go from global memory straight
// into LDS (no registers in between), four K slabs deep. Declared here for gemm.hip, which picks the variant.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace odl
{
struct DmaGemmArgs
{
    const float *A, *B, *bias;
    float *C;
    int64_t M, N, K, lda, ldb, ldc;
    int tiles_m, tiles_n, splits;
    int64_t k_per_split;     // K range of one slice (a multiple of 32)
    int64_t c_split_stride;  // distance between the partial outputs of two slices (0 when splits == 1)
    int epi;                 // 0 plain, 1 bias by column then the activation, 2 bias by row then the activation
    int act;                 // 0 none, 1 relu, 2 silu
    int xcds;
    // Tail split (0 pieces: none): the tiles from tail_first on are cut into tail_splits runs of tail_kps K values each,
    // done by the workgroups from main_blocks on, which write their raw [BM][BN] accumulators to tail_ws, one block
    // per (tile, piece); a fix-up kernel of the caller adds the pieces in order and finishes those tiles.
    int main_blocks, tail_first, tail_splits;
    int64_t tail_kps;
    float *tail_ws;
    // `batch` independent products in one launch (1: a single product): product z reads A + z*a_batch, B + z*b_batch
    // and writes C + z*c_batch (elements). Not combined with K slices or a split tail.
    int batch;
    int64_t a_batch, b_batch, c_batch;
    // c_p > 0 (64-wide tiles only, with epi == 2): column n of the product is (image n / c_p, position n % c_p) and goes to
    // C[(image * M + row) * c_p + position] — an NCHW tensor of M channels, the bias by row
    int64_t c_p;
};

// true when the shape suits the variant (16-byte aligned rows, offsets within 31 bits)
bool sgemm_dma_fits(bool ta, bool tb, const DmaGemmArgs &g);
// tile: 32 (64x32 tiles in 64-wide slabs, four wave sets), 64 (64x64 tiles, one workgroup per compute unit), 128 (128x128 tiles, one per compute unit) or 129 (128x128
// tiles in 16-wide slabs, two workgroups per compute unit: for launches of many tiles); the grid is
// tiles_m * tiles_n * splits workgroups of 512 threads (main_blocks + tail tiles * tail_splits with a tail split)
int sgemm_dma_launch(int tile, bool ta, bool tb, const DmaGemmArgs &g, hipStream_t st);

// Two whole products in one launch, two workgroups per compute unit: g0 = X.Y^T (A [M,K] and B [N,K] row-major) on tiles
// of class tile0, g1 = X^T.Y (A [K,M] and B [K,N] row-major) on tiles of class tile1. Classes: 64 (64x64 tiles), 32 (64x32
// tiles) — these two mix freely — or 128 for both (128x128 tiles). tiles_m / tiles_n of each product count its own tiles.
// `sums` (may be null): a small column sum (reduce_small.h) run by `blocks` more workgroups of the same launch — the bias
// gradient beside a layer's two matrix gradients: dst[c] = sum over the `axis` rows of src[:, c], `inner` columns; quads:
// four columns a lane (inner % 4 == 0, src 16-byte aligned), else one.
struct ColSumJob
{
    const float *src;
    float *dst;
    int64_t axis, inner;
    int quads;
    unsigned blocks;
};
int sgemm_dma_pair_launch(int tile0, const DmaGemmArgs &g0, int tile1, const DmaGemmArgs &g1, hipStream_t st,
                          const ColSumJob *sums = nullptr);

// 1x1 / stride 1 / unpadded convolution as `N` products y[n] = act(W[OC,C] . x[n][C, H*W] + b[oc]) in one launch; false
// when the shape does not suit (rows of H*W or C floats that are not multiples of four, unaligned pointers)
bool conv1x1_dma_ok(const float *x, const float *w, int64_t N, int64_t C, int64_t HW, int64_t OC);
int conv1x1_dma(const float *x, const float *w, const float *b, float *y, int64_t N, int64_t C, int64_t HW, int64_t OC,
                int act, hipStream_t st);
}  // namespace odl
