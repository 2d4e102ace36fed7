// The element types besides float32. The reference dispatches every elementwise, reduction and conversion operator over
// six element types (include/origin/mat/origin/device_common/type_dispatcher.h:26-88); float32 is the type the hot path
// computes in and has the tuned kernels of the other files. This file gives the remaining five (float64, int8, int32,
// int64, uint8) the same operators as plain streaming kernels: conversion between any two types
// (src/mat/origin/cuda/type_conversion.cu; a static_cast per element), add/subtract/multiply/divide and the comparisons,
// the unary set, pow with a scalar exponent, fills, and sums over an axis. Type codes are the reference's DataType
// enumerators (include/origin/mat/basic_types.h:19-27).
#include "odl_common.h"

#include <type_traits>

namespace
{
constexpr int kBlock = 256;

enum : int
{
    DT_F32 = 0,
    DT_F64 = 1,
    DT_I8 = 2,
    DT_I32 = 3,
    DT_I64 = 4,
    DT_U8 = 5,
    DT_COUNT = 6,
};

inline size_t dtype_bytes(int dt)
{
    switch (dt)
    {
        case DT_F64:
        case DT_I64: return 8;
        case DT_I8:
        case DT_U8: return 1;
        default: return 4;
    }
}

// calls f with a value of the element type
template <typename F>
int with_type(int dt, F &&f)
{
    switch (dt)
    {
        case DT_F32: return f(float{});
        case DT_F64: return f(double{});
        case DT_I8: return f(int8_t{});
        case DT_I32: return f(int32_t{});
        case DT_I64: return f(int64_t{});
        case DT_U8: return f(uint8_t{});
        default: return odl::fail(ODL_ERR_INVALID_ARG, "unknown element type code %d", dt);
    }
}

inline unsigned grid_for(int64_t n)
{
    const int64_t b = odl::ceil_div(n, kBlock);
    return (unsigned)(b < 65536 ? b : 65536);  // the kernels stride over what one pass does not cover
}

template <typename S, typename D>
__global__ void convert_kernel(const S *__restrict__ src, D *__restrict__ dst, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        dst[i] = static_cast<D>(src[i]);
}

template <typename T>
struct is_float_type
{
    static constexpr bool value = false;
};
template <>
struct is_float_type<float>
{
    static constexpr bool value = true;
};
template <>
struct is_float_type<double>
{
    static constexpr bool value = true;
};

// integer arithmetic wraps (computed in the unsigned type of the same width); a zero divisor gives 0 instead of a trap
template <typename T>
__device__ inline T bin_op(int op, T a, T b)
{
    if constexpr (is_float_type<T>::value)
    {
        switch (op)
        {
            case 0: return a + b;
            case 1: return a - b;
            case 2: return a * b;
            case 3: return a / b;
        }
    }
    else
    {
        using U = typename std::make_unsigned<T>::type;
        switch (op)
        {
            case 0: return (T)((U)a + (U)b);
            case 1: return (T)((U)a - (U)b);
            case 2: return (T)((U)a * (U)b);
            case 3: return b == 0 ? (T)0 : (T)(a / b);
        }
    }
    // comparisons give a 0/1 mask in the operands' own type (operation_templates.h:177-240)
    switch (op)
    {
        case 4: return (T)(a > b);
        case 5: return (T)(a == b);
        case 6: return (T)(a != b);
        case 7: return (T)(a < b);
        case 8: return (T)(a <= b);
        default: return (T)(a >= b);
    }
}

// mode 0: a[i] op b[i]; 1: a[i] op b[0]; 2: a[0] op b[i]
template <typename T>
__global__ void binary_kernel(int op, int mode, const T *a, const T *b, T *out, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        out[i] = bin_op<T>(op, a[mode == 2 ? 0 : i], b[mode == 1 ? 0 : i]);
}

template <typename T>
__device__ inline T un_op(int op, T v)
{
    switch (op)
    {
        case 0: return v > (T)0 ? v : (T)0;
        case 3:
            if constexpr (is_float_type<T>::value)
                return -v;
            else
                return (T)((typename std::make_unsigned<T>::type)0 - (typename std::make_unsigned<T>::type)v);
        case 4:
            if constexpr (is_float_type<T>::value)
                return v * v;
            else
                return (T)((typename std::make_unsigned<T>::type)v * (typename std::make_unsigned<T>::type)v);
    }
    if constexpr (is_float_type<T>::value)
    {
        switch (op)
        {
            case 1: return (T)exp((double)v);
            case 2: return (T)log((double)v);
            case 5: return (T)sqrt((double)v);
        }
        const double s = 1.0 / (1.0 + exp(-(double)v));
        return (T)(op == 6 ? s : (double)v * s);
    }
    return v;
}

template <typename T>
__global__ void unary_kernel(int op, const T *a, T *out, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        out[i] = un_op<T>(op, a[i]);
}

__global__ void pow_f64_kernel(const double *a, double *out, int64_t n, double e)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        out[i] = pow(a[i], e);
}

template <typename T>
__global__ void fill_kernel(T *dst, int64_t n, T v)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        dst[i] = v;
}

// ---- sums. Integer sums are taken in 64-bit unsigned arithmetic and cut to the element type at the end, which is the
// wrapped sum whatever the order of the additions; float64 sums are added in a fixed (parallel) order.
template <typename T>
struct Acc
{
    using type = uint64_t;
};
template <>
struct Acc<float>
{
    using type = float;
};
template <>
struct Acc<double>
{
    using type = double;
};

template <typename T>
__device__ inline typename Acc<T>::type widen(T v)
{
    if constexpr (is_float_type<T>::value)
        return v;
    else
        return (uint64_t)(int64_t)v;
}

// rows: src[outer][axis] (inner == 1). One workgroup per (row, slice), both folded into the grid's first
// dimension (its 2^31 limit, not the 65535 of the second, bounds the row count); partial[slice * outer + row].
template <typename T>
__global__ __launch_bounds__(kBlock) void row_partial_kernel(const T *__restrict__ src, typename Acc<T>::type *__restrict__ part,
                                                             int64_t outer, int64_t axis, int64_t chunk, int slices)
{
    using A = typename Acc<T>::type;
    __shared__ A red[kBlock];
    const int64_t row = blockIdx.x / (unsigned)slices, slice = blockIdx.x % (unsigned)slices;
    const int64_t k0 = slice * chunk, k1 = (k0 + chunk < axis) ? k0 + chunk : axis;
    A s = 0;
    for (int64_t k = k0 + threadIdx.x; k < k1; k += kBlock)
        s += widen<T>(src[row * axis + k]);
    red[threadIdx.x] = s;
    __syncthreads();
    for (int w = kBlock / 2; w > 0; w >>= 1)
    {
        if ((int)threadIdx.x < w)
            red[threadIdx.x] += red[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0)
        part[slice * outer + row] = red[0];
}

// columns: src[outer][axis][inner], lanes along inner. partial[slice * nout + (o * inner + i)].
template <typename T>
__global__ void col_partial_kernel(const T *__restrict__ src, typename Acc<T>::type *__restrict__ part, int64_t outer,
                                   int64_t axis, int64_t inner, int64_t chunk)
{
    using A = typename Acc<T>::type;
    const int64_t nout = outer * inner;
    const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= nout)
        return;
    const int64_t o = c / inner, i = c - o * inner, slice = blockIdx.y;
    const int64_t k0 = slice * chunk, k1 = (k0 + chunk < axis) ? k0 + chunk : axis;
    A s = 0;
    for (int64_t k = k0; k < k1; ++k)
        s += widen<T>(src[(o * axis + k) * inner + i]);
    part[slice * nout + c] = s;
}

// through_float: the whole-tensor sum of the reference passes through a float on its way back into the element type
// (src/mat/origin/cpu/math/sum.cpp:18-35, 83-90)
template <typename T>
__global__ void fold_kernel(const typename Acc<T>::type *__restrict__ part, T *__restrict__ dst, int64_t nout, int64_t slices,
                            int through_float)
{
    using A = typename Acc<T>::type;
    const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= nout)
        return;
    A s = 0;
    for (int64_t z = 0; z < slices; ++z)
        s += part[z * nout + c];
    T v;
    if constexpr (is_float_type<T>::value)
        v = (T)s;
    else
        v = (T)(typename std::make_unsigned<T>::type)s;
    if (through_float)
        v = static_cast<T>(static_cast<float>(v));
    dst[c] = v;
}

// permute: out[o0..] = in[..] with output dimension d taken from input dimension perm[d]; one thread per output
// element (lanes along the output's last dimension: coalesced writes), the input offset rebuilt from the output index
struct PermuteDims
{
    int nd;
    int64_t oshape[8];
    int64_t istride[8];  // stride in the input of the dimension that became output dimension d
};

template <typename T>
__global__ void permute_kernel(const T *__restrict__ src, T *__restrict__ dst, int64_t total, PermuteDims d)
{
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x)
    {
        int64_t r = t, si = 0;
        for (int k = d.nd - 1; k >= 0; --k)
        {
            si += (r % d.oshape[k]) * d.istride[k];
            r /= d.oshape[k];
        }
        dst[t] = src[si];
    }
}

// Batched 2-D transposition dst[o][c][r] = src[o][r][c] through 64x64 tiles in LDS (rows padded to 65: the column-wise
// reads of the second phase hit 32 different banks). Lanes run along the contiguous side in both phases: a wave reads
// 64 consecutive elements of a source row and writes 64 consecutive elements of a destination row. One workgroup of 256
// threads per tile, tiles numbered with the source's column tiles fastest.
struct TransposeGeom
{
    int64_t rows, cols;
    unsigned tiles_c, tiles_r;
    odl::FastDiv d_tiles, d_group;  // by tiles_r * tiles_c, by kTileGroup * tiles_c
};

// Tile order inside one matrix: groups of 16 tile-rows, inside a group down the rows first. The couple of thousand
// workgroups in flight then read runs of many KB of each source row and write 4 KB runs of each destination row; with
// the source's column tiles fastest every workgroup's 64 destination rows had their DRAM pages to themselves
// (16384 x 4096: 58 % of HBM).
constexpr unsigned kTileGroup = 16;

__device__ inline void transpose_tile_of(const TransposeGeom &g, unsigned bid, unsigned &o, unsigned &tr, unsigned &tc)
{
    o = odl::fastdiv(bid, g.d_tiles);
    const unsigned t = bid - o * (g.tiles_r * g.tiles_c);
    const unsigned grp = odl::fastdiv(t, g.d_group), in_g = t - grp * (kTileGroup * g.tiles_c);
    const unsigned first = grp * kTileGroup;
    const unsigned gm = g.tiles_r - first < kTileGroup ? g.tiles_r - first : kTileGroup;
    tc = gm == kTileGroup ? in_g / kTileGroup : in_g / gm;
    tr = first + (in_g - tc * gm);
}

template <typename T>
__global__ __launch_bounds__(256) void transpose_tile_kernel(const T *__restrict__ src, T *__restrict__ dst, TransposeGeom g)
{
    __shared__ T tile[64][65];
    unsigned o, tr, tc;
    transpose_tile_of(g, blockIdx.x, o, tr, tc);
    const int64_t r0 = (int64_t)tr * 64, c0 = (int64_t)tc * 64;
    const T *s = src + (int64_t)o * g.rows * g.cols;
    T *d = dst + (int64_t)o * g.rows * g.cols;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll 4
    for (int i = wave; i < 64; i += 4)
    {
        const int64_t r = r0 + i, c = c0 + lane;
        if (r < g.rows && c < g.cols)
            tile[i][lane] = s[r * g.cols + c];
    }
    __syncthreads();
#pragma unroll 4
    for (int i = wave; i < 64; i += 4)
    {
        const int64_t c = c0 + i, r = r0 + lane;
        if (r < g.rows && c < g.cols)
            d[c * g.rows + r] = tile[lane][i];
    }
}

// A matrix with at most 128 rows (the detection head's [85][H*W] planes): a workgroup takes all rows of 64 columns, whose
// transposed image is one contiguous run of the destination. Lanes along the columns while reading, along that run
// while writing; LDS rows padded to an odd length.
template <typename T>
__global__ __launch_bounds__(256) void transpose_few_rows_kernel(const T *__restrict__ src, T *__restrict__ dst, int rows,
                                                                  int64_t cols, unsigned tiles_c, odl::FastDiv d_tc,
                                                                  odl::FastDiv d_rows)
{
    extern __shared__ unsigned char few_raw[];
    T *tile = reinterpret_cast<T *>(few_raw);
    const int ld = rows | 1;
    const unsigned o = odl::fastdiv(blockIdx.x, d_tc), tc = blockIdx.x - o * tiles_c;
    const int64_t c0 = (int64_t)tc * 64;
    const int ncols = cols - c0 < 64 ? (int)(cols - c0) : 64;
    const T *s = src + (int64_t)o * rows * cols;
    T *d = dst + (int64_t)o * rows * cols + c0 * rows;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane < ncols)
    {
#pragma unroll 4
        for (int r = wave; r < rows; r += 4)
            tile[lane * ld + r] = s[(int64_t)r * cols + c0 + lane];
    }
    __syncthreads();
    const int n = ncols * rows;
#pragma unroll 4
    for (int e = threadIdx.x; e < n; e += 256)
    {
        const unsigned c = odl::fastdiv((unsigned)e, d_rows);
        d[e] = tile[c * ld + (e - c * rows)];
    }
}

// The mirror image: at most 128 columns. 64 source rows are one contiguous run; lanes along it while reading, along the
// rows (the destination's contiguous side) while writing.
template <typename T>
__global__ __launch_bounds__(256) void transpose_few_cols_kernel(const T *__restrict__ src, T *__restrict__ dst, int64_t rows,
                                                                  int cols, unsigned tiles_r, odl::FastDiv d_tr,
                                                                  odl::FastDiv d_cols)
{
    __shared__ T tile[128 * 65];
    const unsigned o = odl::fastdiv(blockIdx.x, d_tr), tr = blockIdx.x - o * tiles_r;
    const int64_t r0 = (int64_t)tr * 64;
    const int nrows = rows - r0 < 64 ? (int)(rows - r0) : 64;
    const T *s = src + (int64_t)o * rows * cols + r0 * cols;
    T *d = dst + (int64_t)o * rows * cols;
    const int n = nrows * cols;
#pragma unroll 4
    for (int e = threadIdx.x; e < n; e += 256)
    {
        const unsigned r = odl::fastdiv((unsigned)e, d_cols);
        tile[(e - r * cols) * 65 + r] = s[e];
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane < nrows)
    {
#pragma unroll 4
        for (int c = wave; c < cols; c += 4)
            d[(int64_t)c * rows + r0 + lane] = tile[c * 65 + lane];
    }
}

// The same for 4-byte elements when rows and cols are multiples of 4 and both bases are 16-byte aligned: 16 bytes per
// lane on both sides (a wave reads 4 source rows x 256 bytes and writes 4 destination rows x 256 bytes); in LDS the lanes
// of a wave touch (4*cq + r) mod 32 = 32 different banks, twice each.
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void transpose_tile_vec_kernel(const unsigned *__restrict__ src, unsigned *__restrict__ dst,
                                                                  TransposeGeom g)
{
    constexpr int TR = 64, TC = 64;  // (128x64 and 64x128 tiles measured the same)
    __shared__ unsigned tile[TC][TR + 1];
    unsigned o, tr, tc;
    transpose_tile_of(g, blockIdx.x, o, tr, tc);
    const int64_t r0 = (int64_t)tr * TR, c0 = (int64_t)tc * TC;
    const unsigned *s = src + (int64_t)o * g.rows * g.cols;
    unsigned *d = dst + (int64_t)o * g.rows * g.cols;
    {
        constexpr int QPR = TC / 4, LINES = 256 / QPR;  // quads across a source row of the tile, rows per pass
        const int quad = threadIdx.x % QPR, line = threadIdx.x / QPR;
#pragma unroll
        for (int i = 0; i < TR / LINES; ++i)
        {
            const int rr = line + LINES * i;
            const int64_t r = r0 + rr, c = c0 + 4 * quad;
            if (r < g.rows && c < g.cols)
            {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(s + r * g.cols + c);
                tile[4 * quad + 0][rr] = v[0], tile[4 * quad + 1][rr] = v[1];
                tile[4 * quad + 2][rr] = v[2], tile[4 * quad + 3][rr] = v[3];
            }
        }
    }
    __syncthreads();
    {
        constexpr int QPR = TR / 4, LINES = 256 / QPR;
        const int quad = threadIdx.x % QPR, line = threadIdx.x / QPR;
#pragma unroll
        for (int i = 0; i < TC / LINES; ++i)
        {
            const int cc = line + LINES * i;
            const int64_t c = c0 + cc, r = r0 + 4 * quad;
            if (r < g.rows && c < g.cols)
            {
                u32x4 v;
                v[0] = tile[cc][4 * quad + 0], v[1] = tile[cc][4 * quad + 1];
                v[2] = tile[cc][4 * quad + 2], v[3] = tile[cc][4 * quad + 3];
                *reinterpret_cast<u32x4 *>(d + c * g.rows + r) = v;
            }
        }
    }
}

struct SumPlan
{
    int64_t slices, chunk;
    size_t ws_bytes;
};

SumPlan plan_sum(int64_t outer, int64_t axis, int64_t inner)
{
    SumPlan p{1, axis > 0 ? axis : 1, 0};
    const int64_t nout = outer * inner;
    const int64_t want_wgs = 4 * (int64_t)odl::device_cus();
    const int64_t have = inner == 1 ? outer : odl::ceil_div(nout, kBlock);
    int64_t s = odl::ceil_div(want_wgs, have > 0 ? have : 1);
    const int64_t per = inner == 1 ? 4 * kBlock : 32;  // least elements of the axis worth a slice
    if (s > axis / per)
        s = axis / per;
    if (s < 1)
        s = 1;
    if (s > 4096)
        s = 4096;
    p.chunk = odl::ceil_div(axis > 0 ? axis : 1, s);
    p.slices = odl::ceil_div(axis > 0 ? axis : 1, p.chunk);
    p.ws_bytes = (size_t)(p.slices * nout) * 8;
    return p;
}
}  // namespace

namespace odl
{
// dst[o][c][r] = src[o][r][c] for elements of 1, 4 or 8 bytes; ODL_ERR_INVALID_ARG when the tile count does not fit a grid
int transpose_launch(const void *src, void *dst, int elem_bytes, int64_t outer, int64_t rows, int64_t cols, hipStream_t st)
{
    if (outer * rows * cols == 0)
        return ODL_OK;
    const bool vec = elem_bytes == 4 && rows % 4 == 0 && cols % 4 == 0 &&
                     ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0;
    if (elem_bytes == 4 && (rows <= 128) != (cols <= 128))
    {
        // one narrow side: whole rows (or columns) of 64 columns (rows) per workgroup
        const bool few_rows = rows <= 128;
        const int64_t tiles = ceil_div(few_rows ? cols : rows, 64);
        if (tiles < (1ll << 31) && outer * tiles < (1ll << 31))
        {
            const dim3 grid((unsigned)(outer * tiles));
            if (few_rows)
                hipLaunchKernelGGL((transpose_few_rows_kernel<uint32_t>), grid, dim3(256), (size_t)64 * ((int)rows | 1) * 4, st,
                                   static_cast<const uint32_t *>(src), static_cast<uint32_t *>(dst), (int)rows, cols,
                                   (unsigned)tiles, make_fastdiv((unsigned)tiles), make_fastdiv((unsigned)rows));
            else
                hipLaunchKernelGGL((transpose_few_cols_kernel<uint32_t>), grid, dim3(256), 0, st,
                                   static_cast<const uint32_t *>(src), static_cast<uint32_t *>(dst), rows, (int)cols,
                                   (unsigned)tiles, make_fastdiv((unsigned)tiles), make_fastdiv((unsigned)cols));
            ODL_LAUNCH_CHECK();
            return ODL_OK;
        }
    }
    const int64_t tr = ceil_div(rows, 64), tc = ceil_div(cols, 64);
    if (tr >= (1ll << 31) || tc >= (1ll << 31) || outer * tr * tc >= (1ll << 31))
        return fail(ODL_ERR_INVALID_ARG, "transpose: too many tiles");
    if (tr * tc >= (1ll << 31) || kTileGroup * tc >= (1ll << 31))
        return fail(ODL_ERR_INVALID_ARG, "transpose: too many tiles");
    const TransposeGeom g{rows, cols, (unsigned)tc, (unsigned)tr, make_fastdiv((unsigned)(tr * tc)),
                          make_fastdiv((unsigned)(kTileGroup * tc))};
    const dim3 grid((unsigned)(outer * tr * tc)), block(256);
    if (vec)
        hipLaunchKernelGGL(transpose_tile_vec_kernel, grid, block, 0, st, static_cast<const unsigned *>(src),
                           static_cast<unsigned *>(dst), g);
    else if (elem_bytes == 1)
        hipLaunchKernelGGL((transpose_tile_kernel<uint8_t>), grid, block, 0, st, static_cast<const uint8_t *>(src),
                           static_cast<uint8_t *>(dst), g);
    else if (elem_bytes == 8)
        hipLaunchKernelGGL((transpose_tile_kernel<uint64_t>), grid, block, 0, st, static_cast<const uint64_t *>(src),
                           static_cast<uint64_t *>(dst), g);
    else
        hipLaunchKernelGGL((transpose_tile_kernel<uint32_t>), grid, block, 0, st, static_cast<const uint32_t *>(src),
                           static_cast<uint32_t *>(dst), g);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}
}  // namespace odl

extern "C" {

size_t odl_hip_dtype_size(int dtype)
{
    return (dtype >= 0 && dtype < DT_COUNT) ? dtype_bytes(dtype) : 0;
}

int odl_hip_convert(const void *src, int src_dtype, void *dst, int dst_dtype, int64_t n, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(n >= 0, "convert: negative size");
    ODL_REQUIRE(src_dtype >= 0 && src_dtype < DT_COUNT && dst_dtype >= 0 && dst_dtype < DT_COUNT,
                "convert: unknown element type code (%d -> %d)", src_dtype, dst_dtype);
    if (n == 0)
        return ODL_OK;
    ODL_REQUIRE(src && dst, "convert: null operand");
    hipStream_t st = odl::as_stream(stream);
    return with_type(src_dtype, [&](auto s) {
        using S = decltype(s);
        return with_type(dst_dtype, [&](auto d) {
            using D = decltype(d);
            hipLaunchKernelGGL((convert_kernel<S, D>), dim3(grid_for(n)), dim3(kBlock), 0, st, static_cast<const S *>(src),
                               static_cast<D *>(dst), n);
            ODL_LAUNCH_CHECK();
            return ODL_OK;
        });
    });
}

int odl_hip_binary_dtype(int op, int dtype, const void *a, int64_t na, const void *b, int64_t nb, void *out, void *stream)
{
    if (dtype == DT_F32)
        return odl_hip_binary(op, static_cast<const float *>(a), na, static_cast<const float *>(b), nb,
                              static_cast<float *>(out), stream);
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(op >= 0 && op <= 9, "binary: op %d is not defined for this element type", op);
    ODL_REQUIRE(na >= 0 && nb >= 0, "binary: negative extent");
    if (!(na == nb || na == 1 || nb == 1))
        return odl::fail(ODL_ERR_RUNTIME, "Complex broadcasting not yet implemented (%lld vs %lld elements)", (long long)na,
                         (long long)nb);
    if (na == 0 || nb == 0)
        return ODL_OK;
    ODL_REQUIRE(a && b && out, "binary: null operand");
    const int64_t n = na > nb ? na : nb;
    const int mode = (na == nb) ? 0 : (nb == 1 ? 1 : 2);
    hipStream_t st = odl::as_stream(stream);
    return with_type(dtype, [&](auto t) {
        using T = decltype(t);
        hipLaunchKernelGGL((binary_kernel<T>), dim3(grid_for(n)), dim3(kBlock), 0, st, op, mode, static_cast<const T *>(a),
                           static_cast<const T *>(b), static_cast<T *>(out), n);
        ODL_LAUNCH_CHECK();
        return ODL_OK;
    });
}

int odl_hip_unary_dtype(int op, int dtype, const void *a, int64_t n, void *out, void *stream)
{
    if (dtype == DT_F32)
        return odl_hip_unary(op, static_cast<const float *>(a), n, static_cast<float *>(out), stream);
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(op >= 0 && op <= 7, "unary: unknown op %d", op);
    ODL_REQUIRE(dtype >= 0 && dtype < DT_COUNT, "unary: unknown element type code %d", dtype);
    // exp, log, sqrt, sigmoid and silu are defined for the floating-point types only (the reference throws for integers)
    ODL_REQUIRE(dtype == DT_F64 || op == 0 || op == 3 || op == 4, "unary: op %d needs a floating-point element type", op);
    if (n <= 0)
        return ODL_OK;
    ODL_REQUIRE(a && out, "unary: null operand");
    hipStream_t st = odl::as_stream(stream);
    return with_type(dtype, [&](auto t) {
        using T = decltype(t);
        hipLaunchKernelGGL((unary_kernel<T>), dim3(grid_for(n)), dim3(kBlock), 0, st, op, static_cast<const T *>(a),
                           static_cast<T *>(out), n);
        ODL_LAUNCH_CHECK();
        return ODL_OK;
    });
}

int odl_hip_pow_scalar_dtype(int dtype, const void *a, int64_t n, double exponent, void *out, void *stream)
{
    if (dtype == DT_F32)
        return odl_hip_pow_scalar(static_cast<const float *>(a), n, (float)exponent, static_cast<float *>(out), stream);
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(dtype == DT_F64, "pow: element type %d is not floating point (the operator promotes integers first)", dtype);
    if (n <= 0)
        return ODL_OK;
    ODL_REQUIRE(a && out, "pow: null operand");
    hipLaunchKernelGGL(pow_f64_kernel, dim3(grid_for(n)), dim3(kBlock), 0, odl::as_stream(stream),
                       static_cast<const double *>(a), static_cast<double *>(out), n, exponent);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_fill_dtype(void *dst, int dtype, int64_t n, const void *host_value, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(host_value != nullptr, "fill: null value");
    if (n <= 0)
        return ODL_OK;
    ODL_REQUIRE(dst != nullptr, "fill: null destination");
    hipStream_t st = odl::as_stream(stream);
    return with_type(dtype, [&](auto t) {
        using T = decltype(t);
        T v;
        __builtin_memcpy(&v, host_value, sizeof(T));
        hipLaunchKernelGGL((fill_kernel<T>), dim3(grid_for(n)), dim3(kBlock), 0, st, static_cast<T *>(dst), n, v);
        ODL_LAUNCH_CHECK();
        return ODL_OK;
    });
}

int odl_hip_permute(const void *src, int dtype, const int64_t *host_shape, int ndim, const int *host_perm, void *dst,
                    void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(ndim >= 0 && ndim <= 8, "permute: up to 8 dimensions, got %d", ndim);
    ODL_REQUIRE(dtype >= 0 && dtype < DT_COUNT, "permute: unknown element type code %d", dtype);
    ODL_REQUIRE(ndim == 0 || (host_shape && host_perm), "permute: null shape or order");
    PermuteDims d{};
    d.nd = ndim;
    bool used[8] = {false};
    int64_t istr[8], total = 1;
    for (int i = ndim - 1; i >= 0; --i)
    {
        ODL_REQUIRE(host_shape[i] >= 0, "permute: negative extent");
        istr[i] = total;
        total *= host_shape[i];
    }
    for (int k = 0; k < ndim; ++k)
    {
        const int p = host_perm[k];
        // the reference's messages (src/mat/origin/cpu/shape/permute.cpp:33-45)
        ODL_REQUIRE(p >= 0 && p < ndim, "permute: invalid dimension %d (must be in [0, %d))", p, ndim);
        ODL_REQUIRE(!used[p], "permute: duplicate dimension %d", p);
        used[p] = true;
        d.oshape[k] = host_shape[p];
        d.istride[k] = istr[p];
    }
    if (total == 0)
        return ODL_OK;
    ODL_REQUIRE(src && dst, "permute: null operand");
    hipStream_t st = odl::as_stream(stream);
    {
        // Extents of 1 dropped and output dimensions that are neighbours in the input too taken as one, many orders are
        // a copy, or a batched 2-D transposition [o][r][c] -> [o][c][r] (the detection head's (0,1,3,4,2) is one): those
        // go through LDS tiles, with lanes along the contiguous side of both tensors.
        int64_t mshape[8], mstride[8];  // merged output dimensions: extent, stride in the input
        int m = 0;
        for (int k = 0; k < ndim; ++k)
        {
            if (d.oshape[k] == 1)
                continue;
            if (m > 0 && mstride[m - 1] == d.oshape[k] * d.istride[k])
                mshape[m - 1] *= d.oshape[k], mstride[m - 1] = d.istride[k];
            else
                mshape[m] = d.oshape[k], mstride[m] = d.istride[k], ++m;
        }
        const int eb = (int)dtype_bytes(dtype);
        if (m <= 1)
        {
            ODL_HIP_CHECK(hipMemcpyAsync(dst, src, (size_t)total * eb, hipMemcpyDeviceToDevice, st));
            return ODL_OK;
        }
        // [c][r] from [r][c]: output (c, r) with input strides (1, cols); batched: output (o, c, r) with (rows*cols, 1, cols)
        if (m == 2 && mstride[0] == 1 && mstride[1] == mshape[0] && total < (1ll << 40))
            return odl::transpose_launch(src, dst, eb, 1, mshape[1], mshape[0], st);
        if (m == 3 && mstride[1] == 1 && mstride[2] == mshape[1] && mstride[0] == mshape[1] * mshape[2] && total < (1ll << 40))
            return odl::transpose_launch(src, dst, eb, mshape[0], mshape[2], mshape[1], st);
    }
    // elements of equal width move alike: 1, 4 or 8 bytes
    switch (dtype_bytes(dtype))
    {
        case 1:
            hipLaunchKernelGGL((permute_kernel<uint8_t>), dim3(grid_for(total)), dim3(kBlock), 0, st,
                               static_cast<const uint8_t *>(src), static_cast<uint8_t *>(dst), total, d);
            break;
        case 8:
            hipLaunchKernelGGL((permute_kernel<uint64_t>), dim3(grid_for(total)), dim3(kBlock), 0, st,
                               static_cast<const uint64_t *>(src), static_cast<uint64_t *>(dst), total, d);
            break;
        default:
            hipLaunchKernelGGL((permute_kernel<uint32_t>), dim3(grid_for(total)), dim3(kBlock), 0, st,
                               static_cast<const uint32_t *>(src), static_cast<uint32_t *>(dst), total, d);
    }
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

size_t odl_hip_sum_axis_dtype_workspace_bytes(int dtype, int64_t outer, int64_t axis, int64_t inner)
{
    if (outer <= 0 || axis <= 0 || inner <= 0)
        return 0;
    if (dtype == DT_F32)
        return odl_hip_sum_axis_workspace_bytes(outer, axis, inner);
    return plan_sum(outer, axis, inner).ws_bytes;
}

int odl_hip_sum_axis_dtype(int dtype, const void *src, int64_t outer, int64_t axis, int64_t inner, int through_float,
                           void *dst, void *workspace, size_t workspace_bytes, void *stream)
{
    if (dtype == DT_F32)  // a float passes through a float unchanged
        return odl_hip_sum_axis(static_cast<const float *>(src), outer, axis, inner, static_cast<float *>(dst), workspace,
                                workspace_bytes, stream);
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(outer >= 0 && axis >= 0 && inner >= 0, "sum: negative extent");
    ODL_REQUIRE(dtype >= 0 && dtype < DT_COUNT, "sum: unknown element type code %d", dtype);
    const int64_t nout = outer * inner;
    if (nout == 0)
        return ODL_OK;
    ODL_REQUIRE(dst != nullptr, "sum: null destination");
    hipStream_t st = odl::as_stream(stream);
    if (axis == 0)
        return odl::fill_bytes_launch(dst, 0, (size_t)nout * dtype_bytes(dtype), st);
    ODL_REQUIRE(src != nullptr, "sum: null source");
    const SumPlan p = plan_sum(outer, axis, inner);
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= p.ws_bytes && reinterpret_cast<uintptr_t>(workspace) % 8 == 0,
                "sum: an 8-byte aligned workspace of %zu bytes required, got %zu", p.ws_bytes, workspace_bytes);
    ODL_REQUIRE(inner > 1 || outer * p.slices < (1ll << 31), "sum: too many rows for one launch");
    return with_type(dtype, [&](auto t) {
        using T = decltype(t);
        using A = typename Acc<T>::type;
        A *part = static_cast<A *>(workspace);
        if (inner == 1)
            hipLaunchKernelGGL((row_partial_kernel<T>), dim3((unsigned)(p.slices * outer)), dim3(kBlock), 0, st,
                               static_cast<const T *>(src), part, outer, axis, p.chunk, (int)p.slices);
        else
            hipLaunchKernelGGL((col_partial_kernel<T>), dim3((unsigned)odl::ceil_div(nout, kBlock), (unsigned)p.slices),
                               dim3(kBlock), 0, st, static_cast<const T *>(src), part, outer, axis, inner, p.chunk);
        ODL_LAUNCH_CHECK();
        hipLaunchKernelGGL((fold_kernel<T>), dim3((unsigned)odl::ceil_div(nout, kBlock)), dim3(kBlock), 0, st, part,
                           static_cast<T *>(dst), nout, p.slices, through_float);
        ODL_LAUNCH_CHECK();
        return ODL_OK;
    });
}

}  // extern "C"
