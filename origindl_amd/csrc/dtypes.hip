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

// rows: src[outer][axis] (inner == 1). One workgroup per (row, slice); partial[slice * outer + row].
template <typename T>
__global__ __launch_bounds__(kBlock) void row_partial_kernel(const T *__restrict__ src, typename Acc<T>::type *__restrict__ part,
                                                             int64_t outer, int64_t axis, int64_t chunk)
{
    using A = typename Acc<T>::type;
    __shared__ A red[kBlock];
    const int64_t row = blockIdx.y, slice = blockIdx.x;
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
    ODL_REQUIRE(outer < 65536 || inner > 1, "sum: too many rows for the row schedule");
    return with_type(dtype, [&](auto t) {
        using T = decltype(t);
        using A = typename Acc<T>::type;
        A *part = static_cast<A *>(workspace);
        if (inner == 1)
            hipLaunchKernelGGL((row_partial_kernel<T>), dim3((unsigned)p.slices, (unsigned)outer), dim3(kBlock), 0, st,
                               static_cast<const T *>(src), part, outer, axis, p.chunk);
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
