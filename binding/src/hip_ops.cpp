// origin::cuda::* — the free functions OriginDL's device dispatcher calls for a tensor that lives on the device
// (include/origin/mat/origin/cuda/cuda_ops.cuh:57-722, cuda/factory.cuh:23-50 in the reference) — defined over the C ABI
// of the gfx950 backend (include/odl_hip.h, libodl_hip.so). Compiled against the reference's own headers; this is the
// file a maintainer adds next to src/mat/origin/cuda/*.cu to run OriginDL on an MI355X.
//
// Conventions kept from the reference: a function with an `out` parameter allocates and returns the result when out is
// null, else checks out's shape and element type, writes into it and returns null; errors are std::invalid_argument
// (shape, element type, argument) or std::runtime_error (device, unsupported) with the reference's wording where its
// tests look at it; everything is queued on the null stream; copies to the host wait for the device.
#include <cstring>
#include <random>

#include "odl_hip.h"
#include "origin/mat/origin/cuda/cuda_ops.cuh"
#include "origin/mat/origin/cuda/factory.cuh"
#include "origin/mat/origin/origin_mat.h"
#include "origin/mat/scalar.h"
#include "origin/utils/conv_utils.h"
#include "origin/utils/exception.h"

namespace origin
{
namespace cuda
{
namespace
{
void check(int rc)
{
    if (rc == ODL_OK)
        return;
    if (rc == ODL_ERR_INVALID_ARG)
        throw std::invalid_argument(odl_hip_last_error());
    throw std::runtime_error(odl_hip_last_error());
}

void *const kStream = nullptr;  // the null stream, like every launch of the reference

// the C ABI's element type codes are the DataType enumerators
int code(DataType dt)
{
    return static_cast<int>(dt);
}

const OriginMat &on_device(const OriginMat &m, const char *who)
{
    if (m.device().type() != DeviceType::kCUDA)
        THROW_RUNTIME_ERROR("{}: tensor is on {}, expected the device", who, m.device().to_string());
    if (!m.is_contiguous())
        THROW_RUNTIME_ERROR("{}: the tensor is not contiguous", who);
    return m;
}

// a float32 tensor on the device: what the matrix, convolution, pooling and loss kernels compute on
const OriginMat &f32(const OriginMat &m, const char *who)
{
    on_device(m, who);
    if (m.dtype() != DataType::kFloat32)
        THROW_INVALID_ARG("{}: only float32 is supported on the device, got {}", who, dtype_to_string(m.dtype()));
    return m;
}

const float *fp(const OriginMat &m)
{
    return m.data_ptr<float>();
}

// float32 or float64: the convolution operators take both (src/mat/origin/cuda/conv/conv2d.cu:412-664)
const OriginMat &real(const OriginMat &m, const char *who)
{
    on_device(m, who);
    if (m.dtype() != DataType::kFloat32 && m.dtype() != DataType::kFloat64)
        THROW_INVALID_ARG("{}: only float32 and float64 are supported on the device, got {}", who, dtype_to_string(m.dtype()));
    return m;
}

void same_type(const OriginMat &a, const OriginMat &b, const char *who)
{
    if (a.dtype() != b.dtype())
        THROW_INVALID_ARG("{}: operands of different element types ({} and {})", who, dtype_to_string(a.dtype()),
                          dtype_to_string(b.dtype()));
}

const double *dp(const OriginMat &m)
{
    return m.data_ptr<double>();
}

double *dp(OriginMat &m)
{
    return m.data_ptr<double>();
}

float *fp(OriginMat &m)
{
    return m.data_ptr<float>();
}

const void *vp(const OriginMat &m)
{
    return m.storage()->data();
}

std::unique_ptr<OriginMat> fresh(const OriginMat &like, const Shape &shape, DataType dt = DataType::kFloat32)
{
    return std::make_unique<OriginMat>(shape, dt, like.device());
}

// scratch memory of one call, from the tensor's own pool
struct Workspace
{
    std::shared_ptr<Storage> s;
    size_t bytes;
    Workspace(size_t n, const OriginMat &like) : bytes(n)
    {
        if (n)
            s = Storage::create(n, DeviceType::kCUDA, like.device().index());
    }
    void *ptr() const { return s ? s->data() : nullptr; }
};

std::vector<int64_t> dims64(const Shape &s)
{
    std::vector<int64_t> d(s.dims().begin(), s.dims().end());
    if (d.empty())
        d.push_back(1);  // storage for the pointer; the count passed alongside stays 0
    return d;
}

void split_axis(const Shape &s, int axis, int64_t &outer, int64_t &ax, int64_t &inner)
{
    outer = inner = 1;
    for (int i = 0; i < axis; ++i)
        outer *= (int64_t)s[i];
    ax = (int64_t)s[axis];
    for (size_t i = axis + 1; i < s.size(); ++i)
        inner *= (int64_t)s[i];
}

int label_kind(const OriginMat &idx, const char *who)
{
    if (idx.dtype() == DataType::kInt64)
        return 1;
    if (idx.dtype() == DataType::kInt32)
        return 0;
    THROW_INVALID_ARG("{}: indices must be int32 or int64, but got {}", who, dtype_to_string(idx.dtype()));
}

// one element of type dt from a Scalar, converted on the host the way the reference's host factories convert
void element_of(const Scalar &v, DataType dt, unsigned char (&e)[8])
{
    std::memset(e, 0, sizeof(e));
    switch (dt)
    {
        case DataType::kFloat32: { const float x = v.to_float32(); std::memcpy(e, &x, sizeof(x)); break; }
        case DataType::kFloat64: { const double x = v.to_float64(); std::memcpy(e, &x, sizeof(x)); break; }
        case DataType::kInt8: { const int8_t x = (int8_t)v.to_int32(); std::memcpy(e, &x, sizeof(x)); break; }
        case DataType::kInt32: { const int32_t x = v.to_int32(); std::memcpy(e, &x, sizeof(x)); break; }
        case DataType::kInt64: { const int64_t x = v.to_int64(); std::memcpy(e, &x, sizeof(x)); break; }
        default: { const uint8_t x = (uint8_t)v.to_int32(); std::memcpy(e, &x, sizeof(x)); break; }
    }
}

// ---- elementwise: the operator numbers of odl_hip_binary_dtype / odl_hip_unary_dtype
enum { ADD = 0, SUB = 1, MUL = 2, DIV = 3, GT = 4, EQ = 5, NE = 6, LT = 7, LE = 8, GE = 9, SIGMOID_BWD = 10, SILU_BWD = 11 };
enum { RELU = 0, EXP = 1, LOG = 2, NEG = 3, SQUARE = 4, SQRT = 5, SIGMOID = 6, SILU = 7 };

std::unique_ptr<Mat> binary(int op, const char *who, const OriginMat &a, const OriginMat &b, OriginMat *out)
{
    on_device(a, who), on_device(b, who);
    if (a.dtype() != b.dtype())
        THROW_INVALID_ARG("Data type mismatch in {}: expected {} but got {}", who, dtype_to_string(a.dtype()),
                          dtype_to_string(b.dtype()));
    if (op > GE && a.dtype() != DataType::kFloat32)
        THROW_INVALID_ARG("{}: only float32 is supported on the device, got {}", who, dtype_to_string(a.dtype()));
    // same shape, or one side a single element (src/mat/origin/cpu/math/add.cpp:56-93: anything else throws)
    Shape rs = a.shape();
    if (a.shape() != b.shape())
    {
        if (b.elements() == 1)
            rs = a.shape();
        else if (a.elements() == 1)
            rs = b.shape();
        else
            THROW_RUNTIME_ERROR("Complex broadcasting not yet implemented for {} operation: {} vs {}", who,
                                a.shape().to_string(), b.shape().to_string());
    }
    std::unique_ptr<OriginMat> made;
    OriginMat *dst = out;
    if (!dst)
    {
        made = fresh(a, rs, a.dtype());
        dst  = made.get();
    }
    else if (dst->shape() != rs || dst->dtype() != a.dtype() || dst->device() != a.device())
        THROW_INVALID_ARG("Output tensor mismatch. Expected shape={}, dtype={}, got shape={}, dtype={}", rs.to_string(),
                          dtype_to_string(a.dtype()), dst->shape().to_string(), dtype_to_string(dst->dtype()));
    check(odl_hip_binary_dtype(op, code(a.dtype()), vp(a), (int64_t)a.elements(), vp(b), (int64_t)b.elements(),
                               dst->storage()->data(), kStream));
    return made;
}

std::unique_ptr<Mat> unary(int op, const char *who, const OriginMat &a, OriginMat *out)
{
    on_device(a, who);
    // exp, log, sqrt, sigmoid and silu exist for the floating-point types only, as in the reference
    const bool floating = a.dtype() == DataType::kFloat32 || a.dtype() == DataType::kFloat64;
    if (!floating && !(op == RELU || op == NEG || op == SQUARE))
        THROW_INVALID_ARG("{}: only floating-point tensors are supported, got {}", who, dtype_to_string(a.dtype()));
    std::unique_ptr<OriginMat> made;
    OriginMat *dst = out;
    if (!dst)
    {
        made = fresh(a, a.shape(), a.dtype());
        dst  = made.get();
    }
    else if (dst->shape() != a.shape() || dst->dtype() != a.dtype() || dst->device() != a.device())
        THROW_INVALID_ARG("Output tensor mismatch. Expected shape={}, dtype={}, got shape={}, dtype={}",
                          a.shape().to_string(), dtype_to_string(a.dtype()), dst->shape().to_string(),
                          dtype_to_string(dst->dtype()));
    check(odl_hip_unary_dtype(op, code(a.dtype()), vp(a), (int64_t)a.elements(), dst->storage()->data(), kStream));
    return made;
}

[[noreturn]] void not_on_this_backend(const char *what)
{
    THROW_RUNTIME_ERROR("{}: not implemented on the gfx950 backend (outside the matmul / convolution hot path)", what);
}
}  // namespace

// ------------------------------------------------------------------------------------------- factories
std::unique_ptr<OriginMat> full(const Shape &shape, const Scalar &scalar, const TensorOptions &options)
{
    auto m = std::make_unique<OriginMat>(shape, options.dtype(), options.device());
    unsigned char e[8];
    element_of(scalar, options.dtype(), e);
    if (shape.elements() > 0)
        check(odl_hip_fill_dtype(m->storage()->data(), code(options.dtype()), (int64_t)shape.elements(), e, kStream));
    return m;
}

std::unique_ptr<OriginMat> zeros(const Shape &shape, const TensorOptions &options)
{
    return full(shape, Scalar(0.0f), options);
}

std::unique_ptr<OriginMat> ones(const Shape &shape, const TensorOptions &options)
{
    return full(shape, Scalar(1.0f), options);
}

// user data of type user_dtype -> a device tensor of options.dtype(): uploaded as it is, converted on the device
std::unique_ptr<OriginMat> from_memory(const void *data, DataType user_dtype, const Shape &shape,
                                       const TensorOptions &options)
{
    const size_t n = shape.elements();
    auto staged = std::make_unique<OriginMat>(shape, user_dtype, options.device());
    if (n > 0)
        check(odl_hip_memcpy_h2d(staged->storage()->data(), data, n * element_size(user_dtype), kStream));
    if (user_dtype == options.dtype())
        return staged;
    auto m = std::make_unique<OriginMat>(shape, options.dtype(), options.device());
    if (n > 0)
        check(odl_hip_convert(staged->storage()->data(), code(user_dtype), m->storage()->data(), code(options.dtype()),
                              (int64_t)n, kStream));
    return m;
}

// ------------------------------------------------------------------------------------------- elementwise
std::unique_ptr<Mat> add(const OriginMat &a, const OriginMat &b, OriginMat *out) { return binary(ADD, "add", a, b, out); }
std::unique_ptr<Mat> subtract(const OriginMat &a, const OriginMat &b, OriginMat *out) { return binary(SUB, "subtract", a, b, out); }
std::unique_ptr<Mat> multiply(const OriginMat &a, const OriginMat &b, OriginMat *out) { return binary(MUL, "multiply", a, b, out); }
std::unique_ptr<Mat> divide(const OriginMat &a, const OriginMat &b, OriginMat *out) { return binary(DIV, "divide", a, b, out); }
std::unique_ptr<Mat> eq(const OriginMat &a, const OriginMat &b, OriginMat *out) { return binary(EQ, "eq", a, b, out); }
std::unique_ptr<Mat> ne(const OriginMat &a, const OriginMat &b, OriginMat *out) { return binary(NE, "ne", a, b, out); }
std::unique_ptr<Mat> lt(const OriginMat &a, const OriginMat &b, OriginMat *out) { return binary(LT, "lt", a, b, out); }
std::unique_ptr<Mat> le(const OriginMat &a, const OriginMat &b, OriginMat *out) { return binary(LE, "le", a, b, out); }
std::unique_ptr<Mat> gt(const OriginMat &a, const OriginMat &b, OriginMat *out) { return binary(GT, "gt", a, b, out); }
std::unique_ptr<Mat> ge(const OriginMat &a, const OriginMat &b, OriginMat *out) { return binary(GE, "ge", a, b, out); }
std::unique_ptr<Mat> exp(const OriginMat &m, OriginMat *out) { return unary(EXP, "exp", m, out); }
std::unique_ptr<Mat> log(const OriginMat &m, OriginMat *out) { return unary(LOG, "log", m, out); }
std::unique_ptr<Mat> sqrt(const OriginMat &m, OriginMat *out) { return unary(SQRT, "sqrt", m, out); }
std::unique_ptr<Mat> square(const OriginMat &m, OriginMat *out) { return unary(SQUARE, "square", m, out); }
std::unique_ptr<Mat> negate(const OriginMat &m, OriginMat *out) { return unary(NEG, "negate", m, out); }
std::unique_ptr<Mat> relu(const OriginMat &m, OriginMat *out) { return unary(RELU, "relu", m, out); }
std::unique_ptr<Mat> sigmoid(const OriginMat &m, OriginMat *out) { return unary(SIGMOID, "sigmoid", m, out); }
std::unique_ptr<Mat> silu(const OriginMat &m, OriginMat *out) { return unary(SILU, "silu", m, out); }

std::unique_ptr<Mat> sigmoid_backward(const OriginMat &gy, const OriginMat &y)
{
    if (y.shape() != gy.shape() || y.dtype() != gy.dtype())
        THROW_INVALID_ARG("sigmoid_backward: gy and y must have same shape and dtype");
    return binary(SIGMOID_BWD, "sigmoid_backward", gy, y, nullptr);
}

std::unique_ptr<Mat> silu_backward(const OriginMat &gy, const OriginMat &x)
{
    if (x.shape() != gy.shape() || x.dtype() != gy.dtype())
        THROW_INVALID_ARG("silu_backward: gy and x must have same shape and dtype");
    return binary(SILU_BWD, "silu_backward", gy, x, nullptr);
}

std::unique_ptr<Mat> leaky_relu(const OriginMat &, const OriginMat &, OriginMat *) { not_on_this_backend("leaky_relu"); }

std::unique_ptr<Mat> pow(const OriginMat &mat, const Scalar &exponent, OriginMat *out)
{
    on_device(mat, "pow");
    if (mat.dtype() != DataType::kFloat32 && mat.dtype() != DataType::kFloat64)
        THROW_INVALID_ARG("pow: only floating-point tensors are supported on the device, got {}",
                          dtype_to_string(mat.dtype()));
    std::unique_ptr<OriginMat> made;
    OriginMat *dst = out;
    if (!dst)
    {
        made = fresh(mat, mat.shape(), mat.dtype());
        dst  = made.get();
    }
    else if (dst->shape() != mat.shape() || dst->dtype() != mat.dtype())
        THROW_INVALID_ARG("Output tensor mismatch. Expected shape={}, got shape={}", mat.shape().to_string(),
                          dst->shape().to_string());
    // float32: powf with the exponent rounded to float, as the reference's float kernel sees it (cpu/math/pow.cpp:14-44)
    const double e = mat.dtype() == DataType::kFloat32 ? (double)exponent.to_float32() : exponent.to_float64();
    check(odl_hip_pow_scalar_dtype(code(mat.dtype()), vp(mat), (int64_t)mat.elements(), e, dst->storage()->data(), kStream));
    return made;
}

void pow_inplace(OriginMat &mat, const Scalar &exponent)
{
    (void)pow(mat, exponent, &mat);
}

std::unique_ptr<Mat> convert_datatype(const OriginMat &mat, DataType target_type)
{
    on_device(mat, "convert_datatype");
    auto out = fresh(mat, mat.shape(), target_type);
    if (mat.elements() > 0)
        check(odl_hip_convert(vp(mat), code(mat.dtype()), out->storage()->data(), code(target_type), (int64_t)mat.elements(),
                              kStream));
    return out;
}

std::unique_ptr<Mat> clone(const OriginMat &mat)
{
    on_device(mat, "clone");
    auto out = fresh(mat, mat.shape(), mat.dtype());
    const size_t bytes = mat.elements() * element_size(mat.dtype());
    if (bytes > 0)
        check(odl_hip_memcpy_d2d(out->storage()->data(), vp(mat), bytes, kStream));
    return out;
}

void index_put(OriginMat &mat, std::initializer_list<size_t> indices, const Scalar &value)
{
    const Shape shape = mat.shape();
    if (indices.size() != shape.size())
        THROW_INVALID_ARG("Index count ({}) does not match tensor dimension ({}). Shape: {}", indices.size(), shape.size(),
                          shape.to_string());
    size_t offset = 0, d = 0;
    for (size_t i : indices)
    {
        if (i >= shape[d])
            THROW_INVALID_ARG("Index {} out of range for dimension {} (size: {}). Shape: {}", i, d, shape[d],
                              shape.to_string());
        offset += i * mat.strides()[d++];
    }
    unsigned char e[8];
    element_of(value, mat.dtype(), e);
    const size_t width = element_size(mat.dtype());
    check(odl_hip_synchronize());
    check(odl_hip_memcpy_h2d(static_cast<unsigned char *>(mat.storage()->data()) + offset * width, e, width, kStream));
}

// ------------------------------------------------------------------------------------------- shape
std::unique_ptr<Mat> reshape(const OriginMat &mat, const Shape &new_shape)
{
    if (new_shape.elements() != mat.elements())
        THROW_INVALID_ARG("Reshape: total elements must match. Original: {}, Target: {}", mat.elements(),
                          new_shape.elements());
    return std::make_unique<OriginMat>(mat.storage(), new_shape, mat.dtype());
}

// the last two dimensions exchanged, materialised (src/mat/origin/cpu/shape/transpose.cpp:27-77, 130-137)
std::unique_ptr<Mat> transpose(const OriginMat &mat)
{
    on_device(mat, "transpose");
    const Shape s = mat.shape();
    if (s.size() < 2)
        return clone(mat);
    std::vector<int> dims(s.size());
    for (size_t i = 0; i < s.size(); ++i)
        dims[i] = (int)i;
    std::swap(dims[s.size() - 2], dims[s.size() - 1]);
    return permute(mat, dims);
}

std::unique_ptr<Mat> permute(const OriginMat &mat, const std::vector<int> &dims)
{
    on_device(mat, "permute");
    const Shape s = mat.shape();
    if (dims.size() != s.size())
        THROW_INVALID_ARG("permute: dims size {} does not match input dimension {}", dims.size(), s.size());
    std::vector<size_t> od;
    std::vector<bool> seen(s.size(), false);
    for (int d : dims)
    {
        if (d < 0 || d >= (int)s.size() || seen[d])
            THROW_INVALID_ARG("permute: invalid dimension {} (must be a permutation of [0, {}))", d, s.size());
        seen[d] = true;
        od.push_back(s[d]);
    }
    auto out = fresh(mat, Shape(od), mat.dtype());
    const std::vector<int64_t> in = dims64(s);
    if (mat.elements() > 0)
        check(odl_hip_permute(vp(mat), code(mat.dtype()), in.data(), (int)s.size(), dims.data(), out->storage()->data(),
                              kStream));
    return out;
}

std::unique_ptr<Mat> cat(const std::vector<const OriginMat *> &inputs, int dim)
{
    if (inputs.empty())
        THROW_RUNTIME_ERROR("cat: no input");
    const OriginMat &first = on_device(*inputs[0], "cat");
    if (inputs.size() == 1)
        return clone(first);
    const Shape fs = first.shape();
    if (dim < 0 || (size_t)dim >= fs.size())
        THROW_RUNTIME_ERROR("cat: dimension {} out of range for {} dimensions", dim, fs.size());
    size_t total = 0;
    std::vector<const void *> ptrs;
    std::vector<int64_t> sizes;
    for (const OriginMat *m : inputs)
    {
        if (!m)
            THROW_RUNTIME_ERROR("cat: null input");
        same_type(first, on_device(*m, "cat"), "cat");
        const Shape s = m->shape();
        if (s.size() != fs.size())
            THROW_RUNTIME_ERROR("cat: all inputs must have same number of dimensions");
        for (size_t d = 0; d < s.size(); ++d)
            if (d != (size_t)dim && s[d] != fs[d])
                THROW_RUNTIME_ERROR("cat: dimension {} mismatch: {} vs {}", d, s[d], fs[d]);
        if (m->device() != first.device())
            THROW_INVALID_ARG("cat: inputs live on different devices");
        total += s[dim];
        ptrs.push_back(vp(*m));
        sizes.push_back((int64_t)s[dim]);
    }
    std::vector<size_t> od = fs.dims();
    od[dim] = total;
    const Shape os(od);
    int64_t outer, ax, inner;
    split_axis(os, dim, outer, ax, inner);
    auto y = fresh(first, os, first.dtype());
    check(odl_hip_cat_dtype(code(first.dtype()), ptrs.data(), sizes.data(), (int)ptrs.size(), outer, inner, y->storage()->data(),
                            kStream));
    return y;
}

std::vector<std::unique_ptr<Mat>> split(const OriginMat &input, const std::vector<size_t> &split_sizes, int dim)
{
    const OriginMat &x = on_device(input, "split");
    const Shape s = x.shape();
    if (dim < 0 || (size_t)dim >= s.size())
        THROW_RUNTIME_ERROR("split: dimension {} out of range for {} dimensions", dim, s.size());
    size_t total = 0;
    for (size_t z : split_sizes)
        total += z;
    if (total != s[dim])
        THROW_RUNTIME_ERROR("split: sizes sum to {}, but dimension {} has {} elements", total, dim, s[dim]);
    int64_t outer, ax, inner;
    split_axis(s, dim, outer, ax, inner);
    std::vector<std::unique_ptr<Mat>> parts;
    int64_t off = 0;
    for (size_t z : split_sizes)
    {
        std::vector<size_t> d = s.dims();
        d[dim] = z;
        auto piece = fresh(x, Shape(d), x.dtype());
        check(odl_hip_slice_axis_dtype(code(x.dtype()), vp(x), outer, ax, inner, off, (int64_t)z, piece->storage()->data(), kStream));
        off += (int64_t)z;
        parts.push_back(std::move(piece));
    }
    return parts;
}

// ------------------------------------------------------------------------------------------- products, reductions
// C = A.B for 2-D x 2-D, 3-D x 2-D and 3-D x 3-D operands (src/mat/origin/cpu/math/matmul.cpp:27-41, 55-109)
std::unique_ptr<Mat> matmul(const OriginMat &a_, const OriginMat &b_)
{
    const OriginMat &a = f32(a_, "matmul"), &b = f32(b_, "matmul");
    const Shape as = a.shape(), bs = b.shape();
    if (as.size() < 2 || bs.size() < 2)
        THROW_INVALID_ARG("Matrix multiplication requires at least 2D tensors. A shape: {}, B shape: {}", as.to_string(),
                          bs.to_string());
    int64_t batch = 1, M, K, N;
    int b_batched = 0;
    Shape rs;
    if (as.size() == 2 && bs.size() == 2)
    {
        M = as[0], K = as[1], N = bs[1];
        rs = Shape{as[0], bs[1]};
    }
    else if (as.size() == 3 && bs.size() == 2)
    {
        batch = as[0], M = as[1], K = as[2], N = bs[1];
        rs = Shape{as[0], as[1], bs[1]};
    }
    else if (as.size() == 3 && bs.size() == 3)
    {
        if (as[0] != bs[0])
            THROW_INVALID_ARG("Matrix dimensions must be compatible for multiplication. A[0]={} != B[0]={}", as[0], bs[0]);
        batch = as[0], M = as[1], K = as[2], N = bs[2], b_batched = 1;
        rs = Shape{as[0], as[1], bs[2]};
    }
    else
        THROW_INVALID_ARG("Matrix multiplication requires compatible dimensions. A shape: {}, B shape: {}", as.to_string(),
                          bs.to_string());
    if ((int64_t)bs[bs.size() - 2] != K)
        THROW_INVALID_ARG("Matrix dimensions must be compatible for multiplication. A shape: {}, B shape: {}",
                          as.to_string(), bs.to_string());
    auto c = fresh(a, rs);
    Workspace ws(odl_hip_matmul_workspace_bytes(batch, M, N, K, b_batched), a);
    check(odl_hip_matmul(fp(a), fp(b), fp(*c), batch, M, N, K, b_batched, ws.ptr(), ws.bytes, kStream));
    return c;
}

std::unique_ptr<Mat> sum(const OriginMat &mat, int axis, bool keepdim)
{
    const OriginMat &x = on_device(mat, "sum");
    const Shape s = x.shape();
    const int dt = code(x.dtype());
    if (axis == -1)
    {
        const Shape rs = keepdim ? Shape(std::vector<size_t>(s.size(), 1)) : Shape{1};
        auto out = fresh(x, rs, x.dtype());
        // the whole-tensor sum goes back into the element type through a float (cpu/math/sum.cpp:18-35)
        Workspace ws(odl_hip_sum_axis_dtype_workspace_bytes(dt, 1, (int64_t)x.elements(), 1), x);
        check(odl_hip_sum_axis_dtype(dt, vp(x), 1, (int64_t)x.elements(), 1, 1, out->storage()->data(), ws.ptr(), ws.bytes,
                                     kStream));
        return out;
    }
    if (axis < 0 || axis >= (int)s.size())
        THROW_INVALID_ARG("Invalid axis {} for sum operation. Tensor has {} dimensions", axis, s.size());
    std::vector<size_t> rd;
    for (size_t i = 0; i < s.size(); ++i)
    {
        if ((int)i != axis)
            rd.push_back(s[i]);
        else if (keepdim)
            rd.push_back(1);
    }
    int64_t outer, ax, inner;
    split_axis(s, axis, outer, ax, inner);
    auto out = fresh(x, Shape(rd), x.dtype());
    Workspace ws(odl_hip_sum_axis_dtype_workspace_bytes(dt, outer, ax, inner), x);
    check(odl_hip_sum_axis_dtype(dt, vp(x), outer, ax, inner, 0, out->storage()->data(), ws.ptr(), ws.bytes, kStream));
    return out;
}

std::unique_ptr<Mat> max(const OriginMat &mat, int axis)
{
    const OriginMat &x = on_device(mat, "max");
    const Shape s = x.shape();
    if (axis == -1)
    {
        auto out = fresh(x, Shape{1}, x.dtype());
        check(odl_hip_max_all_dtype(code(x.dtype()), vp(x), (int64_t)x.elements(), out->storage()->data(), kStream));
        return out;
    }
    if (axis < 0 || axis >= (int)s.size())
        THROW_INVALID_ARG("Invalid axis {} for max operation. Tensor has {} dimensions", axis, s.size());
    std::vector<size_t> rd;
    for (size_t i = 0; i < s.size(); ++i)
        if ((int)i != axis)
            rd.push_back(s[i]);
    int64_t outer, ax, inner;
    split_axis(s, axis, outer, ax, inner);
    auto out = fresh(x, Shape(rd), x.dtype());
    check(odl_hip_max_axis_dtype(code(x.dtype()), vp(x), outer, ax, inner, out->storage()->data(), kStream));
    return out;
}

std::unique_ptr<Mat> broadcast_to(const OriginMat &mat, const Shape &target_shape)
{
    const OriginMat &x = on_device(mat, "broadcast_to");
    auto out = fresh(x, target_shape, x.dtype());
    const auto sd = dims64(x.shape()), dd = dims64(target_shape);
    check(odl_hip_broadcast_to_dtype(code(x.dtype()), vp(x), sd.data(), (int)x.shape().size(), dd.data(), (int)target_shape.size(),
                                     out->storage()->data(), kStream));
    return out;
}

// shapes aligned from the left (src/mat/origin/cpu/math/sum_to.cpp:36-54); equal shapes share the storage (14-18)
std::unique_ptr<Mat> sum_to(const OriginMat &mat, const Shape &target_shape)
{
    if (mat.shape() == target_shape)
        return std::make_unique<OriginMat>(mat);
    const OriginMat &x = on_device(mat, "sum_to");
    const int dt = code(x.dtype());
    const auto sd = dims64(x.shape()), td = dims64(target_shape);
    Workspace ws(odl_hip_sum_to_dtype_workspace_bytes(dt, sd.data(), (int)x.shape().size(), td.data(), (int)target_shape.size()), x);
    auto out = fresh(x, target_shape, x.dtype());
    check(odl_hip_sum_to_dtype(dt, vp(x), sd.data(), (int)x.shape().size(), td.data(), (int)target_shape.size(),
                               out->storage()->data(), ws.ptr(), ws.bytes, kStream));
    return out;
}

// ------------------------------------------------------------------------------------------- convolution, pooling
std::unique_ptr<Mat> im2col(const OriginMat &img, std::pair<int, int> k, std::pair<int, int> s, std::pair<int, int> p,
                            bool to_matrix)
{
    const OriginMat &x = real(img, "im2col");
    const Shape xs = x.shape();
    if (xs.size() != 4)
        THROW_INVALID_ARG("im2col: input must be 4D (N, C, H, W), but got shape {}", xs.to_string());
    const int64_t N = xs[0], C = xs[1], H = xs[2], W = xs[3];
    const int OH = get_conv_outsize((int)H, k.first, s.first, p.first);
    const int OW = get_conv_outsize((int)W, k.second, s.second, p.second);
    if (OH <= 0 || OW <= 0)
        THROW_INVALID_ARG("im2col: invalid output size OH={}, OW={} for input H={}, W={}", OH, OW, H, W);
    const Shape cs = to_matrix ? Shape{(size_t)(N * OH * OW), (size_t)(C * k.first * k.second)}
                               : Shape{(size_t)N, (size_t)C, (size_t)k.first, (size_t)k.second, (size_t)OH, (size_t)OW};
    auto col = fresh(x, cs, x.dtype());
    if (x.dtype() == DataType::kFloat64)
        check(odl_hip_im2col_f64(dp(x), N, C, H, W, k.first, k.second, s.first, s.second, p.first, p.second, to_matrix ? 1 : 0,
                                 dp(*col), kStream));
    else
        check(odl_hip_im2col(fp(x), N, C, H, W, k.first, k.second, s.first, s.second, p.first, p.second, to_matrix ? 1 : 0,
                             fp(*col), kStream));
    return col;
}

std::unique_ptr<Mat> col2im(const OriginMat &col_, const Shape &is, std::pair<int, int> k, std::pair<int, int> s,
                            std::pair<int, int> p, bool to_matrix)
{
    const OriginMat &col = real(col_, "col2im");
    if (is.size() != 4)
        THROW_INVALID_ARG("col2im: input_shape must be 4D (N, C, H, W), but got shape {}", is.to_string());
    const int64_t N = is[0], C = is[1], H = is[2], W = is[3];
    const int OH = get_conv_outsize((int)H, k.first, s.first, p.first);
    const int OW = get_conv_outsize((int)W, k.second, s.second, p.second);
    const Shape want = to_matrix ? Shape{(size_t)(N * OH * OW), (size_t)(C * k.first * k.second)}
                                 : Shape{(size_t)N, (size_t)C, (size_t)k.first, (size_t)k.second, (size_t)OH, (size_t)OW};
    if (OH <= 0 || OW <= 0 || col.shape() != want)
        THROW_INVALID_ARG("col2im: invalid col shape {} for input_shape {}", col.shape().to_string(), is.to_string());
    auto img = fresh(col, is, col.dtype());
    if (col.dtype() == DataType::kFloat64)
        check(odl_hip_col2im_f64(dp(col), N, C, H, W, k.first, k.second, s.first, s.second, p.first, p.second, to_matrix ? 1 : 0,
                                 dp(*img), kStream));
    else
        check(odl_hip_col2im(fp(col), N, C, H, W, k.first, k.second, s.first, s.second, p.first, p.second, to_matrix ? 1 : 0,
                             fp(*img), kStream));
    return img;
}

std::unique_ptr<Mat> conv2d(const OriginMat &x_, const OriginMat &W_, const OriginMat *b, std::pair<int, int> s,
                            std::pair<int, int> p)
{
    const OriginMat &x = real(x_, "conv2d"), &w = real(W_, "conv2d");
    same_type(x, w, "conv2d");
    const bool f64 = x.dtype() == DataType::kFloat64;
    const Shape xs = x.shape(), wsh = w.shape();
    if (xs.size() != 4)
        THROW_INVALID_ARG("conv2d: x must be 4D (N, C, H, W), but got shape {}", xs.to_string());
    if (wsh.size() != 4)
        THROW_INVALID_ARG("conv2d: W must be 4D (OC, C, KH, KW), but got shape {}", wsh.to_string());
    const int64_t N = xs[0], C = xs[1], H = xs[2], W = xs[3], OC = wsh[0];
    const int KH = (int)wsh[2], KW = (int)wsh[3];
    if ((int64_t)wsh[1] != C)
        THROW_INVALID_ARG("conv2d: channel mismatch - x has {} channels, but W expects {} channels", C, wsh[1]);
    const int OH = get_conv_outsize((int)H, KH, s.first, p.first), OW = get_conv_outsize((int)W, KW, s.second, p.second);
    if (OH <= 0 || OW <= 0)
        THROW_INVALID_ARG("conv2d: invalid output size OH={}, OW={} for input H={}, W={}, kernel=({},{})", OH, OW, H, W, KH,
                          KW);
    const float *bias = nullptr;
    const double *bias64 = nullptr;
    if (b)
    {
        const OriginMat &bm = real(*b, "conv2d");
        same_type(x, bm, "conv2d");
        if (bm.shape().size() != 1 || (int64_t)bm.shape()[0] != OC)
            THROW_INVALID_ARG("conv2d: b must be 1D with size {}, but got shape {}", OC, bm.shape().to_string());
        if (f64)
            bias64 = dp(bm);
        else
            bias = fp(bm);
    }
    auto y = fresh(x, Shape{(size_t)N, (size_t)OC, (size_t)OH, (size_t)OW}, x.dtype());
    if (f64)
    {
        Workspace ws64(odl_hip_conv2d_f64_workspace_bytes(N, C, H, W, OC, KH, KW, s.first, s.second, p.first, p.second), x);
        check(odl_hip_conv2d_f64(dp(x), dp(w), bias64, N, C, H, W, OC, KH, KW, s.first, s.second, p.first, p.second, dp(*y),
                                 ws64.ptr(), ws64.bytes, kStream));
        return y;
    }
    Workspace ws(odl_hip_conv2d_workspace_bytes(N, C, H, W, OC, KH, KW, s.first, s.second, p.first, p.second), x);
    check(odl_hip_conv2d(fp(x), fp(w), bias, N, C, H, W, OC, KH, KW, s.first, s.second, p.first, p.second, fp(*y), ws.ptr(),
                         ws.bytes, kStream));
    return y;
}

// {gx, gW, [gb]} with gy's buffer read as a row-major [N*OH*OW, OC] matrix, as the reference reads it
// (src/mat/origin/cpu/conv/conv2d.cpp:514-599)
std::vector<std::unique_ptr<Mat>> conv2d_backward(const OriginMat &gy_, const OriginMat &x_, const OriginMat &W_,
                                                  const OriginMat *b, std::pair<int, int> s, std::pair<int, int> p)
{
    const OriginMat &gy = real(gy_, "conv2d_backward"), &x = real(x_, "conv2d_backward"), &w = real(W_, "conv2d_backward");
    same_type(x, gy, "conv2d_backward");
    same_type(x, w, "conv2d_backward");
    if (gy.shape().size() != 4)
        THROW_INVALID_ARG("conv2d_backward: gy must be 4D (N, OC, OH, OW), but got shape {}", gy.shape().to_string());
    if (x.shape().size() != 4)
        THROW_INVALID_ARG("conv2d_backward: x must be 4D (N, C, H, W), but got shape {}", x.shape().to_string());
    if (w.shape().size() != 4)
        THROW_INVALID_ARG("conv2d_backward: W must be 4D (OC, C, KH, KW), but got shape {}", w.shape().to_string());
    const int64_t N = x.shape()[0], C = x.shape()[1], H = x.shape()[2], W = x.shape()[3], OC = w.shape()[0];
    const int KH = (int)w.shape()[2], KW = (int)w.shape()[3];
    auto gx = fresh(x, x.shape(), x.dtype());
    auto gw = fresh(x, w.shape(), x.dtype());
    std::unique_ptr<OriginMat> gb;
    if (b)
        gb = fresh(x, Shape{(size_t)OC}, x.dtype());
    if (x.dtype() == DataType::kFloat64)
    {
        Workspace ws64(odl_hip_conv2d_backward_f64_workspace_bytes(N, C, H, W, OC, KH, KW, s.first, s.second, p.first, p.second), x);
        check(odl_hip_conv2d_backward_f64(dp(gy), dp(x), dp(w), N, C, H, W, OC, KH, KW, s.first, s.second, p.first, p.second,
                                          dp(*gx), dp(*gw), gb ? dp(*gb) : nullptr, ws64.ptr(), ws64.bytes, kStream));
    }
    else
    {
        Workspace ws(odl_hip_conv2d_backward_workspace_bytes(N, C, H, W, OC, KH, KW, s.first, s.second, p.first, p.second), x);
        check(odl_hip_conv2d_backward(fp(gy), fp(x), fp(w), N, C, H, W, OC, KH, KW, s.first, s.second, p.first, p.second,
                                      fp(*gx), fp(*gw), gb ? fp(*gb) : nullptr, ws.ptr(), ws.bytes, kStream));
    }
    std::vector<std::unique_ptr<Mat>> grads;
    grads.push_back(std::move(gx));
    grads.push_back(std::move(gw));
    if (gb)
        grads.push_back(std::move(gb));
    return grads;
}

// The window-local indices kh*KW + kw cross the interface as a host vector (mat.h:560-578): copied down after the
// forward kernel and up again before the backward one, as the reference's device backend does.
std::unique_ptr<Mat> max_pool2d(const OriginMat &x_, std::pair<int, int> k, std::pair<int, int> s, std::pair<int, int> p,
                                std::vector<size_t> *indices)
{
    const OriginMat &x = f32(x_, "max_pool2d");
    const Shape xs = x.shape();
    if (xs.size() != 4)
        THROW_INVALID_ARG("max_pool2d: x must be 4D (N, C, H, W), but got shape {}", xs.to_string());
    const int64_t N = xs[0], C = xs[1], H = xs[2], W = xs[3];
    const int OH = get_conv_outsize((int)H, k.first, s.first, p.first);
    const int OW = get_conv_outsize((int)W, k.second, s.second, p.second);
    if (OH <= 0 || OW <= 0)
        THROW_INVALID_ARG("max_pool2d: invalid output size OH={}, OW={} for input H={}, W={}", OH, OW, H, W);
    auto y = fresh(x, Shape{(size_t)N, (size_t)C, (size_t)OH, (size_t)OW});
    Workspace idx(indices ? y->elements() * sizeof(uint64_t) : 0, x);
    check(odl_hip_max_pool2d(fp(x), N, C, H, W, k.first, k.second, s.first, s.second, p.first, p.second, fp(*y),
                             static_cast<uint64_t *>(idx.ptr()), kStream));
    if (indices)
    {
        static_assert(sizeof(size_t) == sizeof(uint64_t), "size_t must be 64-bit");
        indices->resize(y->elements());
        if (y->elements() > 0)
            check(odl_hip_memcpy_d2h(indices->data(), idx.ptr(), idx.bytes));
    }
    return y;
}

std::unique_ptr<Mat> max_pool2d_backward(const OriginMat &gy_, const OriginMat &x, std::pair<int, int> k,
                                         std::pair<int, int> s, std::pair<int, int> p, const std::vector<size_t> &indices)
{
    const OriginMat &gy = f32(gy_, "max_pool2d_backward");
    if (gy.shape().size() != 4)
        THROW_INVALID_ARG("max_pool2d_backward: gy must be 4D (N, C, OH, OW), but got shape {}", gy.shape().to_string());
    if (indices.size() != gy.elements())
        THROW_INVALID_ARG("max_pool2d_backward: indices size mismatch. Expected {}, got {}", gy.elements(), indices.size());
    const Shape xs = x.shape();
    const int64_t N = xs[0], C = xs[1], H = xs[2], W = xs[3];
    Workspace idx(indices.size() * sizeof(uint64_t), gy);
    if (!indices.empty())
        check(odl_hip_memcpy_h2d(idx.ptr(), indices.data(), idx.bytes, kStream));
    auto gx = fresh(gy, xs);
    check(odl_hip_max_pool2d_backward(fp(gy), static_cast<const uint64_t *>(idx.ptr()), N, C, H, W, k.first, k.second,
                                      s.first, s.second, p.first, p.second, fp(*gx), kStream));
    return gx;
}

std::unique_ptr<Mat> avg_pool2d(const OriginMat &, std::pair<int, int>, std::pair<int, int>, std::pair<int, int>)
{
    not_on_this_backend("avg_pool2d");
}
std::unique_ptr<Mat> avg_pool2d_backward(const OriginMat &, const OriginMat &, std::pair<int, int>, std::pair<int, int>,
                                         std::pair<int, int>)
{
    not_on_this_backend("avg_pool2d_backward");
}
std::unique_ptr<Mat> adaptive_avg_pool2d(const OriginMat &, std::pair<int, int>) { not_on_this_backend("adaptive_avg_pool2d"); }
std::unique_ptr<Mat> adaptive_avg_pool2d_backward(const OriginMat &, const OriginMat &, std::pair<int, int>)
{
    not_on_this_backend("adaptive_avg_pool2d_backward");
}

// ------------------------------------------------------------------------------------------- labels
std::unique_ptr<Mat> gather(const OriginMat &input, const OriginMat &indices)
{
    const OriginMat &x = on_device(input, "gather");
    const Shape xs = x.shape();
    if (xs.size() != 2)
        THROW_INVALID_ARG("gather: input must be 2D (N, C), but got shape {}", xs.to_string());
    if (indices.shape().size() != 1)
        THROW_INVALID_ARG("gather: indices must be 1D (N,), but got shape {}", indices.shape().to_string());
    if (xs[0] != indices.shape()[0])
        THROW_INVALID_ARG("gather: batch size mismatch. input has {} samples, indices has {} samples", xs[0],
                          indices.shape()[0]);
    if (indices.device() != x.device())
        THROW_INVALID_ARG("gather: input and indices must be on the same device");
    const int is64 = label_kind(indices, "gather");
    auto out = fresh(x, Shape{xs[0]}, x.dtype());
    // (the labels are checked on the device; a label outside [0, C) comes back as ODL_ERR_INVALID_ARG ->
    // std::invalid_argument, the throw tests/unit_test/operator/test_softmax_cross_entropy.cpp:227-234 expects)
    check(odl_hip_gather_dtype(code(x.dtype()), vp(x), vp(indices), is64, (int64_t)xs[0], (int64_t)xs[1], out->storage()->data(),
                               kStream));
    return out;
}

std::unique_ptr<Mat> one_hot(const OriginMat &indices, int num_classes)
{
    on_device(indices, "one_hot");
    if (indices.shape().size() != 1)
        THROW_INVALID_ARG("one_hot: indices must be 1D (N,), but got shape {}", indices.shape().to_string());
    if (num_classes <= 0)
        THROW_INVALID_ARG("one_hot: num_classes must be positive, but got {}", num_classes);
    const int is64 = label_kind(indices, "one_hot");
    auto out = fresh(indices, Shape{indices.shape()[0], (size_t)num_classes});
    check(odl_hip_one_hot(vp(indices), is64, (int64_t)indices.shape()[0], num_classes, fp(*out), kStream));
    return out;
}

// ------------------------------------------------------------------------------------------- batch normalisation
namespace
{
struct BnDims
{
    int64_t N, C, P;
};

BnDims bn_dims(const char *who, const OriginMat &x, int num_dims, const OriginMat &gamma, const OriginMat &beta,
               const OriginMat &rm, const OriginMat &rv)
{
    if (x.shape().size() != (size_t)num_dims)
        THROW_INVALID_ARG("{}: x must have {} dimensions, but got shape {}", who, num_dims, x.shape().to_string());
    if (num_dims != 2 && num_dims != 4)
        THROW_INVALID_ARG("{}: num_dims must be 2 or 4, but got {}", who, num_dims);
    const size_t C = x.shape()[1];
    const Shape cs{C};
    if (gamma.shape() != cs || beta.shape() != cs || rm.shape() != cs || rv.shape() != cs)
        THROW_INVALID_ARG("{}: gamma, beta, running_mean, running_var must have shape ({})", who, C);
    if (x.dtype() != DataType::kFloat32 && x.dtype() != DataType::kFloat64)
        THROW_INVALID_ARG("{}: input x must be float32 or float64, but got {}", who, static_cast<int>(x.dtype()));
    if (gamma.dtype() != x.dtype() || beta.dtype() != x.dtype() || rm.dtype() != x.dtype() || rv.dtype() != x.dtype())
        THROW_INVALID_ARG("{}: all inputs (x, gamma, beta, running_mean, running_var) must have the same floating-point dtype",
                          who);
    return BnDims{(int64_t)x.shape()[0], (int64_t)C, num_dims == 4 ? (int64_t)(x.shape()[2] * x.shape()[3]) : (int64_t)1};
}

}  // namespace

BatchNormForwardResult batch_norm_forward(const OriginMat &x, const OriginMat &gamma, const OriginMat &beta,
                                          const OriginMat &running_mean, const OriginMat &running_var, bool training,
                                          float eps, int num_dims)
{
    on_device(x, "batch_norm");
    const BnDims d = bn_dims("batch_norm", x, num_dims, gamma, beta, running_mean, running_var);
    const Shape cs{(size_t)d.C};
    BatchNormForwardResult r;
    auto y = fresh(x, x.shape(), x.dtype()), xn = fresh(x, x.shape(), x.dtype());
    auto mean = fresh(x, cs, x.dtype()), var = fresh(x, cs, x.dtype());
    if (x.dtype() == DataType::kFloat64)
        check(odl_hip_batch_norm_forward_f64(dp(x), dp(gamma), dp(beta), dp(running_mean), dp(running_var), training ? 1 : 0,
                                             (double)eps, d.N, d.C, d.P, dp(*y), dp(*mean), dp(*var), dp(*xn), kStream));
    else
    {
        Workspace ws(training ? odl_hip_batch_norm_workspace_bytes(d.N, d.C, d.P) : 0, x);
        check(odl_hip_batch_norm_forward(fp(x), fp(gamma), fp(beta), fp(running_mean), fp(running_var), training ? 1 : 0, eps,
                                         d.N, d.C, d.P, fp(*y), fp(*mean), fp(*var), fp(*xn), ws.ptr(), ws.bytes, kStream));
    }
    r.y = std::move(y), r.mean = std::move(mean), r.var = std::move(var), r.x_norm = std::move(xn);
    return r;
}

std::unique_ptr<Mat> batch_norm(const OriginMat &x, const OriginMat &gamma, const OriginMat &beta,
                                const OriginMat &running_mean, const OriginMat &running_var, bool training, float eps, float,
                                int num_dims)
{
    return std::move(batch_norm_forward(x, gamma, beta, running_mean, running_var, training, eps, num_dims).y);
}

std::vector<std::unique_ptr<Mat>> batch_norm_backward(const OriginMat &gy, const OriginMat &x, const OriginMat &gamma,
                                                      const OriginMat &saved_mean, const OriginMat &saved_var,
                                                      const OriginMat &saved_x_norm, float eps, int num_dims)
{
    on_device(x, "batch_norm_backward");
    if (x.shape().size() != (size_t)num_dims)
        THROW_INVALID_ARG("batch_norm_backward: x must have {} dimensions, but got shape {}", num_dims, x.shape().to_string());
    if (num_dims != 2 && num_dims != 4)
        THROW_INVALID_ARG("batch_norm_backward: num_dims must be 2 or 4, but got {}", num_dims);
    const size_t C = x.shape()[1];
    const Shape cs{C};
    if (gy.shape() != x.shape() || gamma.shape() != cs || saved_mean.shape() != cs || saved_var.shape() != cs ||
        saved_x_norm.shape() != x.shape())
        THROW_INVALID_ARG("batch_norm_backward: shape mismatch");
    if (x.dtype() != DataType::kFloat32 && x.dtype() != DataType::kFloat64)
        THROW_INVALID_ARG("batch_norm_backward: input x must be float32 or float64, but got {}", static_cast<int>(x.dtype()));
    if (gy.dtype() != x.dtype() || gamma.dtype() != x.dtype() || saved_mean.dtype() != x.dtype() ||
        saved_var.dtype() != x.dtype() || saved_x_norm.dtype() != x.dtype())
        THROW_INVALID_ARG("batch_norm_backward: all inputs (gy, x, gamma, saved_mean, saved_var, saved_x_norm) must have the "
                          "same floating-point dtype");
    const int64_t N = (int64_t)x.shape()[0], P = num_dims == 4 ? (int64_t)(x.shape()[2] * x.shape()[3]) : 1;
    auto gx = fresh(x, x.shape(), x.dtype());
    auto dgamma = fresh(x, cs, x.dtype()), dbeta = fresh(x, cs, x.dtype());
    if (x.dtype() == DataType::kFloat64)
    {
        if (N > 0)
            check(odl_hip_batch_norm_backward_f64(dp(gy), dp(saved_x_norm), 0, dp(gamma), dp(saved_mean), dp(saved_var),
                                                  (double)eps, N, (int64_t)C, P, dp(*gx), dp(*dgamma), dp(*dbeta), kStream));
    }
    else
    {
        Workspace ws(odl_hip_batch_norm_workspace_bytes(N, (int64_t)C, P), x);
        check(odl_hip_batch_norm_backward(fp(gy), fp(gamma), fp(saved_var), fp(saved_x_norm), eps, N, (int64_t)C, P, fp(*gx),
                                          fp(*dgamma), fp(*dbeta), ws.ptr(), ws.bytes, kStream));
    }
    std::vector<std::unique_ptr<Mat>> outs;
    outs.push_back(std::move(gx)), outs.push_back(std::move(dgamma)), outs.push_back(std::move(dbeta));
    return outs;
}

RMSNormForwardResult rms_norm_forward(const OriginMat &, const OriginMat &, float) { not_on_this_backend("rms_norm_forward"); }
std::unique_ptr<Mat> rms_norm(const OriginMat &, const OriginMat &, float) { not_on_this_backend("rms_norm"); }
std::vector<std::unique_ptr<Mat>> rms_norm_backward(const OriginMat &, const OriginMat &, const OriginMat &, const OriginMat &,
                                                    float)
{
    not_on_this_backend("rms_norm_backward");
}

// ------------------------------------------------------------------------------------------- detector forward path
std::unique_ptr<Mat> upsample(const OriginMat &x_, const Shape &output_shape, int scale_h, int scale_w, const std::string &)
{
    const OriginMat &x = on_device(x_, "upsample");
    const Shape xs = x.shape();
    if (xs.size() != 4)
        THROW_INVALID_ARG("Upsample: input must be 4D (N, C, H, W), but got shape {}", xs.to_string());
    if (output_shape.size() != 4)
        THROW_INVALID_ARG("Upsample: output_shape must be 4D (N, C, OH, OW), but got shape {}", output_shape.to_string());
    auto y = fresh(x, output_shape, x.dtype());
    check(odl_hip_upsample_nearest_dtype(code(x.dtype()), vp(x), (int64_t)xs[0], (int64_t)xs[1], (int64_t)xs[2], (int64_t)xs[3],
                                         (int64_t)output_shape[2], (int64_t)output_shape[3], scale_h, scale_w,
                                         y->storage()->data(), kStream));
    return y;
}

std::unique_ptr<Mat> upsample_backward(const OriginMat &gy_, const Shape &xs, int scale_h, int scale_w, const std::string &)
{
    const OriginMat &gy = on_device(gy_, "upsample_backward");
    if (gy.shape().size() != 4)
        THROW_INVALID_ARG("Upsample backward: gradient must be 4D (N, C, OH, OW), but got shape {}", gy.shape().to_string());
    if (xs.size() != 4)
        THROW_INVALID_ARG("Upsample backward: x_shape must be 4D (N, C, H, W), but got shape {}", xs.to_string());
    auto gx = fresh(gy, xs, gy.dtype());
    check(odl_hip_upsample_nearest_backward_dtype(code(gy.dtype()), vp(gy), (int64_t)xs[0], (int64_t)xs[1], (int64_t)xs[2],
                                                  (int64_t)xs[3], (int64_t)gy.shape()[2], (int64_t)gy.shape()[3], scale_h,
                                                  scale_w, gx->storage()->data(), kStream));
    return gx;
}

std::unique_ptr<Mat> yolo_detect_forward(const OriginMat &input, const OriginMat &conv_weight, const OriginMat *conv_bias,
                                         const OriginMat &grid, const OriginMat &anchor_grid, float stride,
                                         int32_t num_anchors, int32_t num_classes)
{
    const OriginMat &x = f32(input, "yolo_detect_forward"), &w = f32(conv_weight, "yolo_detect_forward");
    const OriginMat &g = f32(grid, "yolo_detect_forward"), &ag = f32(anchor_grid, "yolo_detect_forward");
    const Shape xs = x.shape();
    if (xs.size() != 4)
        THROW_INVALID_ARG("yolo_detect_forward: input must be 4D (N, C, H, W), but got shape {}", xs.to_string());
    const int64_t N = xs[0], C = xs[1], H = xs[2], W = xs[3], CI = num_classes + 5;
    const Shape wsh = w.shape();
    if (wsh.size() != 4 || (int64_t)wsh[0] != num_anchors * CI || (int64_t)wsh[1] != C || wsh[2] != 1 || wsh[3] != 1)
        THROW_INVALID_ARG("yolo_detect_forward: conv weight {} does not match [{}, {}, 1, 1]", wsh.to_string(),
                          num_anchors * CI, C);
    const Shape as = ag.shape();
    const int64_t aH = as.size() >= 3 ? (int64_t)as[2] : H, aW = as.size() >= 4 ? (int64_t)as[3] : W;
    auto y = fresh(x, Shape{(size_t)N, (size_t)(H * W * num_anchors), (size_t)CI});
    Workspace ws(odl_hip_yolo_detect_workspace_bytes(N, C, H, W, num_anchors, num_classes), x);
    check(odl_hip_yolo_detect_forward(fp(x), fp(w), conv_bias ? fp(f32(*conv_bias, "yolo_detect_forward")) : nullptr, fp(g),
                                      (int64_t)g.elements(), fp(ag), (int64_t)ag.elements(), aH, aW, N, C, H, W, stride,
                                      num_anchors, num_classes, fp(*y), ws.ptr(), ws.bytes, kStream));
    return y;
}

// ------------------------------------------------------------------------------------------- outside the hot path
std::unique_ptr<Mat> dropout(const OriginMat &, float, bool, OriginMat *) { not_on_this_backend("dropout"); }
std::unique_ptr<Mat> dropout_backward(const OriginMat &, const OriginMat &) { not_on_this_backend("dropout_backward"); }
std::unique_ptr<Mat> embedding(const OriginMat &, const OriginMat &) { not_on_this_backend("embedding"); }
std::unique_ptr<Mat> embedding_backward(const OriginMat &, const OriginMat &, int, int) { not_on_this_backend("embedding_backward"); }
}  // namespace cuda
}  // namespace origin
