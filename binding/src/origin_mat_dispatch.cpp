// OriginMat, the device dispatcher of OriginDL, with its device branch enabled on the gfx950 backend.
//
// This translation unit stands where the reference's src/mat/origin/origin_mat.cpp stands, against the reference's own
// class declaration (include/origin/mat/origin/origin_mat.h): every method sends a tensor that lives on the host to the
// reference's own CPU kernels (origin::cpu::*, compiled from the reference's sources) and a tensor that lives on the
// device to the origin::cuda::* entry points of include/origin/mat/origin/cuda/cuda_ops.cuh and cuda/factory.cuh, which
// hip_ops.cpp defines over libodl_hip.so. The reference's file cannot be compiled with those branches: they sit behind
// WITH_CUDA together with `#include <cuda_runtime.h>` and direct cudaMemcpy / cudaDeviceSynchronize calls
// (origin_mat.cpp:46-51, 1002-1010).
#include <cstring>

#include "odl_hip.h"
#include "origin/mat/origin/cpu/cpu_ops.h"
#include "origin/mat/origin/cpu/factory.h"
#include "origin/mat/origin/cuda/cuda_ops.cuh"
#include "origin/mat/origin/cuda/factory.cuh"
#include "origin/mat/origin/origin_mat.h"
#include "origin/mat/origin/origin_mat_utils.h"
#include "origin/mat/scalar.h"
#include "origin/utils/exception.h"

namespace origin
{
namespace
{
// the OriginMat behind a Mat handed in through the abstract interface
const OriginMat &om(const Mat &m, const char *op, const char *role)
{
    const auto *p = dynamic_cast<const OriginMat *>(&m);
    if (!p)
        THROW_RUNTIME_ERROR("{}: {} must be OriginMat type, got backend_type={}", op, role, m.backend_type());
    return *p;
}

const OriginMat *om(const Mat *m, const char *op, const char *role)
{
    return m ? &om(*m, op, role) : nullptr;
}

[[noreturn]] void bad_device(const char *op, DeviceType t)
{
    THROW_RUNTIME_ERROR("Unsupported device type for {}: {}", op, static_cast<int>(t));
}
}  // namespace

// `cpu_expr` for a host tensor, `dev_expr` for a device tensor; `where` is the Mat whose storage decides
#define ODL_ON(where, op, cpu_expr, dev_expr)                          \
    do                                                                 \
    {                                                                  \
        const DeviceType odl_t__ = (where).storage()->device_type();   \
        if (odl_t__ == DeviceType::kCPU)                               \
            return cpu_expr;                                           \
        if (odl_t__ == DeviceType::kCUDA)                              \
            return dev_expr;                                           \
        bad_device(op, odl_t__);                                       \
    } while (0)

// the same call in both namespaces
#define ODL_BOTH(where, op, ...) ODL_ON(where, #op, cpu::op(__VA_ARGS__), cuda::op(__VA_ARGS__))

// ------------------------------------------------------------------------------------------- construction
OriginMat::OriginMat(std::shared_ptr<Storage> storage, const Shape &shape, DataType dtype)
    : storage_(std::move(storage)), shape_(shape), dtype_(dtype)
{
    utils::validate_shape(shape);
    strides_ = utils::compute_strides(shape);
}

OriginMat::OriginMat(std::shared_ptr<Storage> storage, const Shape &shape, const std::vector<size_t> &strides, DataType dtype)
    : storage_(std::move(storage)), shape_(shape), dtype_(dtype), strides_(strides)
{
    utils::validate_shape(shape);
    if (strides.size() != shape.size())
        THROW_INVALID_ARG("Strides size {} must match shape size {}", strides.size(), shape.size());
}

OriginMat::OriginMat(const Shape &shape, DataType dtype) : OriginMat(shape, dtype, Device(DeviceType::kCPU)) {}

OriginMat::OriginMat(const Shape &shape, DataType dtype, Device device) : shape_(shape), dtype_(dtype)
{
    utils::validate_shape(shape);
    strides_ = utils::compute_strides(shape);
    storage_ = Storage::create(shape_.elements() * element_size(dtype_), device.type(), device.index());
}

#define ODL_FACTORY(opts, cpu_expr, dev_expr)                   \
    do                                                          \
    {                                                           \
        if ((opts).device().type() == DeviceType::kCUDA)        \
            return dev_expr;                                    \
        return cpu_expr;                                        \
    } while (0)

std::unique_ptr<Mat> OriginMat::from_scalar(const Scalar &scalar, const Shape &shape, const TensorOptions &options)
{
    utils::validate_shape(shape);
    ODL_FACTORY(options, cpu::full(shape, scalar, options), cuda::full(shape, scalar, options));
}

std::unique_ptr<Mat> OriginMat::from_memory(const void *data, DataType user_dtype, const Shape &shape,
                                            const TensorOptions &options)
{
    utils::validate_shape(shape);
    ODL_FACTORY(options, cpu::from_memory(data, user_dtype, shape, options),
                cuda::from_memory(data, user_dtype, shape, options));
}

std::unique_ptr<Mat> OriginMat::randn(const Shape &shape, const TensorOptions &options)
{
    // drawn on the host by the reference's generator, then moved (origin_mat.cpp:1137-1152)
    if (options.device().type() != DeviceType::kCUDA)
        return cpu::randn(shape, options);
    return cpu::randn(shape, TensorOptions(options.dtype()).device(DeviceType::kCPU))->to_device(options.device());
}

std::unique_ptr<Mat> OriginMat::zeros(const Shape &shape, const TensorOptions &options)
{
    ODL_FACTORY(options, cpu::zeros(shape, options), cuda::zeros(shape, options));
}

std::unique_ptr<Mat> OriginMat::ones(const Shape &shape, const TensorOptions &options)
{
    ODL_FACTORY(options, cpu::ones(shape, options), cuda::ones(shape, options));
}

std::unique_ptr<Mat> OriginMat::full(const Shape &shape, float value, const TensorOptions &options)
{
    ODL_FACTORY(options, cpu::full(shape, value, options), cuda::full(shape, value, options));
}

// ------------------------------------------------------------------------------------------- shape, views
std::unique_ptr<Mat> OriginMat::clone() const
{
    ODL_BOTH(*this, clone, *this);
}

std::unique_ptr<Mat> OriginMat::view(const Shape &new_shape) const
{
    if (new_shape.elements() != shape_.elements())
        THROW_INVALID_ARG("View: total elements must match. Original: {}, Target: {}", shape_.elements(),
                          new_shape.elements());
    utils::validate_shape(new_shape);
    return std::make_unique<OriginMat>(storage_, new_shape, dtype_);  // the same storage, from its first byte
}

bool OriginMat::is_contiguous() const
{
    return shape_.size() == 0 || strides_ == utils::compute_strides(shape_);
}

std::unique_ptr<Mat> OriginMat::contiguous() const
{
    return is_contiguous() ? view(shape_) : clone();
}

std::unique_ptr<Mat> OriginMat::reshape(const Shape &new_shape) const
{
    if (new_shape.elements() != shape_.elements())
        THROW_INVALID_ARG("Reshape: total elements must match. Original: {}, Target: {}", shape_.elements(),
                          new_shape.elements());
    return is_contiguous() ? view(new_shape) : contiguous()->view(new_shape);
}

std::unique_ptr<Mat> OriginMat::transpose() const
{
    ODL_BOTH(*this, transpose, *this);
}

std::unique_ptr<Mat> OriginMat::permute(const std::vector<int> &dims) const
{
    ODL_BOTH(*this, permute, *this, dims);
}

Shape OriginMat::shape() const
{
    return shape_;
}

size_t OriginMat::elements() const
{
    return shape_.elements();
}

bool OriginMat::is_scalar() const
{
    return shape_.is_scalar();
}

bool OriginMat::can_broadcast_to(const Shape &target_shape) const
{
    return utils::can_broadcast_to(shape_, target_shape);
}

DataType OriginMat::dtype() const
{
    return dtype_;
}

Device OriginMat::device() const
{
    return Device(storage_->device_type(), storage_->device_index());
}

int OriginMat::backend_type() const
{
    return ORIGIN_BACKEND_TYPE;
}

std::unique_ptr<Mat> OriginMat::to(DataType target_type) const
{
    ODL_BOTH(*this, convert_datatype, *this, target_type);
}

std::unique_ptr<Mat> OriginMat::to_device(Device device) const
{
    return std::make_unique<OriginMat>(storage_->to_device(device.type(), device.index()), shape_, dtype_);
}

// ------------------------------------------------------------------------------------------- reading values
Scalar OriginMat::scalar_value() const
{
    if (!is_scalar())
        THROW_INVALID_ARG("scalar_value() can only be called on scalar tensors (0-dimensional tensors)");
    if (storage_->device_type() == DeviceType::kCPU)
        return utils::compute::get_scalar_value(storage_->data(), dtype_);
    return utils::compute::get_scalar_value(storage_->to_device(DeviceType::kCPU, 0)->data(), dtype_);
}

std::vector<float> OriginMat::to_vector() const
{
    if (!is_contiguous())
        return static_cast<const OriginMat &>(*contiguous()).to_vector();
    if (storage_->device_type() == DeviceType::kCPU)
        return utils::compute::convert_to_vector(storage_->data(), shape_.elements(), dtype_);
    return utils::compute::convert_to_vector(storage_->to_device(DeviceType::kCPU, 0)->data(), shape_.elements(), dtype_);
}

Scalar OriginMat::index(std::initializer_list<size_t> indices) const
{
    if (indices.size() != shape_.size())
        THROW_INVALID_ARG("Index count ({}) does not match tensor dimension ({}). Shape: {}", indices.size(), shape_.size(),
                          shape_.to_string());
    size_t offset = 0, d = 0;
    for (size_t i : indices)
    {
        if (i >= shape_[d])
            THROW_INVALID_ARG("Index {} out of range for dimension {} (size: {}). Shape: {}", i, d, shape_[d],
                              shape_.to_string());
        offset += i * strides_[d++];
    }
    const size_t width = element_size(dtype_);
    alignas(8) unsigned char element[8] = {0};
    const unsigned char *src = static_cast<const unsigned char *>(storage_->data()) + offset * width;
    if (storage_->device_type() == DeviceType::kCPU)
        std::memcpy(element, src, width);
    else if (odl_hip_memcpy_d2h(element, src, width) != ODL_OK)  // (waits for the device first)
        THROW_RUNTIME_ERROR("index: {}", odl_hip_last_error());
    return utils::compute::get_scalar_value(element, dtype_);
}

void OriginMat::index_put(std::initializer_list<size_t> indices, const Scalar &value)
{
    ODL_BOTH(*this, index_put, *this, indices, value);
}

void OriginMat::print(const std::string &desc) const
{
    utils::visualize::print_origin_mat(desc, to_vector(), shape_.dims(), dtype_, device().to_string());
}

// ------------------------------------------------------------------------------------------- arithmetic
#define ODL_BINARY(method, inplace, op)                                                            \
    std::unique_ptr<Mat> OriginMat::method(const Mat &other) const                                 \
    {                                                                                              \
        const OriginMat &o = static_cast<const OriginMat &>(other);                                \
        ODL_ON(*this, #op, cpu::op(*this, o, nullptr), cuda::op(*this, o, nullptr));               \
    }
#define ODL_BINARY_INPLACE(inplace, compound, op)                                                  \
    void OriginMat::inplace(const Mat &other)                                                      \
    {                                                                                              \
        const OriginMat &o = static_cast<const OriginMat &>(other);                                \
        ODL_ON(*this, #inplace, (void)cpu::op(*this, o, this), (void)cuda::op(*this, o, this));    \
    }                                                                                              \
    Mat &OriginMat::compound(const Mat &other)                                                     \
    {                                                                                              \
        inplace(other);                                                                            \
        return *this;                                                                              \
    }
ODL_BINARY(operator+, add_inplace, add)
ODL_BINARY(operator-, sub_inplace, subtract)
ODL_BINARY(operator*, mul_inplace, multiply)
ODL_BINARY(operator/, div_inplace, divide)
ODL_BINARY(operator==, , eq)
ODL_BINARY(operator!=, , ne)
ODL_BINARY(operator<, , lt)
ODL_BINARY(operator<=, , le)
ODL_BINARY(operator>, , gt)
ODL_BINARY(operator>=, , ge)
ODL_BINARY_INPLACE(add_inplace, operator+=, add)
ODL_BINARY_INPLACE(sub_inplace, operator-=, subtract)
ODL_BINARY_INPLACE(mul_inplace, operator*=, multiply)
ODL_BINARY_INPLACE(div_inplace, operator/=, divide)

#define ODL_UNARY(method, op)                                                            \
    std::unique_ptr<Mat> OriginMat::method() const                                       \
    {                                                                                    \
        ODL_ON(*this, #op, cpu::op(*this, nullptr), cuda::op(*this, nullptr));           \
    }
#define ODL_UNARY_INPLACE(method, op)                                                    \
    void OriginMat::method()                                                             \
    {                                                                                    \
        ODL_ON(*this, #method, (void)cpu::op(*this, this), (void)cuda::op(*this, this)); \
    }
ODL_UNARY(operator-, negate)
ODL_UNARY(square, square)
ODL_UNARY(exp, exp)
ODL_UNARY(log, log)
ODL_UNARY(sqrt, sqrt)
ODL_UNARY(relu, relu)
ODL_UNARY(sigmoid, sigmoid)
ODL_UNARY(silu, silu)
ODL_UNARY_INPLACE(neg_inplace, negate)
ODL_UNARY_INPLACE(square_inplace, square)
ODL_UNARY_INPLACE(exp_inplace, exp)
ODL_UNARY_INPLACE(log_inplace, log)
ODL_UNARY_INPLACE(sqrt_inplace, sqrt)
ODL_UNARY_INPLACE(relu_inplace, relu)

std::unique_ptr<Mat> OriginMat::sin() const
{
    THROW_RUNTIME_ERROR("sin function not implemented yet");
}

std::unique_ptr<Mat> OriginMat::cos() const
{
    THROW_RUNTIME_ERROR("cos function not implemented yet");
}

std::unique_ptr<Mat> OriginMat::pow(const Scalar &exponent) const
{
    ODL_ON(*this, "pow", cpu::pow(*this, exponent), cuda::pow(*this, exponent, nullptr));
}

void OriginMat::pow_inplace(const Scalar &exponent)
{
    ODL_BOTH(*this, pow_inplace, *this, exponent);
}

std::unique_ptr<Mat> OriginMat::leaky_relu(const Mat &other) const
{
    const OriginMat &alpha = static_cast<const OriginMat &>(other);
    ODL_ON(*this, "leaky_relu", cpu::leaky_relu(*this, alpha), cuda::leaky_relu(*this, alpha, nullptr));
}

std::unique_ptr<Mat> OriginMat::sigmoid_backward(const Mat &y) const
{
    ODL_BOTH(*this, sigmoid_backward, *this, om(y, "sigmoid_backward", "y"));
}

std::unique_ptr<Mat> OriginMat::silu_backward(const Mat &x) const
{
    ODL_BOTH(*this, silu_backward, *this, om(x, "silu_backward", "x"));
}

// ------------------------------------------------------------------------------------------- products, reductions
std::unique_ptr<Mat> OriginMat::matmul(const Mat &other) const
{
    ODL_BOTH(*this, matmul, *this, static_cast<const OriginMat &>(other));
}

std::unique_ptr<Mat> OriginMat::sum(int axis, bool keepdim) const
{
    ODL_BOTH(*this, sum, *this, axis, keepdim);
}

std::unique_ptr<Mat> OriginMat::max(int axis) const
{
    ODL_BOTH(*this, max, *this, axis);
}

std::unique_ptr<Mat> OriginMat::broadcast_to(const Shape &target_shape) const
{
    ODL_BOTH(*this, broadcast_to, *this, target_shape);
}

std::unique_ptr<Mat> OriginMat::sum_to(const Shape &target_shape) const
{
    ODL_BOTH(*this, sum_to, *this, target_shape);
}

// ------------------------------------------------------------------------------------------- convolution, pooling
std::unique_ptr<Mat> OriginMat::im2col(std::pair<int, int> kernel_size, std::pair<int, int> stride, std::pair<int, int> pad,
                                       bool to_matrix) const
{
    ODL_BOTH(*this, im2col, *this, kernel_size, stride, pad, to_matrix);
}

std::unique_ptr<Mat> OriginMat::col2im(const Shape &input_shape, std::pair<int, int> kernel_size, std::pair<int, int> stride,
                                       std::pair<int, int> pad, bool to_matrix) const
{
    ODL_BOTH(*this, col2im, *this, input_shape, kernel_size, stride, pad, to_matrix);
}

std::unique_ptr<Mat> OriginMat::conv2d(const Mat &W, const Mat *b, std::pair<int, int> stride, std::pair<int, int> pad) const
{
    ODL_BOTH(*this, conv2d, *this, om(W, "conv2d", "W"), om(b, "conv2d", "b"), stride, pad);
}

std::vector<std::unique_ptr<Mat>> OriginMat::conv2d_backward(const Mat &gy, const Mat &x, const Mat &W, const Mat *b,
                                                             std::pair<int, int> stride, std::pair<int, int> pad) const
{
    ODL_BOTH(*this, conv2d_backward, om(gy, "conv2d_backward", "gy"), om(x, "conv2d_backward", "x"),
             om(W, "conv2d_backward", "W"), om(b, "conv2d_backward", "b"), stride, pad);
}

std::unique_ptr<Mat> OriginMat::avg_pool2d(std::pair<int, int> kernel_size, std::pair<int, int> stride,
                                           std::pair<int, int> pad) const
{
    ODL_BOTH(*this, avg_pool2d, *this, kernel_size, stride, pad);
}

std::unique_ptr<Mat> OriginMat::avg_pool2d_backward(const Mat &gy, std::pair<int, int> kernel_size,
                                                    std::pair<int, int> stride, std::pair<int, int> pad) const
{
    ODL_BOTH(*this, avg_pool2d_backward, om(gy, "avg_pool2d_backward", "gy"), *this, kernel_size, stride, pad);
}

std::unique_ptr<Mat> OriginMat::adaptive_avg_pool2d(std::pair<int, int> output_size) const
{
    ODL_BOTH(*this, adaptive_avg_pool2d, *this, output_size);
}

std::unique_ptr<Mat> OriginMat::adaptive_avg_pool2d_backward(const Mat &gy, std::pair<int, int> output_size) const
{
    ODL_BOTH(*this, adaptive_avg_pool2d_backward, om(gy, "adaptive_avg_pool2d_backward", "gy"), *this, output_size);
}

std::unique_ptr<Mat> OriginMat::max_pool2d(std::pair<int, int> kernel_size, std::pair<int, int> stride,
                                           std::pair<int, int> pad, std::vector<size_t> *indices) const
{
    ODL_BOTH(*this, max_pool2d, *this, kernel_size, stride, pad, indices);
}

std::unique_ptr<Mat> OriginMat::max_pool2d_backward(const Mat &gy, std::pair<int, int> kernel_size,
                                                    std::pair<int, int> stride, std::pair<int, int> pad,
                                                    const std::vector<size_t> &indices) const
{
    ODL_BOTH(*this, max_pool2d_backward, om(gy, "max_pool2d_backward", "gy"), *this, kernel_size, stride, pad, indices);
}

// ------------------------------------------------------------------------------------------- normalisation
OriginMat::BatchNormResult OriginMat::batch_norm_forward(const Mat &gamma, const Mat &beta, const Mat &running_mean,
                                                         const Mat &running_var, bool training, float eps,
                                                         int num_dims) const
{
    const OriginMat &g = om(gamma, "batch_norm_forward", "gamma"), &b = om(beta, "batch_norm_forward", "beta");
    const OriginMat &rm = om(running_mean, "batch_norm_forward", "running_mean");
    const OriginMat &rv = om(running_var, "batch_norm_forward", "running_var");
    auto pack = [](auto &&r) {
        BatchNormResult out;
        out.y = std::move(r.y), out.mean = std::move(r.mean), out.var = std::move(r.var), out.x_norm = std::move(r.x_norm);
        return out;
    };
    ODL_ON(*this, "batch_norm_forward", pack(cpu::batch_norm_forward(*this, g, b, rm, rv, training, eps, num_dims)),
           pack(cuda::batch_norm_forward(*this, g, b, rm, rv, training, eps, num_dims)));
}

std::unique_ptr<Mat> OriginMat::batch_norm(const Mat &gamma, const Mat &beta, const Mat &running_mean, const Mat &running_var,
                                           bool training, float eps, float momentum, int num_dims) const
{
    ODL_BOTH(*this, batch_norm, *this, om(gamma, "batch_norm", "gamma"), om(beta, "batch_norm", "beta"),
             om(running_mean, "batch_norm", "running_mean"), om(running_var, "batch_norm", "running_var"), training, eps,
             momentum, num_dims);
}

std::vector<std::unique_ptr<Mat>> OriginMat::batch_norm_backward(const Mat &gy, const Mat &gamma, const Mat &saved_mean,
                                                                 const Mat &saved_var, const Mat &saved_x_norm, float eps,
                                                                 int num_dims) const
{
    ODL_BOTH(*this, batch_norm_backward, om(gy, "batch_norm_backward", "gy"), *this,
             om(gamma, "batch_norm_backward", "gamma"), om(saved_mean, "batch_norm_backward", "saved_mean"),
             om(saved_var, "batch_norm_backward", "saved_var"), om(saved_x_norm, "batch_norm_backward", "saved_x_norm"),
             eps, num_dims);
}

OriginMat::RMSNormResult OriginMat::rms_norm_forward(const Mat &gamma, float eps) const
{
    const OriginMat &g = om(gamma, "rms_norm_forward", "gamma");
    auto pack = [](auto &&r) {
        RMSNormResult out;
        out.y = std::move(r.y), out.rms = std::move(r.rms);
        return out;
    };
    ODL_ON(*this, "rms_norm_forward", pack(cpu::rms_norm_forward(*this, g, eps)), pack(cuda::rms_norm_forward(*this, g, eps)));
}

std::unique_ptr<Mat> OriginMat::rms_norm(const Mat &gamma, float eps) const
{
    ODL_BOTH(*this, rms_norm, *this, om(gamma, "rms_norm", "gamma"), eps);
}

std::vector<std::unique_ptr<Mat>> OriginMat::rms_norm_backward(const Mat &gy, const Mat &gamma, const Mat &saved_rms,
                                                               float eps) const
{
    ODL_BOTH(*this, rms_norm_backward, om(gy, "rms_norm_backward", "gy"), *this, om(gamma, "rms_norm_backward", "gamma"),
             om(saved_rms, "rms_norm_backward", "saved_rms"), eps);
}

// ------------------------------------------------------------------------------------------- the rest
std::unique_ptr<Mat> OriginMat::gather(const Mat &indices) const
{
    ODL_BOTH(*this, gather, *this, om(indices, "gather", "indices"));
}

std::unique_ptr<Mat> OriginMat::one_hot(const Mat &indices, int num_classes) const
{
    const OriginMat &idx = om(indices, "one_hot", "indices");  // the labels decide where the result lives
    ODL_BOTH(idx, one_hot, idx, num_classes);
}

std::unique_ptr<Mat> OriginMat::yolo_detect_forward(const Mat &conv_weight, const Mat *conv_bias, const Mat &grid,
                                                    const Mat &anchor_grid, float stride, int32_t num_anchors,
                                                    int32_t num_classes) const
{
    ODL_BOTH(*this, yolo_detect_forward, *this, om(conv_weight, "yolo_detect_forward", "conv_weight"),
             om(conv_bias, "yolo_detect_forward", "conv_bias"), om(grid, "yolo_detect_forward", "grid"),
             om(anchor_grid, "yolo_detect_forward", "anchor_grid"), stride, num_anchors, num_classes);
}

std::unique_ptr<Mat> OriginMat::dropout(float p, bool training, Mat *mask) const
{
    OriginMat *m = mask ? const_cast<OriginMat *>(&om(*mask, "dropout", "mask")) : nullptr;
    ODL_BOTH(*this, dropout, *this, p, training, m);
}

std::unique_ptr<Mat> OriginMat::dropout_backward(const Mat &gy, const Mat &mask) const
{
    ODL_BOTH(*this, dropout_backward, om(gy, "dropout_backward", "gy"), om(mask, "dropout_backward", "mask"));
}

std::unique_ptr<Mat> OriginMat::embedding(const Mat &vocab) const
{
    ODL_BOTH(*this, embedding, *this, om(vocab, "embedding", "vocab"));
}

std::unique_ptr<Mat> OriginMat::embedding_back(const Mat &indices, int vocab_size, int embedding_dim) const
{
    ODL_BOTH(*this, embedding_backward, *this, om(indices, "embedding_back", "indices"), vocab_size, embedding_dim);
}

std::unique_ptr<Mat> OriginMat::upsample(const Shape &output_shape, int scale_h, int scale_w, const std::string &mode) const
{
    ODL_BOTH(*this, upsample, *this, output_shape, scale_h, scale_w, mode);
}

std::unique_ptr<Mat> OriginMat::upsample_backward(const Mat &gy, const Shape &x_shape, int scale_h, int scale_w,
                                                  const std::string &mode) const
{
    ODL_BOTH(*this, upsample_backward, om(gy, "upsample_backward", "gy"), x_shape, scale_h, scale_w, mode);
}

std::unique_ptr<Mat> OriginMat::cat(const std::vector<const Mat *> &others, int dim) const
{
    if (others.empty())
        return clone();
    std::vector<const OriginMat *> inputs{this};
    for (const Mat *m : others)
        inputs.push_back(&om(*m, "cat", "input"));
    ODL_BOTH(*this, cat, inputs, dim);
}

std::vector<std::unique_ptr<Mat>> OriginMat::split(const std::vector<size_t> &split_sizes, int dim) const
{
    ODL_BOTH(*this, split, *this, split_sizes, dim);
}
}  // namespace origin
