// The operators that call the hot path (forward/backward pairs over Mat) and their functional:: wrappers and
// arithmetic overloads. Names, argument meaning and gradients follow the reference's src/operators/** for:
// add sub mul div neg pow exp log square sum sum_to broadcast_to mat_mul reshape transpose flatten relu softmax
// softmax_cross_entropy conv2d max_pool2d.
#pragma once
#include <string>

#include <initializer_list>
#include <type_traits>

#include "tensor.h"
#include "utils/size_array_ref.h"

namespace origin
{
namespace functional
{
// src/operators/shape/split.cpp: pieces of x along dim — either the listed sizes (which must add up to the dimension)
// or equal pieces of split_size with a shorter last one; backward concatenates the pieces' gradients.
class Split : public Operator
{
public:
    int dim_;
    std::vector<size_t> split_sizes_;
    explicit Split(SizeArrayRef split_sizes, int dim = 0) : dim_(dim), split_sizes_(split_sizes.to_vector()) {}
    explicit Split(size_t split_size, int dim = 0) : dim_(dim), split_sizes_{split_size} {}
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override;
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override;
};
std::vector<Tensor> split(const Tensor &x, SizeArrayRef split_sizes, int dim = 0);
std::vector<Tensor> split(const Tensor &x, size_t split_size, int dim = 0);
// braced lists of another integer type (split(x, {1, 2, 3}, 0) deduces int)
template <typename T, typename = std::enable_if_t<std::is_integral<T>::value && !std::is_same<T, bool>::value &&
                                                  !std::is_same<T, size_t>::value>>
inline std::vector<Tensor> split(const Tensor &x, std::initializer_list<T> split_sizes, int dim = 0)
{
    std::vector<size_t> sizes;
    for (const auto &v : split_sizes)
        sizes.push_back(static_cast<size_t>(v));
    return split(x, SizeArrayRef(sizes), dim);
}

// src/operators/custom/linear.cpp: y = flatten(x) . weight^T (+ bias) with weight laid out [out_features, in_features],
// the layout of an imported model's fully connected layers. Forward only (backward throws, as there).
class LinearOp : public Operator
{
public:
    int in_features_, out_features_;
    bool use_bias_;
    LinearOp(int in_features, int out_features, bool use_bias = true)
        : in_features_(in_features), out_features_(out_features), use_bias_(use_bias)
    {}
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override;
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override;
};
Tensor custom_linear(const Tensor &x, const Tensor &weight, const Tensor &bias, int in_features, int out_features,
                     bool use_bias = true);
Tensor custom_linear(const Tensor &x, const Tensor &weight, int in_features, int out_features);

// src/operators/activation/leaky_relu.cpp: x where x > 0, alpha*x elsewhere; gx = gy * (alpha + mask*(1-alpha))
Tensor leaky_relu(const Tensor &x, float alpha = 0.01f);

Tensor add(const Tensor &lhs, const Tensor &rhs);
Tensor sub(const Tensor &lhs, const Tensor &rhs);
Tensor mul(const Tensor &lhs, const Tensor &rhs);
Tensor div(const Tensor &lhs, const Tensor &rhs);
Tensor neg(const Tensor &x);
Tensor pow(const Tensor &base, const Scalar &exponent);
Tensor exp(const Tensor &x);
Tensor log(const Tensor &x);
Tensor square(const Tensor &x);
Tensor sum(const Tensor &x, int axis = -1, bool keepdim = false);  // -1: all elements
Tensor sum_to(const Tensor &x, const Shape &shape);
Tensor broadcast_to(const Tensor &x, const Shape &shape);
Tensor mat_mul(const Tensor &x, const Tensor &w);
Tensor reshape(const Tensor &x, const Shape &shape);
Tensor transpose(const Tensor &x);
Tensor flatten(const Tensor &x, int start_dim = 1, int end_dim = -1);
Tensor relu(const Tensor &x);
Tensor sigmoid(const Tensor &x);
Tensor silu(const Tensor &x);
Tensor cat(const std::vector<Tensor> &xs, int dim = 0);
Tensor upsample(const Tensor &x, const std::string &mode = "nearest", std::pair<float, float> scale_factor = {2.0f, 2.0f});
// in-place forms: overwrite the left operand's storage
void add_(Tensor &lhs, const Tensor &rhs);
void sub_(Tensor &lhs, const Tensor &rhs);
void mul_(Tensor &lhs, const Tensor &rhs);
void div_(Tensor &lhs, const Tensor &rhs);
void neg_(Tensor &x);
void exp_(Tensor &x);
void log_(Tensor &x);
void square_(Tensor &x);
void relu_(Tensor &x);
// src/operators/normalization/batch_norm.cpp:16-139. num_dims 2 = [N, C], 4 = [N, C, H, W]; momentum is carried for
// the interface only (the layers update their running statistics themselves).
Tensor batch_norm(const Tensor &x, const Tensor &gamma, const Tensor &beta, const Tensor &running_mean,
                  const Tensor &running_var, bool training = false, float eps = 1e-5f, float momentum = 0.1f,
                  int num_dims = 4);
// the same operator with all of its outputs: y, and in training mode the batch mean and variance
std::vector<Tensor> batch_norm_outputs(const Tensor &x, const Tensor &gamma, const Tensor &beta,
                                       const Tensor &running_mean, const Tensor &running_var, bool training, float eps,
                                       float momentum, int num_dims);
// ... with a ReLU applied to y before it leaves the operator (float32 device tensors): what batch_norm then relu give
std::vector<Tensor> batch_norm_relu_outputs(const Tensor &x, const Tensor &gamma, const Tensor &beta,
                                            const Tensor &running_mean, const Tensor &running_var, bool training,
                                            float eps, float momentum, int num_dims);
// x[M,K] . w[K,N] + b (b of N elements) in one kernel; what nn::Linear::forward uses for 2-D inputs
Tensor linear(const Tensor &x, const Tensor &w, const Tensor &b);
// relu(linear(x, w, b)) and relu(conv2d(x, W, b)) as one operator each, for device tensors (float32)
Tensor linear_relu(const Tensor &x, const Tensor &w, const Tensor &b);
Tensor conv2d_relu(const Tensor &x, const Tensor &W, const Tensor *b, std::pair<int, int> stride, std::pair<int, int> pad);
// max_pool2d(relu(conv2d(x, W, b)), ...) as one operator: same values, and in backward the pooling gradient is masked by
// the ReLU as it is written
Tensor conv2d_relu_max_pool2d(const Tensor &x, const Tensor &W, const Tensor *b, std::pair<int, int> stride,
                              std::pair<int, int> pad, std::pair<int, int> pool_kernel, std::pair<int, int> pool_stride,
                              std::pair<int, int> pool_pad);
Tensor softmax(const Tensor &x, int axis = -1);
Tensor softmax_cross_entropy(const Tensor &x, const Tensor &target);
// After replaying a recorded step on new labels: whether the loss kernel met an out-of-range label (the ordinary call
// throws std::invalid_argument for one, as the reference's gather does; a recorded step cannot). `loss` is the tensor
// softmax_cross_entropy returned while the step was recorded. Reads two words back from the device.
bool softmax_cross_entropy_bad_label(const Tensor &loss);
Tensor conv2d(const Tensor &x, const Tensor &W, const Tensor *b = nullptr, std::pair<int, int> stride = {1, 1},
              std::pair<int, int> pad = {0, 0});
Tensor conv2d(const Tensor &x, const Tensor &W, const Tensor *b, int stride, int pad);
Tensor max_pool2d(const Tensor &x, std::pair<int, int> kernel_size, std::pair<int, int> stride = {0, 0},
                  std::pair<int, int> pad = {0, 0});
Tensor max_pool2d(const Tensor &x, int kernel_size, int stride = 0, int pad = 0);
}  // namespace functional

using functional::conv2d;

Tensor operator+(const Tensor &lhs, const Tensor &rhs);
Tensor operator+(const Tensor &lhs, const Scalar &rhs);
Tensor operator+(const Scalar &lhs, const Tensor &rhs);
Tensor operator-(const Tensor &lhs, const Tensor &rhs);
Tensor operator-(const Tensor &lhs, const Scalar &rhs);
Tensor operator-(const Scalar &lhs, const Tensor &rhs);
Tensor operator*(const Tensor &lhs, const Tensor &rhs);
Tensor operator*(const Tensor &lhs, const Scalar &rhs);
Tensor operator*(const Scalar &lhs, const Tensor &rhs);
Tensor operator/(const Tensor &lhs, const Tensor &rhs);
Tensor operator/(const Tensor &lhs, const Scalar &rhs);
Tensor operator/(const Scalar &lhs, const Tensor &rhs);
Tensor operator-(const Tensor &x);
Tensor operator^(const Tensor &base, const Scalar &exponent);
Tensor operator>(const Tensor &lhs, const Tensor &rhs);
Tensor operator>(const Tensor &lhs, const Scalar &rhs);
Tensor operator==(const Tensor &lhs, const Tensor &rhs);
Tensor operator==(const Tensor &lhs, const Scalar &rhs);
Tensor operator!=(const Tensor &lhs, const Tensor &rhs);
Tensor operator!=(const Tensor &lhs, const Scalar &rhs);
Tensor operator<(const Tensor &lhs, const Tensor &rhs);
Tensor operator<(const Tensor &lhs, const Scalar &rhs);
Tensor operator<=(const Tensor &lhs, const Tensor &rhs);
Tensor operator<=(const Tensor &lhs, const Scalar &rhs);
Tensor operator>=(const Tensor &lhs, const Tensor &rhs);
Tensor operator>=(const Tensor &lhs, const Scalar &rhs);
Tensor &operator+=(Tensor &lhs, const Scalar &rhs);
Tensor &operator-=(Tensor &lhs, const Scalar &rhs);
Tensor &operator*=(Tensor &lhs, const Scalar &rhs);
Tensor &operator/=(Tensor &lhs, const Scalar &rhs);
Tensor &operator+=(Tensor &lhs, const Tensor &rhs);
Tensor &operator-=(Tensor &lhs, const Tensor &rhs);
Tensor &operator*=(Tensor &lhs, const Tensor &rhs);
Tensor &operator/=(Tensor &lhs, const Tensor &rhs);

// mean(argmax(y, 1) == target) as a 0-dim tensor (src/utils/metrics.cpp:11-70)
Tensor accuracy(const Tensor &y, const Tensor &target);
}  // namespace origin
