// Operators over Mat. Gradients restate the reference's backward rules (cited per operator); softmax and
// softmax-cross-entropy go to the fused device kernels instead of the reference's chain of eight Mat ops.
#include "origin/functional.h"
#include "origin/nn.h"

#include <cmath>
#include <string>

namespace origin
{
namespace functional
{
namespace
{
Tensor scalar_like(const Scalar &s, const Tensor &ref)
{
    // a constant inside an operator's own arithmetic: a 0-dim tensor of the other operand's element type and device
    return Tensor(s, Shape({}), dtype(ref.dtype()).device(ref.device()));
}

// include/origin/mat/type_promotion.h:76-102: float64 > float32 > int64 > int32 > int8 > uint8
DataType promote_types(DataType a, DataType b)
{
    if (a == b)
        return a;
    for (DataType t : {DataType::kFloat64, DataType::kFloat32, DataType::kInt64, DataType::kInt32, DataType::kInt8,
                       DataType::kUInt8})
        if (a == t || b == t)
            return t;
    return a;
}

// both operands in the promoted type; an operand that already has it is passed through untouched
// (src/mat/type_promotion.cpp promote_tensors)
std::pair<Tensor, Tensor> promoted(const Tensor &a, const Tensor &b)
{
    if (a.dtype() == b.dtype())
        return {a, b};
    const DataType t = promote_types(a.dtype(), b.dtype());
    return {a.dtype() == t ? a : a.to(t), b.dtype() == t ? b : b.to(t)};
}

// gradient of a broadcasting binary op: reduce back to the operand's shape (left-aligned sum_to, as the reference)
Tensor fit(const Tensor &g, const Shape &shape)
{
    return g.shape() == shape ? g : sum_to(g, shape);
}

struct BinaryBase : Operator
{
    Shape s0, s1;
    void remember(const std::vector<Tensor> &xs, const char *name)
    {
        if (xs.size() != 2)
            THROW_RUNTIME_ERROR("{} operator requires exactly 2 inputs, but got {}", name, xs.size());
        s0 = xs[0].shape();
        s1 = xs[1].shape();
    }
};

struct Add : BinaryBase  // src/operators/math/add.cpp:12-55
{
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        remember(xs, "Add");
        auto [x0, x1] = promoted(xs[0], xs[1]);
        return {wrap(mat(x0) + mat(x1))};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        return {fit(gys[0], s0), fit(gys[0], s1)};
    }
};

struct Sub : BinaryBase  // src/operators/math/sub.cpp
{
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        remember(xs, "Sub");
        auto [x0, x1] = promoted(xs[0], xs[1]);
        return {wrap(mat(x0) - mat(x1))};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        return {fit(gys[0], s0), fit(wrap(-mat(gys[0])), s1)};
    }
};

struct Mul : BinaryBase  // src/operators/math/mul.cpp:12-53
{
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        remember(xs, "Mul");
        auto [x0, x1] = promoted(xs[0], xs[1]);
        return {wrap(mat(x0) * mat(x1))};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        const Mat &gy = mat(gys[0]);
        auto [x0, x1] = promoted(inputs_[0], inputs_[1]);  // the gradient has the promoted type (mul.cpp:36-44)
        return {fit(wrap(gy * mat(x1)), s0), fit(wrap(gy * mat(x0)), s1)};
    }
};

struct Div : BinaryBase  // src/operators/math/div.cpp:28-60
{
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        remember(xs, "Div");
        auto [x0, x1] = promoted(xs[0], xs[1]);
        return {wrap(mat(x0) / mat(x1))};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        auto [p0, p1] = promoted(inputs_[0], inputs_[1]);
        const Mat &gy = mat(gys[0]), &x0 = mat(p0), &x1 = mat(p1);
        auto gx0 = gy / x1;
        auto sq  = x1 * x1;
        auto gx1 = gy * x0;
        *gx1 /= *sq;
        gx1->neg_inplace();
        return {fit(wrap(std::move(gx0)), s0), fit(wrap(std::move(gx1)), s1)};
    }
};

struct Neg : Operator
{
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override { return {wrap(-mat(xs[0]))}; }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override { return {wrap(-mat(gys[0]))}; }
};

struct Pow : Operator  // src/operators/math/pow.cpp
{
    // the exponent arrives already in the result's type: float32 or float64 (pow.cpp:88-110; integers become float32)
    Scalar e;
    explicit Pow(const Scalar &s) : e(s) {}
    Tensor base(const Tensor &x) const { return x.dtype() == e.dtype() ? x : x.to(e.dtype()); }
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override { return {wrap(mat(base(xs[0])).pow(e))}; }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        const Tensor x = base(inputs_[0]);
        const Scalar minus_one = e.dtype() == DataType::kFloat64 ? Scalar(e.to_float64() - 1.0) : Scalar(e.to_float32() - 1.0f);
        auto tmp = mat(x).pow(minus_one);
        tmp->mul_inplace(mat(gys[0]));
        tmp->mul_inplace(mat(scalar_like(e, x)));
        return {wrap(std::move(tmp))};
    }
};

struct Exp : Operator
{
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override { return {wrap(mat(xs[0]).exp())}; }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        auto y = mat(inputs_[0]).exp();
        return {wrap(mat(gys[0]) * *y)};
    }
};

struct Log : Operator
{
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override { return {wrap(mat(xs[0]).log())}; }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        return {wrap(mat(gys[0]) / mat(inputs_[0]))};
    }
};

struct Square : Operator
{
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override { return {wrap(mat(xs[0]).square())}; }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        auto two_x = mat(inputs_[0]) * mat(scalar_like(Scalar(2.0f), inputs_[0]));
        return {wrap(mat(gys[0]) * *two_x)};
    }
};

struct Sum : Operator  // src/operators/math/sum.cpp: backward = broadcast_to(gy, x.shape)
{
    int axis;
    bool keepdim;
    Sum(int a, bool k) : axis(a), keepdim(k) {}
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override { return {wrap(mat(xs[0]).sum(axis, keepdim))}; }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        const Shape xs = inputs_[0].shape();
        if (axis >= 0 && !keepdim && xs.size() > 1)
        {
            // put the reduced dim back as size 1 so that the right-aligned broadcast lands on the right axis
            std::vector<size_t> d = xs.dims();
            d[axis] = 1;
            return {wrap(mat(gys[0]).reshape(Shape(d))->broadcast_to(xs))};
        }
        return {wrap(mat(gys[0]).broadcast_to(xs))};
    }
};

struct SumTo : Operator  // src/operators/math/sum_to.cpp
{
    Shape shape;
    explicit SumTo(const Shape &s) : shape(s) {}
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override { return {wrap(mat(xs[0]).sum_to(shape))}; }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        return {wrap(mat(gys[0]).broadcast_to(inputs_[0].shape()))};
    }
};

struct BroadcastTo : Operator  // src/operators/math/broadcast_to.cpp:10-46: backward = sum_to(gy, x.shape)
{
    Shape shape, x_shape;
    explicit BroadcastTo(const Shape &s) : shape(s) {}
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        x_shape = xs[0].shape();
        return {wrap(mat(xs[0]).broadcast_to(shape))};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        return {wrap(mat(gys[0]).sum_to(x_shape))};
    }
};

struct MatMul : Operator  // src/operators/math/mat_mul.cpp:12-182
{
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        if (xs.size() != 2)
            THROW_RUNTIME_ERROR("MatMul operator requires exactly 2 inputs, but got {}", xs.size());
        auto [x0, x1] = promoted(xs[0], xs[1]);  // mat_mul.cpp promotes too; the product itself is a float32 kernel
        return {wrap(mat(x0).matmul(mat(x1)))};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        // gx = gy . w^T, gw = x^T . gy. The reference copies both transposes first (mat_mul.cpp:171-174); for 2-D
        // operands this backend's GEMM reads w and x in place instead — the same products, two copies fewer.
        const Mat &x = mat(inputs_[0]), &w = mat(inputs_[1]), &gy = mat(gys[0]);
        if (x.shape().size() == 2 && w.shape().size() == 2 && gy.shape().size() == 2)
        {
            auto g = OriginMat::matmul_backward_2d(x, w, gy);
            return {wrap(std::move(g.first)), wrap(std::move(g.second))};
        }
        auto wT = w.transpose();
        auto xT = x.transpose();
        return {wrap(gy.matmul(*wT)), wrap(xT->matmul(gy))};
    }
};

struct Reshape : Operator
{
    Shape shape;
    explicit Reshape(const Shape &s) : shape(s) {}
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override { return {wrap(mat(xs[0]).reshape(shape))}; }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        return {wrap(mat(gys[0]).reshape(inputs_[0].shape()))};
    }
};

struct Transpose : Operator
{
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override { return {wrap(mat(xs[0]).transpose())}; }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override { return {wrap(mat(gys[0]).transpose())}; }
};

// src/operators/activation/relu.cpp:13-54: mask = x > 0, gx = gy * mask. The mask is not kept: backward forms it from
// the input again inside the one kernel that also multiplies (same 0/1 factor, same product).
struct ReLU : Operator
{
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override { return {wrap(mat(xs[0]).relu())}; }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        return {wrap(omat(gys[0]).relu_backward(mat(inputs_[0])))};
    }
};

// Linear::forward's matmul + broadcast_to + add (src/nn/layers/linear.cpp:88-104) as one operator for 2-D inputs:
// the bias is added in the product's epilogue, and backward is the three gradients those operators would produce
// (gx = gy.W^T, gW = x^T.gy, gb = gy summed to the bias's shape).
struct FusedLinear : Operator
{
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        return {wrap(omat(xs[0]).linear(mat(xs[1]), mat(xs[2])))};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        auto g = OriginMat::linear_backward_2d(mat(inputs_[0]), mat(inputs_[1]), mat(gys[0]), inputs_[2].shape());
        return {wrap(std::move(g[0])), wrap(std::move(g[1])), wrap(std::move(g[2]))};
    }
};

// A layer followed by ReLU as one operator (Sequential pairs them up): the activation runs in the layer's epilogue, so the
// pre-activation tensor is never written, and backward first masks the incoming gradient with (y > 0) — the same
// elements as the (x > 0) of ReLU's own backward (src/operators/activation/relu.cpp), since y = max(x, 0) — and then
// does what the layer's backward does. The values are those of the two operators run one after the other.
struct FusedLinearRelu : Operator
{
    std::shared_ptr<Mat> y;  // the output's data (not its tensor: that would own this operator in turn)
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        Tensor out = wrap(omat(xs[0]).linear_act(mat(xs[1]), mat(xs[2]), 0));
        y = out.impl_->data_;
        return {out};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        auto g0 = omat(gys[0]).relu_backward(*y);
        auto g  = OriginMat::linear_backward_2d(mat(inputs_[0]), mat(inputs_[1]), *g0, inputs_[2].shape());
        return {wrap(std::move(g[0])), wrap(std::move(g[1])), wrap(std::move(g[2]))};
    }
};

// src/operators/activation/leaky_relu.cpp:17-72. Forward from the operations at hand, exact in both branches:
// r = relu(x); y = r + alpha*(x - r) — where x > 0 that is x + alpha*0, elsewhere 0 + alpha*x. Backward as there:
// gy * (alpha + mask*(1-alpha)) with mask = (x > 0).
struct LeakyReLU : Operator
{
    float alpha;
    explicit LeakyReLU(float a) : alpha(a) {}
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        if (xs.size() != 1)
            THROW_RUNTIME_ERROR("LeakyReLU operator requires exactly 1 input, but got {}", xs.size());
        const Mat &x = mat(xs[0]);
        auto r       = x.relu();
        auto rest    = x - *r;
        auto scaled  = *rest * mat(scalar_like(Scalar(alpha), xs[0]));
        return {wrap(*r + *scaled)};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        if (gys.size() != 1)
            THROW_RUNTIME_ERROR("LeakyReLU backward requires exactly 1 gradient, but got {}", gys.size());
        const Tensor &x = inputs_[0];
        auto mask   = mat(x) > mat(scalar_like(Scalar(0.0f), x));
        auto scaled = *mask * mat(scalar_like(Scalar(1.0f - alpha), x));
        auto slope  = *scaled + mat(scalar_like(Scalar(alpha), x));
        return {wrap(mat(gys[0]) * *slope)};
    }
};

struct Softmax : Operator  // src/operators/activation/softmax.cpp:14-129
{
    int axis;
    explicit Softmax(int a) : axis(a) {}
    int resolved(const Tensor &x) const
    {
        const int nd = (int)x.shape().size();
        const int a  = axis < 0 ? nd + axis : axis;
        if (a < 0 || a >= nd)
            THROW_INVALID_ARG("Invalid axis {} for softmax. Tensor has {} dimensions", axis, nd);
        return a;
    }
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        return {wrap(omat(xs[0]).softmax(resolved(xs[0])))};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        // gx = y * (gy - sum(gy * y, axis))
        const Tensor &x = inputs_[0];
        const int a     = resolved(x);
        auto y   = omat(x).softmax(a);
        auto gyy = mat(gys[0]) * *y;
        std::vector<size_t> d = x.shape().dims();
        d[a] = 1;
        auto s    = gyy->sum(a, false)->reshape(Shape(d))->broadcast_to(x.shape());
        auto diff = mat(gys[0]) - *s;
        return {wrap(*y * *diff)};
    }
};

struct SoftmaxCrossEntropy : Operator  // src/operators/loss/softmax_cross_entropy.cpp:17-111
{
    static bool bad_label(const Tensor &loss) { return omat(loss).loss_bad_label_flag(); }
    // the gradient for an upstream gradient of 1, when the loss's launch wrote it along (small batches of few classes):
    // backward() starts from that constant, and then has nothing to launch here
    std::unique_ptr<Mat> unit_grad;
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        if (xs.size() != 2)
            THROW_RUNTIME_ERROR("SoftmaxCrossEntropy operator requires exactly 2 inputs (x and target), but got {}",
                                xs.size());
        const Tensor &x = xs[0], &t = xs[1];
        if (x.shape().size() != 2)
            THROW_INVALID_ARG("SoftmaxCrossEntropy expects x to be 2D (N, C), but got shape {}", x.shape().to_string());
        if (t.shape().size() != 1)
            THROW_INVALID_ARG("SoftmaxCrossEntropy expects target to be 1D (N,), but got shape {}",
                              t.shape().to_string());
        if (x.shape()[0] != t.shape()[0])
            THROW_INVALID_ARG("SoftmaxCrossEntropy: batch size mismatch. x has {} samples, target has {} samples",
                              x.shape()[0], t.shape()[0]);
        unit_grad.reset();
        std::unique_ptr<Mat> *want = x.requires_grad() ? &unit_grad : nullptr;
        if (cuda::is_capturing())  // a recorded step cannot visit the host: the loss stays where it is computed
            return {wrap(omat(x).softmax_cross_entropy_device(mat(t), want))};
        // synchronises once, as the reference's .item() does, to report an out-of-range label; the loss is not sent
        // back up afterwards: it is the device scalar the kernel wrote
        return {wrap(omat(x).softmax_cross_entropy_checked(mat(t), want))};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        const Tensor &x = inputs_[0], &t = inputs_[1];
        std::unique_ptr<Mat> gx;
        // the upstream gradient is read where it lies when it is a float32 device scalar (no host round trip; gy/N
        // is formed in the kernel as the host would form it)
        float seed = 0.f;
        if (gys[0].elements() == 1 && omat(gys[0]).unwritten_constant(&seed) && seed == 1.0f && unit_grad)
            gx = std::move(unit_grad);  // written by the loss's own launch
        else if (gys[0].elements() == 1 && omat(gys[0]).unwritten_constant(&seed))
            gx = omat(x).softmax_cross_entropy_backward(mat(t), seed);  // the ones backward() starts from: no read at all
        else if (cuda::is_capturing() || (OriginMat::device_f32(mat(gys[0])) && gys[0].elements() == 1))
            gx = omat(x).softmax_cross_entropy_backward_device(mat(t), mat(gys[0]));
        else
            gx = omat(x).softmax_cross_entropy_backward(mat(t), gys[0].item<float>());
        auto gt = Tensor::zeros(t.shape(), dtype(DataType::kFloat32).device(t.device()));
        return {wrap(std::move(gx)), gt};
    }
};

struct Conv2dOp : Operator  // src/operators/conv/conv2d.cpp:14-89
{
    std::pair<int, int> stride, pad;
    Conv2dOp(std::pair<int, int> s, std::pair<int, int> p) : stride(s), pad(p) {}
    static void validate(const std::vector<Tensor> &xs)
    {
        if (xs.size() < 2 || xs.size() > 3)
            THROW_RUNTIME_ERROR("Conv2d operator requires 2 or 3 inputs (x, W, [b]), but got {}", xs.size());
        if (xs[0].shape().size() != 4)
            THROW_RUNTIME_ERROR("Conv2d forward: x must be 4D (N, C, H, W), but got shape {}", xs[0].shape().to_string());
        if (xs[1].shape().size() != 4)
            THROW_RUNTIME_ERROR("Conv2d forward: W must be 4D (OC, C, KH, KW), but got shape {}",
                                xs[1].shape().to_string());
        if (xs[0].shape()[1] != xs[1].shape()[1])
            THROW_RUNTIME_ERROR("Conv2d forward: channel mismatch - x has {} channels, but W expects {} channels",
                                xs[0].shape()[1], xs[1].shape()[1]);
    }
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        validate(xs);
        const Mat *b = xs.size() == 3 ? &mat(xs[2]) : nullptr;
        return {wrap(mat(xs[0]).conv2d(mat(xs[1]), b, stride, pad))};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        const Mat &gy = mat(gys[0]);
        const Mat *b  = inputs_.size() == 3 ? &mat(inputs_[2]) : nullptr;
        auto grads    = gy.conv2d_backward(gy, mat(inputs_[0]), mat(inputs_[1]), b, stride, pad);
        std::vector<Tensor> out;
        for (auto &g : grads)
            out.push_back(wrap(std::move(g)));
        return out;
    }
};

// Conv2d followed by ReLU as one operator, as FusedLinearRelu above
struct Conv2dReluOp : Conv2dOp
{
    std::shared_ptr<Mat> y;
    using Conv2dOp::Conv2dOp;
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        validate(xs);
        const Mat *b = xs.size() == 3 ? &mat(xs[2]) : nullptr;
        Tensor out   = wrap(omat(xs[0]).conv2d_act(mat(xs[1]), b, stride, pad, 0));
        y            = out.impl_->data_;
        return {out};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        auto g0 = omat(gys[0]).relu_backward(*y);
        const Mat *b  = inputs_.size() == 3 ? &mat(inputs_[2]) : nullptr;
        auto grads    = g0->conv2d_backward(*g0, mat(inputs_[0]), mat(inputs_[1]), b, stride, pad);
        std::vector<Tensor> out;
        for (auto &g : grads)
            out.push_back(wrap(std::move(g)));
        return out;
    }
};

struct MaxPool2d : Operator  // src/operators/pooling/max_pool2d.cpp:14-86
{
    std::pair<int, int> k, s, p;
    std::shared_ptr<Storage> indices;  // window-local argmax per output, uint64, kept on the device
    MaxPool2d(std::pair<int, int> kk, std::pair<int, int> ss, std::pair<int, int> pp) : k(kk), s(ss), p(pp) {}
    static const OriginMat &origin(const Mat &m)
    {
        const auto *o = dynamic_cast<const OriginMat *>(&m);
        if (!o)
            THROW_RUNTIME_ERROR("MaxPool2d: expected an OriginMat, got backend_type={}", m.backend_type());
        return *o;
    }
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        return {wrap(origin(mat(xs[0])).max_pool2d_device(k, s, p, xs[0].requires_grad() ? &indices : nullptr))};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        if (!indices)
            THROW_RUNTIME_ERROR("MaxPool2d backward: indices not found. This should not happen when requires_grad=true");
        return {wrap(origin(mat(inputs_[0])).max_pool2d_backward_device(mat(gys[0]), k, s, p, *indices))};
    }
};

// Conv2d -> ReLU -> MaxPool2d as one operator (the two tensors in between are not visible from outside): the activation
// in the convolution's epilogue, and in backward the pooling gradient masked by the ReLU as it is written. The values are
// those of the three operators run in turn (src/operators/conv/conv2d.cpp, activation/relu.cpp, pooling/max_pool2d.cpp).
struct Conv2dReluPoolOp : Conv2dOp
{
    std::pair<int, int> pk, ps, pp;
    std::shared_ptr<Mat> y;            // relu(conv(x)), the tensor that is pooled — or null after the one-pass forward
    std::shared_ptr<Mat> pooled;       // then the output's data instead (not its tensor: that would own this operator)
    Shape conv_shape;                  // and the shape relu(conv(x)) would have had
    std::shared_ptr<Storage> indices;  // window-local argmax per output, uint64, kept on the device
    Conv2dReluPoolOp(std::pair<int, int> st, std::pair<int, int> pd, std::pair<int, int> k, std::pair<int, int> s,
                     std::pair<int, int> p)
        : Conv2dOp(st, pd), pk(k), ps(s), pp(p)
    {}
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        validate(xs);
        const Mat *b = xs.size() == 3 ? &mat(xs[2]) : nullptr;
        if (OriginMat::conv_relu_pool_fused(mat(xs[0]), mat(xs[1]), stride, pad, pk, ps, pp))
        {
            // a first layer under a 2x2 pooling: one pass, relu(conv(x)) is never written
            const Shape xs0 = xs[0].shape();
            conv_shape      = Shape{xs0[0], mat(xs[1]).shape()[0], xs0[2], xs0[3]};
            Tensor out      = wrap(omat(xs[0]).conv2d_relu_max_pool2d_device(mat(xs[1]), b, stride, pad, pk, ps, pp, &indices));
            pooled          = out.impl_->data_;
            y.reset();
            return {out};
        }
        pooled.reset();
        y            = std::shared_ptr<Mat>(omat(xs[0]).conv2d_act(mat(xs[1]), b, stride, pad, 0));
        const auto *yo = dynamic_cast<const OriginMat *>(y.get());
        // windows that tile the image (2x2/2, 3x3/3, no padding): the backward's mask can come from the pooled tensor, a
        // quarter or a ninth of the reads, relu(conv(x)) need not be kept until then, and the indices — which never leave
        // this operator — are kept as bytes
        const Shape ys = y->shape();
        const bool tiles = y->dtype() == DataType::kFloat32 && pk.first == pk.second && (pk.first == 2 || pk.first == 3) &&
                           ps == pk && pp.first == 0 && pp.second == 0 && ys[2] % pk.first == 0 && ys[3] % pk.second == 0 &&
                           ys[2] > 0 && ys[3] > 0 && ys.elements() < (size_t(1) << 31) - 256;
        if (tiles)
        {
            Tensor out = wrap(yo->max_pool2d_device_compact(pk, ps, pp, &indices));
            conv_shape = ys;
            pooled     = out.impl_->data_;
            y.reset();
            return {out};
        }
        return {wrap(yo->max_pool2d_device(pk, ps, pp, &indices))};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        std::unique_ptr<Mat> g0;
        if (y)
            g0 = dynamic_cast<const OriginMat *>(y.get())->max_pool2d_backward_relu_device(mat(gys[0]), pk, ps, pp, *indices);
        else
            g0 = dynamic_cast<const OriginMat *>(pooled.get())
                     ->max_pool2d_backward_relu_pooled_device(mat(gys[0]), conv_shape, pk, ps, pp, *indices);
        const Mat *b   = inputs_.size() == 3 ? &mat(inputs_[2]) : nullptr;
        auto grads     = g0->conv2d_backward(*g0, mat(inputs_[0]), mat(inputs_[1]), b, stride, pad);
        std::vector<Tensor> out;
        for (auto &g : grads)
            out.push_back(wrap(std::move(g)));
        return out;
    }
};

struct Sigmoid : Operator  // src/operators/activation/sigmoid.cpp:13-44: keeps y, gx = gy*y*(1-y)
{
    Tensor y;
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        y = wrap(mat(xs[0]).sigmoid());
        return {y};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        return {wrap(mat(gys[0]).sigmoid_backward(mat(y)))};
    }
};

struct SiLU : Operator  // src/operators/activation/silu.cpp: gx = gy*(s + x*s*(1-s))
{
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override { return {wrap(mat(xs[0]).silu())}; }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        return {wrap(mat(gys[0]).silu_backward(mat(inputs_[0])))};
    }
};

struct Cat : Operator  // src/operators/shape/cat.cpp: backward splits the gradient back along dim
{
    int dim;
    std::vector<size_t> sizes;
    explicit Cat(int d) : dim(d) {}
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        if (xs.empty())
            THROW_RUNTIME_ERROR("cat: requires at least 1 input");
        std::vector<const Mat *> others;
        sizes.clear();
        for (size_t i = 0; i < xs.size(); ++i)
        {
            if (dim < 0 || (size_t)dim >= xs[i].shape().size())
                THROW_RUNTIME_ERROR("cat: dimension {} out of range for shape {}", dim, xs[i].shape().to_string());
            sizes.push_back(xs[i].shape()[dim]);
            if (i)
                others.push_back(&mat(xs[i]));
        }
        return {wrap(mat(xs[0]).cat(others, dim))};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        std::vector<Tensor> out;
        for (auto &piece : mat(gys[0]).split(sizes, dim))
            out.push_back(wrap(std::move(piece)));
        return out;
    }
};

struct Upsample : Operator  // src/operators/nn/upsample.cpp:13-90
{
    std::string mode;
    std::pair<float, float> scale;
    std::pair<int, int> size;
    int sh = 1, sw = 1;
    Upsample(const std::string &m, std::pair<float, float> sc, std::pair<int, int> sz) : mode(m), scale(sc), size(sz) {}
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        const Shape s = xs[0].shape();
        if (s.size() != 4)
            THROW_RUNTIME_ERROR("Upsample forward: x must be 4D (N, C, H, W), but got shape {}", s.to_string());
        size_t OH, OW;
        if (size.first > 0 && size.second > 0)
            OH = (size_t)size.first, OW = (size_t)size.second;
        else
            OH = (size_t)std::lround(s[2] * scale.first), OW = (size_t)std::lround(s[3] * scale.second);
        sh = (int)(OH / s[2]), sw = (int)(OW / s[3]);
        return {wrap(mat(xs[0]).upsample(Shape{s[0], s[1], OH, OW}, sh, sw, mode))};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        return {wrap(mat(inputs_[0]).upsample_backward(mat(gys[0]), inputs_[0].shape(), sh, sw, mode))};
    }
};

struct BatchNorm : Operator  // src/operators/normalization/batch_norm.cpp:16-122
{
    bool training;
    float eps, momentum;
    int num_dims;
    bool relu;  // the output passes through a ReLU before leaving (the layer pair BatchNorm, ReLU folded into one)
    Tensor saved_mean, saved_var;  // x_norm is not kept: backward forms it again from x and these two (same floats)
    BatchNorm(bool t, float e, float m, int nd, bool r = false) : training(t), eps(e), momentum(m), num_dims(nd), relu(r) {}
    std::vector<Tensor> forward(const std::vector<Tensor> &xs) override
    {
        if (xs.size() != 5)
            THROW_RUNTIME_ERROR("BatchNorm operator requires exactly 5 inputs (x, gamma, beta, running_mean, "
                                "running_var), but got {}", xs.size());
        Tensor y;
        if (relu || training || xs[0].requires_grad() || xs[1].requires_grad() || xs[2].requires_grad())
        {
            // in training mode the layers read the batch statistics off the operator's outputs even without a graph
            auto r = omat(xs[0]).batch_norm_forward_no_xnorm(mat(xs[1]), mat(xs[2]), mat(xs[3]), mat(xs[4]), training, eps,
                                                             num_dims, relu);
            y = wrap(std::move(r.y));
            saved_mean = wrap(std::move(r.mean)), saved_var = wrap(std::move(r.var));
        }
        else
            y = wrap(mat(xs[0]).batch_norm(mat(xs[1]), mat(xs[2]), mat(xs[3]), mat(xs[4]), training, eps, momentum, num_dims));
        if (training)
            return {y, saved_mean, saved_var};
        return {y};
    }
    std::vector<Tensor> backward(const std::vector<Tensor> &gys) override
    {
        // the gradient of y only: the statistics outputs feed the running averages, outside the graph
        auto r = omat(inputs_[0]).batch_norm_backward_from_x(mat(gys[0]), mat(inputs_[1]), mat(saved_mean), mat(saved_var),
                                                             eps, num_dims, relu ? &mat(inputs_[2]) : nullptr);
        const auto opt = dtype(DataType::kFloat32).device(inputs_[0].device());
        return {wrap(std::move(r[0])), wrap(std::move(r[1])), wrap(std::move(r[2])), Tensor::zeros(inputs_[3].shape(), opt),
                Tensor::zeros(inputs_[4].shape(), opt)};
    }
};

template <typename Op, typename... A>
Tensor apply(const std::vector<Tensor> &xs, A &&...args)
{
    auto op = std::make_shared<Op>(std::forward<A>(args)...);
    return (*op)(xs)[0];
}
}  // namespace

// ---- Split (src/operators/shape/split.cpp:14-128)
std::vector<Tensor> Split::forward(const std::vector<Tensor> &xs)
{
    if (xs.size() != 1)
        THROW_RUNTIME_ERROR("Split operator requires exactly 1 input, but got {}", xs.size());
    const Shape shape = xs[0].shape();
    if (dim_ < 0 || (size_t)dim_ >= shape.size())
        THROW_INVALID_ARG("Split: dim {} is out of range for input shape {}", dim_, shape.to_string());
    const size_t extent = shape[dim_];
    std::vector<size_t> sizes;
    if (split_sizes_.size() == 1 && split_sizes_[0] > 0)
    {
        // equal pieces, the last one takes what is left
        const size_t piece = split_sizes_[0], count = (extent + piece - 1) / piece;
        for (size_t i = 0; i < count; ++i)
            sizes.push_back(i + 1 < count ? piece : extent - (count - 1) * piece);
    }
    else
    {
        sizes = split_sizes_;
        size_t total = 0;
        for (size_t s : sizes)
            total += s;
        if (total != extent)
            THROW_INVALID_ARG("Split: sum of split_sizes {} does not match dimension size {} at dim {}", total, extent, dim_);
    }
    std::vector<Tensor> out;
    for (auto &piece : mat(xs[0]).split(sizes, dim_))
        out.push_back(wrap(std::move(piece)));
    return out;
}

std::vector<Tensor> Split::backward(const std::vector<Tensor> &gys)
{
    if (gys.empty())
        THROW_RUNTIME_ERROR("Split backward requires at least 1 gradient, but got 0");
    if (gys.size() == 1)
        return gys;
    const Shape first = gys[0].shape();
    std::vector<const Mat *> others;
    for (size_t i = 1; i < gys.size(); ++i)
    {
        const Shape s = gys[i].shape();
        if (s.size() != first.size())
            THROW_RUNTIME_ERROR("Split backward: all gradients must have same number of dimensions");
        for (size_t d = 0; d < s.size(); ++d)
            if (d != (size_t)dim_ && s[d] != first[d])
                THROW_RUNTIME_ERROR("Split backward: dimension {} mismatch: {} vs {}", d, s[d], first[d]);
        if (gys[i].device() != gys[0].device())
            THROW_RUNTIME_ERROR("Split backward: device mismatch at gradient {}, expected {}, got {}", i,
                                gys[0].device().to_string(), gys[i].device().to_string());
        others.push_back(&mat(gys[i]));
    }
    return {wrap(mat(gys[0]).cat(others, dim_))};
}

std::vector<Tensor> split(const Tensor &x, SizeArrayRef split_sizes, int dim)
{
    auto op = std::make_shared<Split>(split_sizes, dim);
    return (*op)(std::vector<Tensor>{x});
}

std::vector<Tensor> split(const Tensor &x, size_t split_size, int dim)
{
    auto op = std::make_shared<Split>(split_size, dim);
    return (*op)(std::vector<Tensor>{x});
}

// ---- LinearOp (src/operators/custom/linear.cpp:12-110)
std::vector<Tensor> LinearOp::forward(const std::vector<Tensor> &xs)
{
    const size_t expected = use_bias_ ? 3 : 2;
    if (xs.size() != expected)
        THROW_RUNTIME_ERROR("Linear operator requires {} inputs (x, weight{}), but got {}", expected,
                            use_bias_ ? ", bias" : "", xs.size());
    const Shape xs0 = xs[0].shape(), ws = xs[1].shape();
    std::unique_ptr<Mat> flat;  // [batch, everything else]
    const Mat *x2 = &mat(xs[0]);
    if (xs0.size() > 2)
    {
        size_t features = 1;
        for (size_t i = 1; i < xs0.size(); ++i)
            features *= xs0[i];
        flat = x2->reshape(Shape{xs0[0], features});
        x2   = flat.get();
    }
    if (x2->shape().size() != 2)
        THROW_RUNTIME_ERROR("Linear forward: x must be 2D after flattening, but got shape {}", x2->shape().to_string());
    if (ws.size() != 2)
        THROW_RUNTIME_ERROR("Linear forward: weight must be 2D (out_features, in_features), but got shape {}", ws.to_string());
    if (x2->shape()[1] != ws[1])
        THROW_RUNTIME_ERROR("Linear forward: feature mismatch - x has {} features, but weight expects {} features",
                            x2->shape()[1], ws[1]);
    if (ws[0] != (size_t)out_features_)
        THROW_RUNTIME_ERROR("Linear forward: output feature mismatch - weight has {} out_features, but expected {}", ws[0],
                            out_features_);
    auto wt = mat(xs[1]).transpose();
    auto y  = x2->matmul(*wt);
    if (use_bias_)
    {
        auto b = mat(xs[2]).broadcast_to(y->shape());
        y      = *y + *b;
    }
    return {wrap(std::move(y))};
}

std::vector<Tensor> LinearOp::backward(const std::vector<Tensor> &)
{
    THROW_RUNTIME_ERROR("LinearOp backward is not implemented");
}

Tensor custom_linear(const Tensor &x, const Tensor &weight, const Tensor &bias, int in_features, int out_features, bool use_bias)
{
    auto op = std::make_shared<LinearOp>(in_features, out_features, use_bias);
    return use_bias ? (*op)(std::vector<Tensor>{x, weight, bias})[0] : (*op)(std::vector<Tensor>{x, weight})[0];
}

Tensor custom_linear(const Tensor &x, const Tensor &weight, int in_features, int out_features)
{
    return custom_linear(x, weight, Tensor(), in_features, out_features, false);
}

Tensor leaky_relu(const Tensor &x, float alpha) { return apply<LeakyReLU>({x}, alpha); }

Tensor add(const Tensor &a, const Tensor &b) { return apply<Add>({a, b}); }
Tensor sub(const Tensor &a, const Tensor &b) { return apply<Sub>({a, b}); }
Tensor mul(const Tensor &a, const Tensor &b) { return apply<Mul>({a, b}); }
Tensor div(const Tensor &a, const Tensor &b) { return apply<Div>({a, b}); }
Tensor neg(const Tensor &x) { return apply<Neg>({x}); }
Tensor pow(const Tensor &x, const Scalar &e)
{
    // src/operators/math/pow.cpp:88-110: base and exponent promote as two operands would, and a result that would be an
    // integer type becomes float32; the exponent is stored in that type
    DataType t = promote_types(x.dtype(), e.dtype());
    if (t != DataType::kFloat32 && t != DataType::kFloat64)
        t = DataType::kFloat32;
    return apply<Pow>({x}, t == DataType::kFloat64 ? Scalar(e.to_float64()) : Scalar(e.to_float32()));
}
Tensor exp(const Tensor &x) { return apply<Exp>({x}); }
Tensor log(const Tensor &x) { return apply<Log>({x}); }
Tensor square(const Tensor &x) { return apply<Square>({x}); }
Tensor sum(const Tensor &x, int axis, bool keepdim) { return apply<Sum>({x}, axis, keepdim); }
Tensor sum_to(const Tensor &x, const Shape &s) { return apply<SumTo>({x}, s); }
Tensor broadcast_to(const Tensor &x, const Shape &s) { return apply<BroadcastTo>({x}, s); }
Tensor mat_mul(const Tensor &x, const Tensor &w) { return apply<MatMul>({x, w}); }
Tensor reshape(const Tensor &x, const Shape &s) { return apply<Reshape>({x}, s); }
Tensor transpose(const Tensor &x) { return apply<Transpose>({x}); }
Tensor relu(const Tensor &x) { return apply<ReLU>({x}); }
Tensor sigmoid(const Tensor &x) { return apply<Sigmoid>({x}); }
Tensor silu(const Tensor &x) { return apply<SiLU>({x}); }
Tensor cat(const std::vector<Tensor> &xs, int dim) { return apply<Cat>(xs, dim); }
Tensor upsample(const Tensor &x, const std::string &mode, std::pair<float, float> scale_factor)
{
    return apply<Upsample>({x}, mode, scale_factor, std::make_pair(0, 0));
}

// in-place forms: the left operand's storage is overwritten (src/operators/math/add.cpp:57-100 and its siblings)
namespace
{
Mat &writable(Tensor &t) { return *t.impl_->data_; }
}  // namespace
void add_(Tensor &a, const Tensor &b) { writable(a).add_inplace(*b.impl_->data_); }
void sub_(Tensor &a, const Tensor &b) { writable(a).sub_inplace(*b.impl_->data_); }
void mul_(Tensor &a, const Tensor &b) { writable(a).mul_inplace(*b.impl_->data_); }
void div_(Tensor &a, const Tensor &b) { writable(a).div_inplace(*b.impl_->data_); }
void neg_(Tensor &x) { writable(x).neg_inplace(); }
void exp_(Tensor &x) { writable(x).exp_inplace(); }
void log_(Tensor &x) { writable(x).log_inplace(); }
void square_(Tensor &x) { writable(x).square_inplace(); }
void relu_(Tensor &x) { writable(x).relu_inplace(); }
std::vector<Tensor> batch_norm_relu_outputs(const Tensor &x, const Tensor &gamma, const Tensor &beta, const Tensor &rm,
                                            const Tensor &rv, bool training, float eps, float momentum, int num_dims)
{
    auto op = std::make_shared<BatchNorm>(training, eps, momentum, num_dims, true);
    return (*op)({x, gamma, beta, rm, rv});
}

std::vector<Tensor> batch_norm_outputs(const Tensor &x, const Tensor &gamma, const Tensor &beta, const Tensor &rm,
                                       const Tensor &rv, bool training, float eps, float momentum, int num_dims)
{
    auto op = std::make_shared<BatchNorm>(training, eps, momentum, num_dims);
    return (*op)({x, gamma, beta, rm, rv});
}
Tensor batch_norm(const Tensor &x, const Tensor &gamma, const Tensor &beta, const Tensor &rm, const Tensor &rv,
                  bool training, float eps, float momentum, int num_dims)
{
    return batch_norm_outputs(x, gamma, beta, rm, rv, training, eps, momentum, num_dims)[0];
}
Tensor linear(const Tensor &x, const Tensor &w, const Tensor &b) { return apply<FusedLinear>({x, w, b}); }
Tensor linear_relu(const Tensor &x, const Tensor &w, const Tensor &b) { return apply<FusedLinearRelu>({x, w, b}); }
Tensor conv2d_relu(const Tensor &x, const Tensor &W, const Tensor *b, std::pair<int, int> stride, std::pair<int, int> pad)
{
    std::vector<Tensor> in{x, W};
    if (b)
        in.push_back(*b);
    return apply<Conv2dReluOp>(in, stride, pad);
}
Tensor conv2d_relu_max_pool2d(const Tensor &x, const Tensor &W, const Tensor *b, std::pair<int, int> stride,
                              std::pair<int, int> pad, std::pair<int, int> pool_kernel, std::pair<int, int> pool_stride,
                              std::pair<int, int> pool_pad)
{
    std::vector<Tensor> in{x, W};
    if (b)
        in.push_back(*b);
    return apply<Conv2dReluPoolOp>(in, stride, pad, pool_kernel, pool_stride, pool_pad);
}
Tensor softmax(const Tensor &x, int axis) { return apply<Softmax>({x}, axis); }
Tensor softmax_cross_entropy(const Tensor &x, const Tensor &t) { return apply<SoftmaxCrossEntropy>({x, t}); }
bool softmax_cross_entropy_bad_label(const Tensor &loss) { return SoftmaxCrossEntropy::bad_label(loss); }

Tensor flatten(const Tensor &x, int start_dim, int end_dim)  // src/operators/shape/flatten.cpp
{
    const std::vector<size_t> d = x.shape().dims();
    const int nd = (int)d.size();
    const int s = start_dim < 0 ? nd + start_dim : start_dim, e = end_dim < 0 ? nd + end_dim : end_dim;
    if (s < 0 || s >= nd || e < 0 || e >= nd || s > e)
        THROW_INVALID_ARG("Flatten: invalid dims - start_dim={}, end_dim={}, shape={}", start_dim, end_dim,
                          x.shape().to_string());
    std::vector<size_t> out(d.begin(), d.begin() + s);
    size_t flat = 1;
    for (int i = s; i <= e; ++i)
        flat *= d[i];
    out.push_back(flat);
    out.insert(out.end(), d.begin() + e + 1, d.end());
    return reshape(x, Shape(out));
}

Tensor conv2d(const Tensor &x, const Tensor &W, const Tensor *b, std::pair<int, int> stride, std::pair<int, int> pad)
{
    std::vector<Tensor> in{x, W};
    if (b)
        in.push_back(*b);
    return apply<Conv2dOp>(in, stride, pad);
}
Tensor conv2d(const Tensor &x, const Tensor &W, const Tensor *b, int stride, int pad)
{
    return conv2d(x, W, b, pair(stride), pair(pad));
}
Tensor max_pool2d(const Tensor &x, std::pair<int, int> k, std::pair<int, int> s, std::pair<int, int> p)
{
    if (s.first == 0 && s.second == 0)
        s = k;  // stride defaults to the kernel size
    return apply<MaxPool2d>({x}, k, s, p);
}
Tensor max_pool2d(const Tensor &x, int k, int s, int p)
{
    return max_pool2d(x, pair(k), pair(s), pair(p));
}
}  // namespace functional

namespace F = functional;
namespace
{
// a Scalar operand of an arithmetic operator: a 0-dim tensor of the scalar's own element type on the other operand's
// device; the operator then promotes the two (src/operators/math/add.cpp:110-114)
Tensor scalar_of(const Scalar &s, const Tensor &ref)
{
    return Tensor(s, Shape({}), dtype(s.dtype()).device(ref.device()));
}
// in a comparison or a compound assignment the tensor's type stands: the scalar is brought to it
Tensor scalar_as(const Scalar &s, const Tensor &ref)
{
    return Tensor(s, Shape({}), dtype(ref.dtype()).device(ref.device()));
}
}  // namespace

Tensor operator+(const Tensor &a, const Tensor &b) { return F::add(a, b); }
Tensor operator+(const Tensor &a, const Scalar &b) { return F::add(a, scalar_of(b, a)); }
Tensor operator+(const Scalar &a, const Tensor &b) { return F::add(scalar_of(a, b), b); }
Tensor operator-(const Tensor &a, const Tensor &b) { return F::sub(a, b); }
Tensor operator-(const Tensor &a, const Scalar &b) { return F::sub(a, scalar_of(b, a)); }
Tensor operator-(const Scalar &a, const Tensor &b) { return F::sub(scalar_of(a, b), b); }
Tensor operator*(const Tensor &a, const Tensor &b) { return F::mul(a, b); }
Tensor operator*(const Tensor &a, const Scalar &b) { return F::mul(a, scalar_of(b, a)); }
Tensor operator*(const Scalar &a, const Tensor &b) { return F::mul(scalar_of(a, b), b); }
Tensor operator/(const Tensor &a, const Tensor &b) { return F::div(a, b); }
Tensor operator/(const Tensor &a, const Scalar &b) { return F::div(a, scalar_of(b, a)); }
Tensor operator/(const Scalar &a, const Tensor &b) { return F::div(scalar_of(a, b), b); }
Tensor operator-(const Tensor &x) { return F::neg(x); }
Tensor operator^(const Tensor &x, const Scalar &e) { return F::pow(x, e); }
Tensor operator>(const Tensor &a, const Tensor &b) { return Tensor(*a.impl_->data_ > *b.impl_->data_); }
Tensor operator>(const Tensor &a, const Scalar &b) { return a > scalar_as(b, a); }
#define ODL_COMPARE(OP)                                                                                     \
    Tensor operator OP(const Tensor &a, const Tensor &b) { return Tensor(*a.impl_->data_ OP * b.impl_->data_); } \
    Tensor operator OP(const Tensor &a, const Scalar &b) { return a OP scalar_as(b, a); }
ODL_COMPARE(==)
ODL_COMPARE(!=)
ODL_COMPARE(<)
ODL_COMPARE(<=)
ODL_COMPARE(>=)
#undef ODL_COMPARE
// compound assignment works in place on the left operand's storage, as the reference's does (add.cpp:121-133)
Tensor &operator+=(Tensor &a, const Tensor &b) { F::add_(a, b); return a; }
Tensor &operator-=(Tensor &a, const Tensor &b) { F::sub_(a, b); return a; }
Tensor &operator*=(Tensor &a, const Tensor &b) { F::mul_(a, b); return a; }
Tensor &operator/=(Tensor &a, const Tensor &b) { F::div_(a, b); return a; }
Tensor &operator+=(Tensor &a, const Scalar &b) { F::add_(a, scalar_as(b, a)); return a; }
Tensor &operator-=(Tensor &a, const Scalar &b) { F::sub_(a, scalar_as(b, a)); return a; }
Tensor &operator*=(Tensor &a, const Scalar &b) { F::mul_(a, scalar_as(b, a)); return a; }
Tensor &operator/=(Tensor &a, const Scalar &b) { F::div_(a, scalar_as(b, a)); return a; }

Tensor Tensor::reshape(const Shape &shape) const { return F::reshape(*this, shape); }
Tensor Tensor::transpose() const { return F::transpose(*this); }

Tensor accuracy(const Tensor &y, const Tensor &target)
{
    if (y.shape().size() != 2)
        THROW_INVALID_ARG("accuracy expects y to be 2D (N, C), but got shape {}", y.shape().to_string());
    if (target.shape().size() != 1)
        THROW_INVALID_ARG("accuracy expects target to be 1D (N,), but got shape {}", target.shape().to_string());
    if (y.shape()[0] != target.shape()[0])
        THROW_INVALID_ARG("accuracy: batch size mismatch. y has {} samples, target has {} samples", y.shape()[0],
                          target.shape()[0]);
    const Tensor t32 = target.dtype() == DataType::kInt32 ? target : target.to(DataType::kInt32);
    const float acc  = static_cast<const OriginMat &>(*y.impl_->data_).accuracy(*t32.impl_->data_);
    return Tensor({acc}, Shape{}, dtype(DataType::kFloat32).device(y.device()));
}
}  // namespace origin
