// TEST INFRASTRUCTURE: one driver source, two backends.
// A C-ABI driver written against OriginDL's public Tensor / Operator / Mat API only — no algorithm is restated
// here. It is compiled twice:
//   * against the reference's own headers and CPU backend (oracle/Makefile -> oracle/_ref/libodl_ref.so, entry
//     points odl_ref_*, tensors on the CPU): the real reference, used to pin the plain-C oracle bit for bit, to
//     write tests/golden fixtures and as the CPU baseline of the benchmark;
//   * against this repository's host layer (origindl_amd/host, -DDRV_ON_DEVICE -DDRV_PREFIX=odl_host_, tensors on
//     the GPU): the same calls then run on the gfx950 backend, which is what "drop-in behind the Tensor/Operator/
//     Mat interfaces" means; tests compare its results with the fixtures and the oracle.
// Every entry point returns 0, or -1 for std::invalid_argument, -2 for any other std::exception.
#include <any>
#include <cstdint>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <random>
#include <stdexcept>
#include <vector>

#include "origin/core/operator.h"
#include "origin/core/parameter.h"
#include "origin/core/tensor.h"
#include "origin/mat/origin/origin_mat.h"
#include "origin/nn/layers/conv2d.h"
#include "origin/nn/layers/flatten.h"
#include "origin/nn/layers/linear.h"
#include "origin/nn/layers/max_pool2d.h"
#include "origin/nn/layers/relu.h"
#include "origin/nn/sequential.h"
#include "origin/pnnx/pnnx_graph.h"
#include "origin/operators/activation/relu.h"
#include "origin/operators/activation/softmax.h"
#include "origin/operators/conv/conv2d.h"
#include "origin/operators/loss/softmax_cross_entropy.h"
#include "origin/operators/math/add.h"
#include "origin/operators/math/broadcast_to.h"
#include "origin/operators/math/compare.h"
#include "origin/operators/math/div.h"
#include "origin/operators/math/exp.h"
#include "origin/operators/math/log.h"
#include "origin/utils/log.h"
#include "origin/operators/math/mat_mul.h"
#include "origin/operators/math/mul.h"
#include "origin/operators/math/neg.h"
#include "origin/operators/math/pow.h"
#include "origin/operators/math/square.h"
#include "origin/operators/math/sub.h"
#include "origin/operators/math/sum.h"
#include "origin/operators/math/sum_to.h"
#include "origin/io/checkpoint.h"
#include "origin/io/model_io.h"
#include "origin/nn/layers/batch_norm1d.h"
#include "origin/nn/models/mlp.h"
#include "origin/nn/layers/batch_norm2d.h"
#include "origin/operators/normalization/batch_norm.h"
#include "origin/operators/pooling/max_pool2d.h"
#include "origin/optim/adam.h"
#include "origin/optim/hooks.h"
#include "origin/optim/sgd.h"
#include "origin/utils/metrics.h"

using namespace origin;
namespace F = origin::functional;

#ifndef DRV_PREFIX
#    define DRV_PREFIX odl_ref_
#endif
#define DRV_CAT_(a, b) a##b
#define DRV_CAT(a, b) DRV_CAT_(a, b)
#define DRV(name) DRV_CAT(DRV_PREFIX, name)

namespace
{
#if defined(DRV_ON_DEVICE) || defined(DRV_DEVICE_TENSORS)
// (DRV_DEVICE_TENSORS alone: tensors on the device, but only calls the reference's own API has - the build against the
// reference's headers and objects with the gfx950 binding underneath)
const Device kDev(DeviceType::kCUDA, 0);
#else
const Device kDev(DeviceType::kCPU, 0);
#endif

Shape make_shape(const int64_t *dims, int n)
{
    std::vector<size_t> d(dims, dims + n);
    return Shape(d);
}

Tensor f32(const float *p, const Shape &s, bool grad = false)
{
    std::vector<float> v(p, p + s.elements());
    return Tensor(v, s, dtype(DataType::kFloat32).requires_grad(grad).device(kDev));
}

Tensor labels(const void *p, int is64, int64_t n)
{
    if (is64)
    {
        std::vector<int64_t> v((const int64_t *)p, (const int64_t *)p + n);
        return Tensor(v, Shape{(size_t)n}, dtype(DataType::kInt64).device(kDev));
    }
    std::vector<int32_t> v((const int32_t *)p, (const int32_t *)p + n);
    return Tensor(v, Shape{(size_t)n}, dtype(DataType::kInt32).device(kDev));
}

std::unique_ptr<origin::Mat> mat_f32(const float *p, const Shape &s)
{
    return OriginMat::from_memory(p, DataType::kFloat32, s, TensorOptions(DataType::kFloat32).device(kDev));
}

std::unique_ptr<origin::Mat> mat_labels(const void *p, int is64, int64_t n)
{
    return OriginMat::from_memory(p, is64 ? DataType::kInt64 : DataType::kInt32, Shape{(size_t)n},
                                  TensorOptions(is64 ? DataType::kInt64 : DataType::kInt32).device(kDev));
}

void out(const Tensor &t, float *dst)
{
    auto v = t.to_vector<float>();
    std::memcpy(dst, v.data(), v.size() * sizeof(float));
}

void out(const origin::Mat &m, float *dst)
{
    // (the reference's OriginMat::to_vector<T>() reads the storage in place: a device Mat comes to the host first)
    const auto host = m.device().type() == DeviceType::kCPU ? nullptr : m.to_device(Device(DeviceType::kCPU, 0));
    auto v = static_cast<const OriginMat &>(host ? *host : m).to_vector<float>();
    std::memcpy(dst, v.data(), v.size() * sizeof(float));
}

#ifdef DRV_ON_DEVICE
// a created stream made current for the scope (graph capture needs one: the null stream cannot be captured)
struct StreamScope
{
    void *s;
    StreamScope() : s(origin::cuda::create_stream()) { origin::cuda::set_stream(s); }
    ~StreamScope()
    {
        origin::cuda::set_stream(nullptr);
        origin::cuda::destroy_stream(s);
    }
};
#endif

template <typename Fn>
int guarded(Fn &&fn)
{
    try
    {
        fn();
        return 0;
    }
    catch (const std::invalid_argument &e)
    {
        if (std::getenv("ODL_DRV_VERBOSE"))
            std::fprintf(stderr, "driver: invalid_argument: %s\n", e.what());
        return -1;
    }
    catch (const std::exception &e)
    {
        if (std::getenv("ODL_DRV_VERBOSE"))
            std::fprintf(stderr, "driver: exception: %s\n", e.what());
        return -2;
    }
}
}  // namespace

namespace
{
template <class L>
void bn_layer_run(L &layer, const float *x, const Shape &xs, int64_t C, int steps, float scale, float *y_train,
                  float *y_eval, float *grads, bool with_backward)
{
    layer.to(kDev);
    layer.train(true);
    Tensor X, Y;
    for (int s = 0; s < steps; ++s)
    {
        std::vector<float> xv(x, x + xs.elements());
        for (auto &v : xv)
            v = v * (1.0f + scale * (float)s);
        X = f32(xv.data(), xs, true);  // a leaf, so that its gradient survives backward
        Y = layer.forward(X);
    }
    out(Y, y_train);
    if (with_backward)
    {
        // The reference itself cannot do this step: its operator moves the saved batch statistics into its outputs
        // (src/operators/normalization/batch_norm.cpp:78-83) and backward then finds them empty.
        auto loss = F::sum(Y * Y);
        layer.zero_grad();
        loss.backward();
        float *gp = grads;
        out(X.grad(), gp), gp += xs.elements();
        out(layer.weight()->grad(), gp), gp += C;
        out(layer.bias()->grad(), gp);
    }
    layer.train(false);
    out(layer.forward(f32(x, xs)), y_eval);
}
}  // namespace

// ---- model files and checkpoints (include/origin/io/model_io.h, checkpoint.h). An nn::MLP({4, 8, 2}) whose four
// parameters are set from `params` (layer_0.weight [4,8], layer_0.bias, layer_1.weight [8,2], layer_1.bias: 58 floats).
namespace
{
const char *const kMlpNames[4] = {"layer_0.weight", "layer_0.bias", "layer_1.weight", "layer_1.bias"};

void set_mlp(nn::MLP &model, const float *params)
{
    auto named = model.named_parameters("");
    const float *p = params;
    for (const char *name : kMlpNames)
    {
        Parameter *dst = named.at(name);
        *dst = Parameter(f32(p, dst->shape(), true));
        p += dst->shape().elements();
    }
}

void get_mlp(nn::MLP &model, float *params)
{
    auto named = model.named_parameters("");
    float *p = params;
    for (const char *name : kMlpNames)
    {
        out(static_cast<const Tensor &>(*named.at(name)), p);
        p += named.at(name)->shape().elements();
    }
}
}  // namespace

extern "C" {

int DRV(ping)()
{
#ifdef origin_logger
    // the reference's logger opens its file sink relative to the working directory when first used; touching it here
    // lets the loader choose that directory
    (void)origin_logger;
#endif
    return 1;
}

int DRV(matmul)(const float *a, const float *b, float *c, int64_t m, int64_t n, int64_t k)
{
    return guarded([&] {
        auto y = F::mat_mul(f32(a, Shape{(size_t)m, (size_t)k}), f32(b, Shape{(size_t)k, (size_t)n}));
        out(y, c);
    });
}

int DRV(matmul_batched)(const float *a, const float *b, float *c, int64_t batch, int64_t m, int64_t n, int64_t k,
                           int b_is_batched)
{
    return guarded([&] {
        auto A = f32(a, Shape{(size_t)batch, (size_t)m, (size_t)k});
        auto B = b_is_batched ? f32(b, Shape{(size_t)batch, (size_t)k, (size_t)n}) : f32(b, Shape{(size_t)k, (size_t)n});
        out(F::mat_mul(A, B), c);
    });
}

// forward + backward with an injected upstream gradient: z = y * dC; z.backward() seeds ones.
int DRV(matmul_fwd_bwd)(const float *x, const float *w, const float *gy, float *y, float *gx, float *gw, int64_t m,
                           int64_t k, int64_t n)
{
    return guarded([&] {
        auto X = f32(x, Shape{(size_t)m, (size_t)k}, true);
        auto W = f32(w, Shape{(size_t)k, (size_t)n}, true);
        auto G = f32(gy, Shape{(size_t)m, (size_t)n});
        auto Y = F::mat_mul(X, W);
        auto Z = Y * G;
        Z.backward();
        out(Y, y);
        out(X.grad(), gx);
        out(W.grad(), gw);
    });
}

// the same on float64 tensors: the product, and both gradients through the autograd graph
int DRV(matmul_f64_fwd_bwd)(const double *x, const double *w, const double *gy, double *y, double *gx, double *gw, int64_t m,
                            int64_t k, int64_t n)
{
    return guarded([&] {
        auto f64 = [](const double *p, const Shape &s, bool grad) {
            std::vector<double> v(p, p + s.elements());
            return Tensor(v, s, dtype(DataType::kFloat64).requires_grad(grad).device(kDev));
        };
        auto put = [](const Tensor &t, double *dst) {
            auto v = t.to_vector<double>();
            std::memcpy(dst, v.data(), v.size() * sizeof(double));
        };
        auto X = f64(x, Shape{(size_t)m, (size_t)k}, true);
        auto W = f64(w, Shape{(size_t)k, (size_t)n}, true);
        auto G = f64(gy, Shape{(size_t)m, (size_t)n}, false);
        auto Y = F::mat_mul(X, W);
        auto Z = Y * G;
        Z.backward();
        put(Y, y);
        put(X.grad(), gx);
        put(W.grad(), gw);
    });
}

// conv2d on float64 tensors through the whole operator path: y = conv2d(x, W, b); (y * gy).backward()
int DRV(conv2d_f64_fwd_bwd)(const double *gy, const double *x, const double *w, const double *b, int64_t N, int64_t C, int64_t H,
                            int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, double *y, double *gx,
                            double *gw, double *gb)
{
    return guarded([&] {
        auto f64 = [](const double *p, const Shape &s, bool grad) {
            std::vector<double> v(p, p + s.elements());
            return Tensor(v, s, dtype(DataType::kFloat64).requires_grad(grad).device(kDev));
        };
        auto put = [](const Tensor &t, double *dst) {
            auto v = t.to_vector<double>();
            std::memcpy(dst, v.data(), v.size() * sizeof(double));
        };
        auto X  = f64(x, Shape{(size_t)N, (size_t)C, (size_t)H, (size_t)W}, true);
        auto Wt = f64(w, Shape{(size_t)OC, (size_t)C, (size_t)KH, (size_t)KW}, true);
        Tensor B;
        if (b)
            B = f64(b, Shape{(size_t)OC}, true);
        auto Y = F::conv2d(X, Wt, b ? &B : nullptr, {SH, SW}, {PH, PW});
        auto G = f64(gy, Y.shape(), false);
        auto Z = Y * G;
        Z.backward();
        put(Y, y);
        put(X.grad(), gx);
        put(Wt.grad(), gw);
        if (b && gb)
            put(B.grad(), gb);
    });
}

// softmax on a float64 tensor, forward and backward: y = softmax(x, axis); (y * gy).backward()
int DRV(softmax_f64_fwd_bwd)(const double *x, const double *gy, const int64_t *shape, int nd, int axis, double *y, double *gx)
{
    return guarded([&] {
        const Shape s = make_shape(shape, nd);
        std::vector<double> xv(x, x + s.elements()), gv(gy, gy + s.elements());
        auto X = Tensor(xv, s, dtype(DataType::kFloat64).requires_grad(true).device(kDev));
        auto G = Tensor(gv, s, dtype(DataType::kFloat64).device(kDev));
        auto Y = F::softmax(X, axis);
        auto Z = Y * G;
        Z.backward();
        auto yv = Y.to_vector<double>(), gxv = X.grad().to_vector<double>();
        std::memcpy(y, yv.data(), yv.size() * sizeof(double));
        std::memcpy(gx, gxv.data(), gxv.size() * sizeof(double));
    });
}

int DRV(transpose)(const float *src, float *dst, const int64_t *shape, int nd)
{
    return guarded([&] { out(f32(src, make_shape(shape, nd)).transpose(), dst); });
}

int DRV(im2col)(const float *img, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH,
                   int PW, int to_matrix, float *col)
{
    return guarded([&] {
        auto m = mat_f32(img, Shape{(size_t)N, (size_t)C, (size_t)H, (size_t)W});
        out(*m->im2col({KH, KW}, {SH, SW}, {PH, PW}, to_matrix != 0), col);
    });
}

int DRV(col2im)(const float *col, const int64_t *col_shape, int col_nd, int64_t N, int64_t C, int64_t H, int64_t W,
                   int KH, int KW, int SH, int SW, int PH, int PW, int to_matrix, float *img)
{
    return guarded([&] {
        auto m = mat_f32(col, make_shape(col_shape, col_nd));
        out(*m->col2im(Shape{(size_t)N, (size_t)C, (size_t)H, (size_t)W}, {KH, KW}, {SH, SW}, {PH, PW}, to_matrix != 0),
            img);
    });
}

int DRV(conv2d)(const float *x, const float *w, const float *b, int64_t N, int64_t C, int64_t H, int64_t W,
                   int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, float *y)
{
    return guarded([&] {
        auto X  = f32(x, Shape{(size_t)N, (size_t)C, (size_t)H, (size_t)W});
        auto Wt = f32(w, Shape{(size_t)OC, (size_t)C, (size_t)KH, (size_t)KW});
        Tensor B;
        if (b)
            B = f32(b, Shape{(size_t)OC});
        out(F::conv2d(X, Wt, b ? &B : nullptr, {SH, SW}, {PH, PW}), y);
    });
}

// full operator path: y = conv2d(x, W, b); (y * gy).backward()
int DRV(conv2d_backward)(const float *gy, const float *x, const float *w, const float *b, int64_t N, int64_t C,
                            int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, float *gx,
                            float *gw, float *gb)
{
    return guarded([&] {
        auto X  = f32(x, Shape{(size_t)N, (size_t)C, (size_t)H, (size_t)W}, true);
        auto Wt = f32(w, Shape{(size_t)OC, (size_t)C, (size_t)KH, (size_t)KW}, true);
        Tensor B;
        if (b)
            B = f32(b, Shape{(size_t)OC}, true);
        auto Y = F::conv2d(X, Wt, b ? &B : nullptr, {SH, SW}, {PH, PW});
        auto G = f32(gy, Y.shape());
        auto Z = Y * G;
        Z.backward();
        out(X.grad(), gx);
        out(Wt.grad(), gw);
        if (b && gb)
            out(B.grad(), gb);
    });
}

int DRV(sum)(const float *src, const int64_t *shape, int nd, int axis, int keepdim, float *dst)
{
    return guarded([&] { out(F::sum(f32(src, make_shape(shape, nd)), axis, keepdim != 0), dst); });
}

int DRV(max)(const float *src, const int64_t *shape, int nd, int axis, float *dst)
{
    return guarded([&] { out(*mat_f32(src, make_shape(shape, nd))->max(axis), dst); });
}

int DRV(sum_to)(const float *src, const int64_t *sshape, int sn, const int64_t *tshape, int tn, float *dst)
{
    return guarded([&] { out(F::sum_to(f32(src, make_shape(sshape, sn)), make_shape(tshape, tn)), dst); });
}

int DRV(broadcast_to)(const float *src, const int64_t *sshape, int sn, const int64_t *dshape, int dn, float *dst)
{
    return guarded([&] { out(F::broadcast_to(f32(src, make_shape(sshape, sn)), make_shape(dshape, dn)), dst); });
}

// backward of broadcast_to with upstream gradient g (left-aligned sum_to inside the reference)
int DRV(broadcast_to_backward)(const float *src, const int64_t *sshape, int sn, const int64_t *dshape, int dn,
                                  const float *g, float *gsrc)
{
    return guarded([&] {
        auto X = f32(src, make_shape(sshape, sn), true);
        auto Y = F::broadcast_to(X, make_shape(dshape, dn));
        auto Z = Y * f32(g, make_shape(dshape, dn));
        Z.backward();
        out(X.grad(), gsrc);
    });
}

int DRV(softmax)(const float *x, const int64_t *shape, int nd, int axis, float *y)
{
    return guarded([&] { out(F::softmax(f32(x, make_shape(shape, nd)), axis), y); });
}

int DRV(gather)(const float *in, const void *idx, int is64, int64_t N, int64_t C, float *o)
{
    return guarded([&] {
        auto m = mat_f32(in, Shape{(size_t)N, (size_t)C});
        out(*m->gather(*mat_labels(idx, is64, N)), o);
    });
}

int DRV(one_hot)(const void *idx, int is64, int64_t N, int64_t C, float *o)
{
    return guarded([&] {
        auto t = mat_labels(idx, is64, N);
        out(*t->one_hot(*t, (int)C), o);
    });
}

int DRV(softmax_ce)(const float *x, const void *t, int is64, int64_t N, int64_t C, float *loss, float *gx)
{
    return guarded([&] {
        auto X = f32(x, Shape{(size_t)N, (size_t)C}, true);
        auto T = labels(t, is64, N);
        auto L = F::softmax_cross_entropy(X, T);
        *loss  = L.item<float>();
        if (gx)
        {
            L.backward();
            out(X.grad(), gx);
        }
    });
}

int DRV(max_pool2d)(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW,
                       int PH, int PW, float *y, uint64_t *idx)
{
    return guarded([&] {
        auto m = mat_f32(x, Shape{(size_t)N, (size_t)C, (size_t)H, (size_t)W});
        std::vector<size_t> ind;
        out(*m->max_pool2d({KH, KW}, {SH, SW}, {PH, PW}, &ind), y);
        for (size_t i = 0; i < ind.size(); ++i)
            idx[i] = ind[i];
    });
}

int DRV(max_pool2d_backward)(const float *gy, const uint64_t *idx, int64_t N, int64_t C, int64_t H, int64_t W,
                                int KH, int KW, int SH, int SW, int PH, int PW, float *gx)
{
    return guarded([&] {
        int OH = (int)((H + 2 * PH - KH) / SH + 1), OW = (int)((W + 2 * PW - KW) / SW + 1);
        std::vector<float> zeros((size_t)(N * C * H * W), 0.0f);
        auto xm = mat_f32(zeros.data(), Shape{(size_t)N, (size_t)C, (size_t)H, (size_t)W});
        auto gm = mat_f32(gy, Shape{(size_t)N, (size_t)C, (size_t)OH, (size_t)OW});
        std::vector<size_t> ind(idx, idx + (size_t)(N * C * OH * OW));
        out(*xm->max_pool2d_backward(*gm, {KH, KW}, {SH, SW}, {PH, PW}, ind), gx);
    });
}

int DRV(accuracy)(const float *y, const int32_t *t, int64_t N, int64_t C, float *acc)
{
    return guarded([&] {
        std::vector<int32_t> tv(t, t + N);
        auto T = Tensor(tv, Shape{(size_t)N}, dtype(DataType::kInt32).device(kDev));
        *acc   = accuracy(f32(y, Shape{(size_t)N, (size_t)C}), T).item<float>();
    });
}

// op: 0 add 1 sub 2 mul 3 div 4 gt
int DRV(binary)(int op, const float *a, const int64_t *ashape, int an, const float *b, const int64_t *bshape, int bn,
                   float *o)
{
    return guarded([&] {
        auto A = f32(a, make_shape(ashape, an));
        auto B = f32(b, make_shape(bshape, bn));
        Tensor R;
        switch (op)
        {
            case 0: R = A + B; break;
            case 1: R = A - B; break;
            case 2: R = A * B; break;
            case 3: R = A / B; break;
            default: R = A > B; break;
        }
        out(R, o);
    });
}

// op: 0 relu 1 exp 2 log 3 neg 4 square
int DRV(unary)(int op, const float *a, int64_t n, float *o)
{
    return guarded([&] {
        auto A = f32(a, Shape{(size_t)n});
        Tensor R;
        switch (op)
        {
            case 0: R = F::relu(A); break;
            case 1: R = F::exp(A); break;
            case 2: R = F::log(A); break;
            case 3: R = -A; break;
            default: R = F::square(A); break;
        }
        out(R, o);
    });
}

// ---- detector forward path, at the Mat interface (mat.h:392-405, 719-797)
int DRV(activation)(int op, const float *a, int64_t n, float *o)  // 6 sigmoid, 7 silu
{
    return guarded([&] {
        auto m = mat_f32(a, Shape{(size_t)n});
        out(op == 6 ? *m->sigmoid() : *m->silu(), o);
    });
}

int DRV(upsample)(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW, int sh, int sw,
                  float *y)
{
    return guarded([&] {
        auto m = mat_f32(x, Shape{(size_t)N, (size_t)C, (size_t)H, (size_t)W});
        out(*m->upsample(Shape{(size_t)N, (size_t)C, (size_t)OH, (size_t)OW}, sh, sw, "nearest"), y);
    });
}

int DRV(cat)(const float *const *inputs, const int64_t *axis_sizes, int count, int64_t outer, int64_t inner, float *o)
{
    return guarded([&] {
        std::vector<std::unique_ptr<origin::Mat>> mats;
        for (int i = 0; i < count; ++i)
            mats.push_back(mat_f32(inputs[i], Shape{(size_t)outer, (size_t)axis_sizes[i], (size_t)inner}));
        std::vector<const origin::Mat *> others;
        for (int i = 1; i < count; ++i)
            others.push_back(mats[i].get());
        out(*mats[0]->cat(others, 1), o);
    });
}

int DRV(yolo_detect)(const float *x, const float *w, const float *b, const float *grid, const float *anchor_grid,
                     int64_t anchor_H, int64_t anchor_W, int64_t N, int64_t C, int64_t H, int64_t W, float stride,
                     int num_anchors, int num_classes, float *o)
{
    return guarded([&] {
        const size_t A = (size_t)num_anchors, CI = (size_t)num_classes + 5;
        auto xm = mat_f32(x, Shape{(size_t)N, (size_t)C, (size_t)H, (size_t)W});
        auto wm = mat_f32(w, Shape{A * CI, (size_t)C, 1, 1});
        std::unique_ptr<origin::Mat> bm;
        if (b)
            bm = mat_f32(b, Shape{A * CI});
        auto gm = mat_f32(grid, Shape{1, A, (size_t)H, (size_t)W, 2});
        auto am = mat_f32(anchor_grid, Shape{1, A, (size_t)anchor_H, (size_t)anchor_W, 2});
        out(*xm->yolo_detect_forward(*wm, bm.get(), *gm, *am, stride, num_anchors, num_classes), o);
    });
}

// ---- batch normalisation at the Mat interface (mat.h:584-649); H == 0 selects the two-dimensional [N, C] form
int DRV(batch_norm_forward)(const float *x, const float *gamma, const float *beta, const float *rm, const float *rv,
                            int training, float eps, int64_t N, int64_t C, int64_t H, int64_t W, float *y, float *mean,
                            float *var, float *x_norm)
{
    return guarded([&] {
        const int nd = H == 0 ? 2 : 4;
        const Shape xs = nd == 2 ? Shape{(size_t)N, (size_t)C} : Shape{(size_t)N, (size_t)C, (size_t)H, (size_t)W};
        auto xm = mat_f32(x, xs);
        auto g = mat_f32(gamma, Shape{(size_t)C}), b = mat_f32(beta, Shape{(size_t)C});
        auto m = mat_f32(rm, Shape{(size_t)C}), v = mat_f32(rv, Shape{(size_t)C});
        if (x_norm)
        {
            auto r = xm->batch_norm_forward(*g, *b, *m, *v, training != 0, eps, nd);
            out(*r.y, y), out(*r.mean, mean), out(*r.var, var), out(*r.x_norm, x_norm);
        }
        else
            out(*xm->batch_norm(*g, *b, *m, *v, training != 0, eps, 0.1f, nd), y);
    });
}

int DRV(batch_norm_backward)(const float *gy, const float *x, const float *gamma, const float *saved_mean,
                             const float *saved_var, const float *saved_x_norm, float eps, int64_t N, int64_t C, int64_t H,
                             int64_t W, float *gx, float *dgamma, float *dbeta)
{
    return guarded([&] {
        const int nd = H == 0 ? 2 : 4;
        const Shape xs = nd == 2 ? Shape{(size_t)N, (size_t)C} : Shape{(size_t)N, (size_t)C, (size_t)H, (size_t)W};
        auto xm = mat_f32(x, xs), gm = mat_f32(gy, xs), xn = mat_f32(saved_x_norm, xs);
        auto g = mat_f32(gamma, Shape{(size_t)C});
        auto m = mat_f32(saved_mean, Shape{(size_t)C}), v = mat_f32(saved_var, Shape{(size_t)C});
        auto r = xm->batch_norm_backward(*gm, *g, *m, *v, *xn, eps, nd);
        out(*r[0], gx), out(*r[1], dgamma), out(*r[2], dbeta);
    });
}

// nn::BatchNorm2d (H > 0) or nn::BatchNorm1d (H == 0) in training mode, `steps` forwards of x * (1 + scale*step):
// the last output, with_backward: the gradients of sum(y*y) from that forward (the scaled input, then gamma, then
// beta), and one evaluation-mode forward of x. Exercises the running-statistics update (batch_norm2d.cpp:62-86) and the operator's
// backward through the autograd engine.
int DRV(batch_norm_layer)(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int steps, float eps, float momentum,
                          float scale, int with_backward, float *y_train, float *y_eval, float *grads)
{
    return guarded([&] {
        if (H == 0)
        {
            nn::BatchNorm1d layer((int)C, eps, momentum);
            bn_layer_run(layer, x, Shape{(size_t)N, (size_t)C}, C, steps, scale, y_train, y_eval, grads, with_backward != 0);
        }
        else
        {
            nn::BatchNorm2d layer((int)C, eps, momentum);
            bn_layer_run(layer, x, Shape{(size_t)N, (size_t)C, (size_t)H, (size_t)W}, C, steps, scale, y_train, y_eval,
                         grads, with_backward != 0);
        }
    });
}

// writes the model's state_dict() to `path` in the .odl format
int DRV(save_mlp)(const float *params, const char *path)
{
    return guarded([&] {
        nn::MLP model({4, 8, 2});
        set_mlp(model, params);
        save(model.state_dict(), path);
    });
}

// Module::load(path, strict) into a fresh model; the loaded parameters come back in `params`, and y = model(x[3,4])
// after moving the model to the driver's device
int DRV(load_mlp)(const char *path, int strict, const float *x, float *params, float *y)
{
    return guarded([&] {
        nn::MLP model({4, 8, 2});
        model.load(path, strict != 0);
        get_mlp(model, params);
        if (y)
        {
            model.to(kDev);
            out(model(f32(x, Shape{3, 4})), y);
        }
    });
}

// save(Checkpoint) then load_checkpoint of the same path: the metadata read back, and the parameters
int DRV(checkpoint_roundtrip)(const float *params, const char *path, int epoch, int step, float loss, float lr, float beta1,
                              float beta2, float eps, int *epoch_step /*2*/, float *floats /* loss lr beta1 beta2 eps */,
                              float *params_out)
{
    return guarded([&] {
        nn::MLP model({4, 8, 2});
        set_mlp(model, params);
        Adam opt(model, lr, beta1, beta2, eps);
        Checkpoint ck;
        ck.model_state_dict = model.state_dict();
        ck.optimizer_state_dict["adam"] = opt.state_dict();
        ck.epoch = epoch, ck.step = step, ck.loss = loss, ck.optimizer_type = "Adam";
        ck.optimizer_config["lr"] = lr, ck.optimizer_config["beta1"] = beta1;
        ck.optimizer_config["beta2"] = beta2, ck.optimizer_config["eps"] = eps;
        save(ck, path);
        Checkpoint back = load_checkpoint(path);
        epoch_step[0] = back.epoch, epoch_step[1] = back.step;
        floats[0] = back.loss, floats[1] = back.optimizer_config.at("lr"), floats[2] = back.optimizer_config.at("beta1");
        floats[3] = back.optimizer_config.at("beta2"), floats[4] = back.optimizer_config.at("eps");
        if (back.optimizer_type != "Adam")
            throw std::runtime_error("optimizer type lost");
        nn::MLP fresh({4, 8, 2});
        fresh.load_state_dict(back.model_state_dict);
        get_mlp(fresh, params_out);
        auto st = opt.state_dict();
        if (std::any_cast<float>(st.at("lr")) != lr || std::any_cast<float>(st.at("eps")) != eps)
            throw std::runtime_error("optimizer state_dict does not hold its settings");
    });
}
// A PNNX model (`.pnnx.param` + `.pnnx.bin`) run forward `reps` times on x[N,C,H,W]; the first output of
// `pnnx_output_0` is copied to out (capacity in floats) and its shape to out_shape[0..out_nd). ms = mean time of the
// forwards after the first (which also loads weights), each complete on the device; the output is read back once, after.
// 0: every node of a PNNX graph runs on its own, as in the reference's runner (only this repository's runner has the
// switch; the reference's classes ignore it). The launches of the forward recorded last are read back below.
static int g_pnnx_fusion = 1;
static int64_t g_pnnx_graph_nodes = 0;
static float g_pnnx_host_ms = 0.0f;  // mean time forward() took to return (its launches queued, not yet run)
int DRV(pnnx_set_fusion)(int on)
{
    g_pnnx_fusion = on;
    return 0;
}
int DRV(pnnx_last_graph_nodes)(int64_t *nodes)
{
    *nodes = g_pnnx_graph_nodes;
    return 0;
}
int DRV(pnnx_last_host_ms)(float *ms)
{
    *ms = g_pnnx_host_ms;
    return 0;
}

int DRV(pnnx_forward)(const char *param_path, const char *bin_path, const float *x, int64_t N, int64_t C, int64_t H,
                      int64_t W, int reps, float *o, int64_t capacity, int64_t *out_shape, int *out_nd, float *ms)
{
    return guarded([&] {
        origin::pnnx::PNNXGraph graph(param_path, bin_path);
#ifdef ORIGINDL_AMD_PNNX_FUSION
        graph.set_fusion(g_pnnx_fusion != 0);
#endif
        graph.build();
        auto X = f32(x, Shape{(size_t)N, (size_t)C, (size_t)H, (size_t)W});
        std::vector<Tensor> outs;
        float host_ms = 0.0f;
        auto t0 = std::chrono::steady_clock::now();
        for (int r = 0; r < (reps < 1 ? 1 : reps); ++r)
        {
            if (r == 1)
                t0 = std::chrono::steady_clock::now();
            graph.set_inputs("pnnx_input_0", {X});
            const auto h0 = std::chrono::steady_clock::now();
            graph.forward();
            if (r >= 1)
                host_ms += std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - h0).count();
            outs = graph.get_outputs("pnnx_output_0");
#ifdef DRV_ON_DEVICE
            origin::cuda::synchronize();  // the forward is complete on the device; the copy to the host comes after the loop
#endif
        }
        const auto t1 = std::chrono::steady_clock::now();
        if (outs.empty())
            throw std::runtime_error("pnnx_forward: the graph produced no output");
        const Shape shp         = outs[0].shape();
        std::vector<float> last = outs[0].to_vector<float>();
        if (ms)
            *ms = reps > 1 ? std::chrono::duration<float, std::milli>(t1 - t0).count() / (float)(reps - 1) : 0.0f;
        g_pnnx_host_ms = reps > 1 ? host_ms / (float)(reps - 1) : 0.0f;
        if ((int64_t)last.size() > capacity)
            throw std::invalid_argument("pnnx_forward: output larger than the buffer");
        std::memcpy(o, last.data(), last.size() * sizeof(float));
        *out_nd = (int)shp.size();
        for (size_t i = 0; i < shp.size(); ++i)
            out_shape[i] = (int64_t)shp[i];
    });
}

#ifdef DRV_ON_DEVICE
// The same model with its forward recorded into a graph: two ordinary forwards (weights uploaded, pool warm), the
// capture, then `reps` replays. Before every replay the input tensor is rewritten in place with x scaled by
// (1 + 0.125 * replay), the last replay with x itself, so the output returned is the one of x and a replay that
// ignored its input would be caught. ms = mean time of a replay, complete on the device.
int DRV(pnnx_forward_graph)(const char *param_path, const char *bin_path, const float *x, int64_t N, int64_t C, int64_t H,
                            int64_t W, int reps, float *o, int64_t capacity, int64_t *out_shape, int *out_nd, float *ms)
{
    return guarded([&] {
        StreamScope stream;
        origin::pnnx::PNNXGraph graph(param_path, bin_path);
#ifdef ORIGINDL_AMD_PNNX_FUSION
        graph.set_fusion(g_pnnx_fusion != 0);
#endif
        graph.build();
        const Shape xs{(size_t)N, (size_t)C, (size_t)H, (size_t)W};
        auto X = f32(x, xs);
        graph.set_inputs("pnnx_input_0", {X});
        for (int r = 0; r < 2; ++r)
            graph.forward();
        origin::cuda::Graph recorded;
        recorded.begin_capture();
        graph.forward();
        recorded.end_capture();
        g_pnnx_graph_nodes = (int64_t)recorded.node_count();
        std::vector<Tensor> outs = graph.get_outputs("pnnx_output_0");
        if (outs.empty())
            throw std::runtime_error("pnnx_forward: the graph produced no output");
        const int n = reps < 1 ? 1 : reps;
        std::vector<float> scaled(xs.elements());
        float total_ms = 0.0f;
        for (int r = 0; r < n; ++r)
        {
            const float f = r + 1 == n ? 1.0f : 1.0f + 0.125f * (float)(r + 1);
            for (size_t i = 0; i < scaled.size(); ++i)
                scaled[i] = x[i] * f;
            X.upload(scaled.data(), scaled.size() * sizeof(float));
            const auto t0 = std::chrono::steady_clock::now();
            recorded.launch();
            origin::cuda::synchronize();
            total_ms += std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - t0).count();
        }
        const Shape shp         = outs[0].shape();
        std::vector<float> last = outs[0].to_vector<float>();
        if (ms)
            *ms = total_ms / (float)n;
        if ((int64_t)last.size() > capacity)
            throw std::invalid_argument("pnnx_forward: output larger than the buffer");
        std::memcpy(o, last.data(), last.size() * sizeof(float));
        *out_nd = (int)shp.size();
        for (size_t i = 0; i < shp.size(); ++i)
            out_shape[i] = (int64_t)shp[i];
    });
}
#endif

int DRV(pow_scalar)(const float *a, int64_t n, float e, float *o)
{
    return guarded([&] { out(F::pow(f32(a, Shape{(size_t)n}), Scalar(e)), o); });
}

// MLP D -> Hd -> C (Linear, ReLU, Linear), softmax CE, WeightDecay hook, Adam; `steps` steps on the same batch.
// Parameters are read and written in place; loss/grads/logits of the LAST step are returned.
}  // extern "C"

namespace
{
// use_graph (device build only): the first step runs ordinarily, then one step is recorded into a graph and the
// remaining steps are replays of it — the results must be the ones of `steps` ordinary steps, bit for bit.
int mlp_train_impl(const float *x, const void *t, int is64, int64_t N, int64_t D, int64_t Hd, int64_t C, float *W1,
                   float *b1, float *W2, float *b2, int steps, float lr, float beta1, float beta2, float eps, float wd,
                   float *loss, float *gW1, float *gb1, float *gW2, float *gb2, float *logits, bool use_graph)
{
    return guarded([&] {
#ifdef DRV_ON_DEVICE
        std::unique_ptr<StreamScope> stream;
        if (use_graph)
            stream = std::make_unique<StreamScope>();
#else
        if (use_graph)
            throw std::runtime_error("graph replay is only available on the device build of this driver");
#endif
        Sequential model;
        model.add(std::make_unique<nn::Linear>((int)D, (int)Hd, true));
        model.add(std::make_unique<nn::ReLU>());
        model.add(std::make_unique<nn::Linear>((int)Hd, (int)C, true));
        auto &l1 = dynamic_cast<nn::Linear &>(model[0]);
        auto &l2 = dynamic_cast<nn::Linear &>(model[2]);
        Adam opt(model, lr, beta1, beta2, eps);
        if (wd != 0.0f)
            opt.register_hook(WeightDecay(wd).hook());
        *l1.weight() = Parameter(f32(W1, Shape{(size_t)D, (size_t)Hd}, true));
        *l1.bias()   = Parameter(f32(b1, Shape{1, (size_t)Hd}, true));
        *l2.weight() = Parameter(f32(W2, Shape{(size_t)Hd, (size_t)C}, true));
        *l2.bias()   = Parameter(f32(b2, Shape{1, (size_t)C}, true));
        auto X = f32(x, Shape{(size_t)N, (size_t)D});
        auto T = labels(t, is64, N);
        model.train();
        for (int s = 0; s < (use_graph ? 1 : steps); ++s)
        {
            opt.zero_grad();
            auto y = model(X);
            auto L = F::softmax_cross_entropy(y, T);
            L.backward();
            *loss = L.item<float>();
            out(y, logits);
            out(l1.weight()->grad(), gW1);
            out(l1.bias()->grad(), gb1);
            out(l2.weight()->grad(), gW2);
            out(l2.bias()->grad(), gb2);
            opt.step();
        }
#ifdef DRV_ON_DEVICE
        if (use_graph && steps > 1)
        {
            origin::cuda::Graph graph;
            graph.begin_capture();
            opt.zero_grad();
            auto y = model(X);
            auto L = F::softmax_cross_entropy(y, T);
            L.backward();
            opt.step();
            graph.end_capture();
            for (int s = 1; s < steps; ++s)
            {
                opt.prepare_replay();
                graph.launch();
                // ordinary work between the replays, on memory the graph does not own: a replay must not depend on
                // what ran in between
                auto scratch = (X * Scalar(2.0f)).to_vector<float>();
                (void)scratch;
            }
            *loss = L.item<float>();
            out(y, logits);
            // the gradients of the last replay, after the weight-decay hook of the recorded step (the ordinary loop
            // above reports them before the hook): equal to it only when wd == 0
            out(l1.weight()->grad(), gW1);
            out(l1.bias()->grad(), gb1);
            out(l2.weight()->grad(), gW2);
            out(l2.bias()->grad(), gb2);
        }
#endif
        out(*l1.weight(), W1);
        out(*l1.bias(), b1);
        out(*l2.weight(), W2);
        out(*l2.bias(), b2);
    });
}
}  // namespace

extern "C" {
int DRV(mlp_train)(const float *x, const void *t, int is64, int64_t N, int64_t D, int64_t Hd, int64_t C, float *W1,
                      float *b1, float *W2, float *b2, int steps, float lr, float beta1, float beta2, float eps,
                      float wd, float *loss, float *gW1, float *gb1, float *gW2, float *gb2, float *logits)
{
    return mlp_train_impl(x, t, is64, N, D, Hd, C, W1, b1, W2, b2, steps, lr, beta1, beta2, eps, wd, loss, gW1, gb1, gW2,
                          gb2, logits, false);
}

#ifdef DRV_ON_DEVICE
int DRV(mlp_train_graph)(const float *x, const void *t, int is64, int64_t N, int64_t D, int64_t Hd, int64_t C, float *W1,
                         float *b1, float *W2, float *b2, int steps, float lr, float beta1, float beta2, float eps,
                         float wd, float *loss, float *gW1, float *gb1, float *gW2, float *gb2, float *logits)
{
    return mlp_train_impl(x, t, is64, N, D, Hd, C, W1, b1, W2, b2, steps, lr, beta1, beta2, eps, wd, loss, gW1, gb1, gW2,
                          gb2, logits, true);
}
#endif

#ifdef DRV_ON_DEVICE
// Uploads into recycled device memory must wait for the kernels that still read it. On a created (non-blocking) stream:
// `reps` products of an all-ones [n,n] matrix are queued, the matrix is dropped while they are still running — its block
// returns to the pool — and a host array of the same size is uploaded at once, which the pool serves from that block.
// wrong[0] counts product elements that are not n (a product that read the overwritten operand), wrong[1] elements of
// the uploaded tensor that did not arrive.
int DRV(upload_ordering)(int64_t n, int reps, int64_t *wrong)
{
    return guarded([&] {
        StreamScope stream;
        const Shape shp{(size_t)n, (size_t)n};
        std::vector<float> ones((size_t)(n * n), 1.0f), twos((size_t)(n * n), 2.0f);
        auto w = mat_f32(ones.data(), shp);
        auto x = mat_f32(ones.data(), shp);
        std::vector<std::unique_ptr<origin::Mat>> ys;
        for (int r = 0; r < reps; ++r)
            ys.push_back(x->matmul(*w));
        x.reset();
        auto b = mat_f32(twos.data(), shp);
        wrong[0] = wrong[1] = 0;
        for (auto &y : ys)
            for (float v : static_cast<const OriginMat &>(*y).to_vector<float>())
                wrong[0] += v != (float)n;
        for (float v : static_cast<const OriginMat &>(*b).to_vector<float>())
            wrong[1] += v != 2.0f;
    });
}

// A capture that fails in the middle must leave the thread usable. stage[0] counts how far the scenario got:
// 1 the exception of a host read inside a capture arrived, 2 an ordinary step ran afterwards, 3 a fresh capture and a
// replay ran and the replayed loss equals the ordinary one of the same step, 4 end_capture from a Graph that did not begin
// the capture was refused (and that capture given up cleanly), 5 ordinary work still runs. After a replay on labels with
// an out-of-range entry flags[0] holds the loss's bad-label flag, after a replay on the good labels again flags[1].
int DRV(graph_abort_recovery)(const float *x, const int32_t *t, int64_t N, int64_t D, int64_t C, int *stage, int *flags)
{
    return guarded([&] {
        StreamScope stream;
        *stage = 0;
        auto run = [&](int steps, bool replay_last, float *loss_out) {
            Sequential model;
            model.add(std::make_unique<nn::Linear>((int)D, (int)C, true));
            auto &l = dynamic_cast<nn::Linear &>(model[0]);
            std::vector<float> w((size_t)(D * C));
            for (size_t i = 0; i < w.size(); ++i)
                w[i] = 0.01f * (float)((int)(i % 7) - 3);
            *l.weight() = Parameter(f32(w.data(), Shape{(size_t)D, (size_t)C}, true));
            std::vector<float> zeros((size_t)C, 0.0f);
            *l.bias() = Parameter(f32(zeros.data(), Shape{1, (size_t)C}, true));
            SGD opt(model, 0.1f);
            auto X = f32(x, Shape{(size_t)N, (size_t)D});
            auto T = labels(t, 0, N);
            model.train();
            auto step = [&] {
                opt.zero_grad();
                auto L = F::softmax_cross_entropy(model(X), T);
                L.backward();
                opt.step();
                return L;
            };
            for (int s = 0; s + 1 < steps; ++s)
                step();
            if (!replay_last)
            {
                *loss_out = step().item<float>();
                return;
            }
            origin::cuda::Graph g;
            g.begin_capture();
            auto L = step();
            g.end_capture();
            // the capture run itself executed nothing: the replay is step number `steps`
            g.launch();
            *loss_out = L.item<float>();
            if (flags)
            {
                std::vector<int32_t> bad(t, t + N);
                bad[(size_t)(N / 2)] = (int32_t)C;  // one past the last class
                T.upload(bad.data(), bad.size() * sizeof(int32_t));
                g.launch();
                flags[0] = F::softmax_cross_entropy_bad_label(L) ? 1 : 0;
                T.upload(t, (size_t)N * sizeof(int32_t));
                g.launch();
                flags[1] = F::softmax_cross_entropy_bad_label(L) ? 1 : 0;
            }
        };
        try
        {
            origin::cuda::Graph g;
            g.begin_capture();
            auto X = f32(x, Shape{(size_t)N, (size_t)D});  // a host-to-device copy: not allowed while recording
            (void)X;
            g.end_capture();
        }
        catch (const std::runtime_error &)
        {
            *stage = 1;
        }
        if (*stage != 1 || origin::cuda::is_capturing())
            return;
        float eager = 0.f, replayed = 0.f;
        run(3, false, &eager);
        *stage = 2;
        run(3, true, &replayed);
        if (eager != replayed)
            return;
        *stage = 3;
        {
            origin::cuda::Graph a, b;
            a.begin_capture();
            bool refused = false;
            try
            {
                b.end_capture();
            }
            catch (const std::runtime_error &)
            {
                refused = true;
            }
            a.abort_capture();
            if (!refused || origin::cuda::is_capturing())
                return;
        }
        *stage = 4;
        float again = 0.f;
        flags = nullptr;
        run(3, false, &again);
        if (again == eager)
            *stage = 5;
    });
}
#endif

// CNN of the benchmark's CNN training configuration (no BatchNorm), SGD without momentum/weight decay, one step.
int DRV(cnn_train)(const float *x, const void *t, int is64, int64_t N, int64_t S, int64_t C1, int64_t C2, int64_t Hd,
                      int64_t Cc, float *Wc1, float *bc1, float *Wc2, float *bc2, float *Wl1, float *bl1, float *Wl2,
                      float *bl2, float lr, float *loss, float *gWc1, float *gbc1, float *gWc2, float *gbc2,
                      float *gWl1, float *gbl1, float *gWl2, float *gbl2, float *logits)
{
    return guarded([&] {
        int64_t Fdim = C2 * (S / 4) * (S / 4);
        Sequential model;
        model.add(std::make_unique<nn::Conv2d>(1, (int)C1, 3, 1, 1, true));
        model.add(std::make_unique<nn::ReLU>());
        model.add(std::make_unique<nn::MaxPool2d>(2, 2, 0));
        model.add(std::make_unique<nn::Conv2d>((int)C1, (int)C2, 3, 1, 1, true));
        model.add(std::make_unique<nn::ReLU>());
        model.add(std::make_unique<nn::MaxPool2d>(2, 2, 0));
        model.add(std::make_unique<nn::Flatten>());
        model.add(std::make_unique<nn::Linear>((int)Fdim, (int)Hd, true));
        model.add(std::make_unique<nn::ReLU>());
        model.add(std::make_unique<nn::Linear>((int)Hd, (int)Cc, true));
        auto &c1 = dynamic_cast<nn::Conv2d &>(model[0]);
        auto &c2 = dynamic_cast<nn::Conv2d &>(model[3]);
        auto &l1 = dynamic_cast<nn::Linear &>(model[7]);
        auto &l2 = dynamic_cast<nn::Linear &>(model[9]);
        SGD opt(model, lr);
        *c1.weight() = Parameter(f32(Wc1, Shape{(size_t)C1, 1, 3, 3}, true));
        *c1.bias()   = Parameter(f32(bc1, Shape{(size_t)C1}, true));
        *c2.weight() = Parameter(f32(Wc2, Shape{(size_t)C2, (size_t)C1, 3, 3}, true));
        *c2.bias()   = Parameter(f32(bc2, Shape{(size_t)C2}, true));
        *l1.weight() = Parameter(f32(Wl1, Shape{(size_t)Fdim, (size_t)Hd}, true));
        *l1.bias()   = Parameter(f32(bl1, Shape{1, (size_t)Hd}, true));
        *l2.weight() = Parameter(f32(Wl2, Shape{(size_t)Hd, (size_t)Cc}, true));
        *l2.bias()   = Parameter(f32(bl2, Shape{1, (size_t)Cc}, true));
        auto X = f32(x, Shape{(size_t)N, 1, (size_t)S, (size_t)S});
        auto T = labels(t, is64, N);
        model.train();
        opt.zero_grad();
        auto y = model(X);
        auto L = F::softmax_cross_entropy(y, T);
        L.backward();
        *loss = L.item<float>();
        out(y, logits);
        out(c1.weight()->grad(), gWc1);
        out(c1.bias()->grad(), gbc1);
        out(c2.weight()->grad(), gWc2);
        out(c2.bias()->grad(), gbc2);
        out(l1.weight()->grad(), gWl1);
        out(l1.bias()->grad(), gbl1);
        out(l2.weight()->grad(), gWl2);
        out(l2.bias()->grad(), gbl2);
        opt.step();
        out(*c1.weight(), Wc1);
        out(*c1.bias(), bc1);
        out(*c2.weight(), Wc2);
        out(*c2.bias(), bc2);
        out(*l1.weight(), Wl1);
        out(*l1.bias(), bl1);
        out(*l2.weight(), Wl2);
        out(*l2.bias(), bl2);
    });
}

}  // extern "C"

// ---- whole training steps timed on resident tensors (benchmark configs 1 and 4): `warmup` untimed steps, then
// `steps` timed ones; every step ends with the loss read back to the host (as the reference's loop does), which
// also drains the device queue, so wall-clock time around the loop is the step time.
namespace
{
std::vector<float> uniform_vec(std::mt19937 &gen, size_t n, float lo, float hi)
{
    std::uniform_real_distribution<float> d(lo, hi);
    std::vector<float> v(n);
    for (auto &e : v)
        e = d(gen);
    return v;
}

Parameter kaiming_uniform(std::mt19937 &gen, const Shape &s, size_t fan_in)
{
    const float bound = std::sqrt(6.0f / (float)fan_in);
    return Parameter(Tensor(uniform_vec(gen, s.elements(), -bound, bound), s,
                            dtype(DataType::kFloat32).requires_grad(true).device(kDev)));
}

Parameter zeros_param(const Shape &s)
{
    return Parameter(Tensor(std::vector<float>(s.elements(), 0.0f), s,
                            dtype(DataType::kFloat32).requires_grad(true).device(kDev)));
}

template <typename Model, typename Opt>
void timed_steps(Model &model, Opt &opt, const Tensor &X, const Tensor &T, int steps, int warmup, float *ms, float *loss)
{
    model.train();
    auto one = [&] {
        opt.zero_grad();
        // a new handle on the batch every step, as a data loader hands out new tensors (mlp_mnist.cpp's loop): the
        // gradients the step leaves on its inputs are assigned, not accumulated over the steps
        const Tensor x = X.detach(), t = T.detach();
        auto y = model(x);
        auto L = F::softmax_cross_entropy(y, t);
        L.backward();
        opt.step();
        return L.template item<float>();
    };
    // loss[0]: the loss of the first step taken from the initial parameters (the same number whichever way the steps
    // are run afterwards, so the runs can be compared); loss[1]: the loss of the last step
    bool first = true;
    auto note = [&](float v) {
        if (first)
            loss[0] = v;
        first   = false;
        loss[1] = v;
    };
    for (int i = 0; i < warmup; ++i)
        note(one());
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < steps; ++i)
        note(one());
    // the parameters of the last step are still in flight: reading the smallest one back drains the queue
    // (a large one would add its own copy time to the steps)
    auto params = model.parameters();
    auto *smallest = params[0];
    for (auto *p : params)
        if (p->shape().elements() < smallest->shape().elements())
            smallest = p;
    float sink = smallest->template to_vector<float>()[0];
    (void)sink;
    const auto t1 = std::chrono::steady_clock::now();
    *ms = std::chrono::duration<float, std::milli>(t1 - t0).count() / (float)(steps > 0 ? steps : 1);
}

#ifdef DRV_ON_DEVICE
// The same step recorded once into a graph and replayed (this backend only: the reference has no streams or
// graphs). Two ordinary steps first (memory pool warm, optimizer buffers made), then the capture, then `steps`
// replays; the loss is read back after every replay when read_loss != 0, as the loop above does, or once at the end.

template <typename Model, typename Opt>
void timed_graph_steps(Model &model, Opt &opt, const Tensor &X, const Tensor &T, int steps, int warmup, int read_loss,
                       float *ms, float *loss)
{
    StreamScope stream;
    model.train();
    for (int i = 0; i < (warmup > 2 ? warmup : 2); ++i)
    {
        opt.zero_grad();
        auto L = F::softmax_cross_entropy(model(X.detach()), T.detach());  // new handles on the batch, as in timed_steps
        L.backward();
        opt.step();
        loss[1] = L.template item<float>();
        if (i == 0)
            loss[0] = loss[1];  // the first step from the initial parameters, as in timed_steps
    }
    origin::cuda::Graph graph;
    Tensor L;
    graph.begin_capture();
    opt.zero_grad();
    L = F::softmax_cross_entropy(model(X.detach()), T.detach());
    L.backward();
    opt.step();
    graph.end_capture();
    for (int i = 0; i < 2; ++i)  // untimed replays
    {
        opt.prepare_replay();
        graph.launch();
    }
    loss[1] = L.template item<float>();
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < steps; ++i)
    {
        opt.prepare_replay();
        graph.launch();
        if (read_loss)
            loss[1] = L.template item<float>();
    }
    loss[1] = L.template item<float>();  // synchronises: every replay is complete
    const auto t1 = std::chrono::steady_clock::now();
    *ms = std::chrono::duration<float, std::milli>(t1 - t0).count() / (float)(steps > 0 ? steps : 1);
}
#endif
}  // namespace

extern "C" {

}  // extern "C"

namespace
{
// graph_mode 0: ordinary steps; 1: a recorded step replayed, loss read back every step; 2: read back at the end only
template <typename Model, typename Opt>
void run_timed(Model &model, Opt &opt, const Tensor &X, const Tensor &T, int steps, int warmup, int graph_mode, float *ms,
               float *loss)
{
#ifdef DRV_ON_DEVICE
    if (graph_mode != 0)
        return timed_graph_steps(model, opt, X, T, steps, warmup, graph_mode == 1, ms, loss);
#endif
    if (graph_mode != 0)
        throw std::runtime_error("graph replay is only available on the device build of this driver");
    timed_steps(model, opt, X, T, steps, warmup, ms, loss);
}

int mlp_bench_impl(int64_t N, int64_t D, int64_t Hd, int64_t C, int steps, int warmup, int graph_mode, float *ms_per_step,
                   float *loss)
{
    return guarded([&] {
        std::mt19937 gen(1234);
        Sequential model;
        model.add(std::make_unique<nn::Linear>((int)D, (int)Hd, true));
        model.add(std::make_unique<nn::ReLU>());
        model.add(std::make_unique<nn::Linear>((int)Hd, (int)C, true));
        auto &l1 = dynamic_cast<nn::Linear &>(model[0]);
        auto &l2 = dynamic_cast<nn::Linear &>(model[2]);
        Adam opt(model, 1e-3f, 0.9f, 0.999f, 1e-8f);
        opt.register_hook(WeightDecay(1e-4f).hook());
        *l1.weight() = kaiming_uniform(gen, Shape{(size_t)D, (size_t)Hd}, (size_t)D);
        *l1.bias()   = zeros_param(Shape{1, (size_t)Hd});
        *l2.weight() = kaiming_uniform(gen, Shape{(size_t)Hd, (size_t)C}, (size_t)Hd);
        *l2.bias()   = zeros_param(Shape{1, (size_t)C});
        auto X = Tensor(uniform_vec(gen, (size_t)(N * D), 0.0f, 1.0f), Shape{(size_t)N, (size_t)D},
                        dtype(DataType::kFloat32).device(kDev));
        std::vector<int64_t> tv((size_t)N);
        for (auto &e : tv)
            e = (int64_t)(gen() % (uint32_t)C);
        auto T = Tensor(tv, Shape{(size_t)N}, dtype(DataType::kInt64).device(kDev));
        run_timed(model, opt, X, T, steps, warmup, graph_mode, ms_per_step, loss);
    });
}

// The same step with the network built as the reference's own loop builds it (tests/example/mnist/mlp_mnist.cpp:227):
// one nn::MLP({D, Hd, C}) object instead of a Sequential of layers. Same seed, same draws in the same order, so the
// first step's loss is the Sequential's.
int mlp_model_bench_impl(int64_t N, int64_t D, int64_t Hd, int64_t C, int steps, int warmup, int graph_mode,
                         float *ms_per_step, float *loss)
{
    return guarded([&] {
        std::mt19937 gen(1234);
        nn::MLP model({(int)D, (int)Hd, (int)C});
        Adam opt(model, 1e-3f, 0.9f, 0.999f, 1e-8f);
        opt.register_hook(WeightDecay(1e-4f).hook());
        auto named = model.named_parameters("");
        *named.at("layer_0.weight") = kaiming_uniform(gen, Shape{(size_t)D, (size_t)Hd}, (size_t)D);
        *named.at("layer_0.bias")   = zeros_param(Shape{1, (size_t)Hd});
        *named.at("layer_1.weight") = kaiming_uniform(gen, Shape{(size_t)Hd, (size_t)C}, (size_t)Hd);
        *named.at("layer_1.bias")   = zeros_param(Shape{1, (size_t)C});
        auto X = Tensor(uniform_vec(gen, (size_t)(N * D), 0.0f, 1.0f), Shape{(size_t)N, (size_t)D},
                        dtype(DataType::kFloat32).device(kDev));
        std::vector<int64_t> tv((size_t)N);
        for (auto &e : tv)
            e = (int64_t)(gen() % (uint32_t)C);
        auto T = Tensor(tv, Shape{(size_t)N}, dtype(DataType::kInt64).device(kDev));
        run_timed(model, opt, X, T, steps, warmup, graph_mode, ms_per_step, loss);
    });
}

int cnn_bench_impl(int64_t N, int steps, int warmup, int graph_mode, float *ms_per_step, float *loss)
{
    return guarded([&] {
        std::mt19937 gen(4321);
        const int64_t S = 28, C1 = 32, C2 = 64, Hd = 128, Cc = 10, Fdim = C2 * 7 * 7;
        Sequential model;
        model.add(std::make_unique<nn::Conv2d>(1, (int)C1, 3, 1, 1, true));
        model.add(std::make_unique<nn::ReLU>());
        model.add(std::make_unique<nn::MaxPool2d>(2, 2, 0));
        model.add(std::make_unique<nn::Conv2d>((int)C1, (int)C2, 3, 1, 1, true));
        model.add(std::make_unique<nn::ReLU>());
        model.add(std::make_unique<nn::MaxPool2d>(2, 2, 0));
        model.add(std::make_unique<nn::Flatten>());
        model.add(std::make_unique<nn::Linear>((int)Fdim, (int)Hd, true));
        model.add(std::make_unique<nn::ReLU>());
        model.add(std::make_unique<nn::Linear>((int)Hd, (int)Cc, true));
        auto &c1 = dynamic_cast<nn::Conv2d &>(model[0]);
        auto &c2 = dynamic_cast<nn::Conv2d &>(model[3]);
        auto &l1 = dynamic_cast<nn::Linear &>(model[7]);
        auto &l2 = dynamic_cast<nn::Linear &>(model[9]);
        SGD opt(model, 0.01f);
        *c1.weight() = kaiming_uniform(gen, Shape{(size_t)C1, 1, 3, 3}, 9);
        *c1.bias()   = zeros_param(Shape{(size_t)C1});
        *c2.weight() = kaiming_uniform(gen, Shape{(size_t)C2, (size_t)C1, 3, 3}, (size_t)(9 * C1));
        *c2.bias()   = zeros_param(Shape{(size_t)C2});
        *l1.weight() = kaiming_uniform(gen, Shape{(size_t)Fdim, (size_t)Hd}, (size_t)Fdim);
        *l1.bias()   = zeros_param(Shape{1, (size_t)Hd});
        *l2.weight() = kaiming_uniform(gen, Shape{(size_t)Hd, (size_t)Cc}, (size_t)Hd);
        *l2.bias()   = zeros_param(Shape{1, (size_t)Cc});
        auto X = Tensor(uniform_vec(gen, (size_t)(N * S * S), 0.0f, 1.0f), Shape{(size_t)N, 1, (size_t)S, (size_t)S},
                        dtype(DataType::kFloat32).device(kDev));
        std::vector<int64_t> tv((size_t)N);
        for (auto &e : tv)
            e = (int64_t)(gen() % (uint32_t)Cc);
        auto T = Tensor(tv, Shape{(size_t)N}, dtype(DataType::kInt64).device(kDev));
        run_timed(model, opt, X, T, steps, warmup, graph_mode, ms_per_step, loss);
    });
}
}  // namespace

extern "C" {
#ifdef DRV_ON_DEVICE
// A Linear, Conv2d or BatchNorm2d that a ReLU follows inside a Sequential runs as one operator (Conv2d, ReLU, MaxPool2d
// as one too). The same network, the same input:
// once through the Sequential, once module by module (nothing paired). diffs[0] counts output elements that differ in
// any bit, diffs[1] the same over the gradients of all parameters and of the input.
int DRV(paired_layers_match_separate_modules)(int64_t N, int64_t *diffs)
{
    return guarded([&] {
        std::mt19937 gen(99);
        Sequential model;
        model.add(std::make_unique<nn::Conv2d>(3, 32, 3, 1, 1, true));
        model.add(std::make_unique<nn::ReLU>());
        model.add(std::make_unique<nn::MaxPool2d>(2, 2, 0));
        model.add(std::make_unique<nn::Conv2d>(32, 32, 3, 1, 1, true));
        model.add(std::make_unique<nn::BatchNorm2d>(32));
        model.add(std::make_unique<nn::ReLU>());
        model.add(std::make_unique<nn::Flatten>());
        model.add(std::make_unique<nn::Linear>(32 * 8 * 8, 100, true));
        model.add(std::make_unique<nn::ReLU>());
        model.add(std::make_unique<nn::Linear>(100, 10, true));
        *dynamic_cast<nn::Conv2d &>(model[0]).weight() = kaiming_uniform(gen, Shape{32, 3, 3, 3}, 27);
        *dynamic_cast<nn::Conv2d &>(model[3]).weight() = kaiming_uniform(gen, Shape{32, 32, 3, 3}, 288);
        // scale and shift away from 1 and 0, so that the ReLU's mask depends on both
        *dynamic_cast<nn::BatchNorm2d &>(model[4]).weight() = kaiming_uniform(gen, Shape{32}, 3);
        *dynamic_cast<nn::BatchNorm2d &>(model[4]).bias() = kaiming_uniform(gen, Shape{32}, 24);
        *dynamic_cast<nn::Linear &>(model[7]).weight() = kaiming_uniform(gen, Shape{32 * 8 * 8, 100}, 32 * 8 * 8);
        *dynamic_cast<nn::Linear &>(model[9]).weight() = kaiming_uniform(gen, Shape{100, 10}, 100);
        model.to(kDev);
        model.train();
        auto xv = uniform_vec(gen, (size_t)(N * 3 * 16 * 16), -1.0f, 1.0f);
        std::vector<int64_t> tv((size_t)N);
        for (auto &e : tv)
            e = (int64_t)(gen() % 10u);
        auto T = Tensor(tv, Shape{(size_t)N}, dtype(DataType::kInt64).device(kDev));
        auto run = [&](bool paired, std::vector<std::vector<float>> &out) {
            auto X = Tensor(xv, Shape{(size_t)N, 3, 16, 16}, dtype(DataType::kFloat32).device(kDev).requires_grad(true));
            for (auto *p : model.parameters())
                p->clear_grad();
            Tensor y = X;
            if (paired)
                y = model(X);
            else
                for (size_t i = 0; i < model.size(); ++i)
                    y = model[i].forward(y);
            auto L = F::softmax_cross_entropy(y, T);
            L.backward();
            out.push_back(y.to_vector<float>());
            out.push_back(X.grad().to_vector<float>());
            for (auto *p : model.parameters())
                out.push_back(p->grad().to_vector<float>());
        };
        std::vector<std::vector<float>> a, b;
        run(true, a);
        run(false, b);
        diffs[0] = diffs[1] = 0;
        for (size_t k = 0; k < a.size(); ++k)
        {
            if (a[k].size() != b[k].size())
                throw std::runtime_error("paired and separate runs gave tensors of different sizes");
            for (size_t i = 0; i < a[k].size(); ++i)
                diffs[k == 0 ? 0 : 1] += std::memcmp(&a[k][i], &b[k][i], sizeof(float)) != 0;
        }
    });
}
#endif

#ifdef DRV_ON_DEVICE
// zeros / ones / full on the device queue their fill kernel only when the buffer is first asked for. What must hold:
// out[0] the sum of a ones tensor that went to the host untouched (n); out[1] an accumulator made with zeros BEFORE a
// capture and first touched inside it, after three replays of `acc += ones` (3 in every element: its fill ran before
// the capture and is not part of the replays), read as the sum / n; out[2] the sum of zeros + zeros added in place,
// neither written before (0); out[3] element 0 of -0.0f filled then added to zeros (+0.0, sign bit clear -> 0, the
// addition may not be skipped); out[4] x.grad of sum(x * full(2.5)) (2.5 * n) / n.
int DRV(pending_fill_semantics)(int64_t n, double *out)
{
    return guarded([&] {
        StreamScope stream;
        const auto opt = dtype(DataType::kFloat32).device(kDev);
        const Shape shp{(size_t)n};
        auto total = [](const Tensor &t) {
            double s = 0;
            for (float v : t.to_vector<float>())
                s += v;
            return s;
        };
        out[0] = total(Tensor::ones(shp, opt).to(Device(DeviceType::kCPU)));
        {
            Tensor acc = Tensor::zeros(shp, opt), one = Tensor::ones(shp, opt);
            one.to_vector<float>();  // written now
            origin::cuda::Graph graph;
            graph.begin_capture();
            acc += one;
            graph.end_capture();
            for (int i = 0; i < 3; ++i)
                graph.launch();
            out[1] = total(acc) / (double)n;
        }
        {
            Tensor a = Tensor::zeros(shp, opt), b = Tensor::zeros(shp, opt);
            a += b;
            out[2] = total(a);
        }
        {
            Tensor a = Tensor::full(shp, -0.0f, opt), b = Tensor::zeros(shp, opt);
            a += b;
            const float v = a.to_vector<float>()[0];
            uint32_t bits;
            std::memcpy(&bits, &v, sizeof(bits));
            out[3] = (double)(bits >> 31);
        }
        {
            std::vector<float> h((size_t)n, 1.0f);
            Tensor x = f32(h.data(), shp, true);
            auto y = F::sum(x * Tensor::full(shp, 2.5f, opt));
            y.backward();
            out[4] = total(x.grad()) / (double)n;
        }
    });
}
#endif

int DRV(mlp_bench)(int64_t N, int64_t D, int64_t Hd, int64_t C, int steps, int warmup, float *ms_per_step, float *loss)
{
    return mlp_bench_impl(N, D, Hd, C, steps, warmup, 0, ms_per_step, loss);
}

// graph_mode: 0 ordinary steps; 1 / 2: a recorded step replayed (device build of this repository's host layer only)
int DRV(mlp_model_bench)(int64_t N, int64_t D, int64_t Hd, int64_t C, int steps, int warmup, int graph_mode,
                         float *ms_per_step, float *loss)
{
    return mlp_model_bench_impl(N, D, Hd, C, steps, warmup, graph_mode, ms_per_step, loss);
}

int DRV(cnn_bench)(int64_t N, int steps, int warmup, float *ms_per_step, float *loss)
{
    return cnn_bench_impl(N, steps, warmup, 0, ms_per_step, loss);
}

#ifdef DRV_ON_DEVICE
// The network of the reference's own tests/example/mnist/conv_mnist.cpp:16-104 (conv 1->64, BatchNorm, ReLU, pool,
// conv 64->128, BatchNorm, ReLU, pool, 6272->128->10) with its optimizer (Adam 1e-4 + WeightDecay), on a fixed
// synthetic batch. Device build only: the reference cannot run this step (its BatchNorm operator throws in
// backward). losses[0] / losses[1] = the loss before training and at the last step: training must bring it down;
// losses[2] = the loss of an evaluation-mode forward afterwards (it uses the running statistics the steps folded).
int DRV(cnn_bn_bench)(int64_t N, int steps, int warmup, int graph_mode, float *ms_per_step, float *losses)
{
    return guarded([&] {
        std::mt19937 gen(777);
        Sequential model;
        model.add(std::make_unique<nn::Conv2d>(1, 64, 3, 1, 1, true));
        model.add(std::make_unique<nn::BatchNorm2d>(64));
        model.add(std::make_unique<nn::ReLU>());
        model.add(std::make_unique<nn::MaxPool2d>(2, 2, 0));
        model.add(std::make_unique<nn::Conv2d>(64, 128, 3, 1, 1, true));
        model.add(std::make_unique<nn::BatchNorm2d>(128));
        model.add(std::make_unique<nn::ReLU>());
        model.add(std::make_unique<nn::MaxPool2d>(2, 2, 0));
        model.add(std::make_unique<nn::Flatten>());
        model.add(std::make_unique<nn::Linear>(7 * 7 * 128, 128, true));
        model.add(std::make_unique<nn::ReLU>());
        model.add(std::make_unique<nn::Linear>(128, 10, true));
        *dynamic_cast<nn::Conv2d &>(model[0]).weight() = kaiming_uniform(gen, Shape{64, 1, 3, 3}, 9);
        *dynamic_cast<nn::Conv2d &>(model[4]).weight() = kaiming_uniform(gen, Shape{128, 64, 3, 3}, 9 * 64);
        *dynamic_cast<nn::Linear &>(model[9]).weight() = kaiming_uniform(gen, Shape{6272, 128}, 6272);
        *dynamic_cast<nn::Linear &>(model[11]).weight() = kaiming_uniform(gen, Shape{128, 10}, 128);
        model.to(kDev);
        Adam opt(model, 1e-4f);
        opt.register_hook(WeightDecay(1e-4f).hook());
        auto X = Tensor(uniform_vec(gen, (size_t)(N * 28 * 28), 0.0f, 1.0f), Shape{(size_t)N, 1, 28, 28},
                        dtype(DataType::kFloat32).device(kDev));
        std::vector<int64_t> tv((size_t)N);
        for (auto &e : tv)
            e = (int64_t)(gen() % 10u);
        auto T = Tensor(tv, Shape{(size_t)N}, dtype(DataType::kInt64).device(kDev));
        model.train();
        {
            auto guard = no_grad();
            losses[0] = F::softmax_cross_entropy(model(X), T).item<float>();
        }
        float first_last[2] = {0.0f, 0.0f};
        run_timed(model, opt, X, T, steps, warmup, graph_mode, ms_per_step, first_last);
        losses[1] = first_last[1];
        model.eval();
        auto guard = no_grad();
        losses[2] = F::softmax_cross_entropy(model(X), T).item<float>();
    });
}

int DRV(mlp_bench_graph)(int64_t N, int64_t D, int64_t Hd, int64_t C, int steps, int warmup, int read_loss_each_step,
                         float *ms_per_step, float *loss)
{
    return mlp_bench_impl(N, D, Hd, C, steps, warmup, read_loss_each_step ? 1 : 2, ms_per_step, loss);
}

int DRV(cnn_bench_graph)(int64_t N, int steps, int warmup, int read_loss_each_step, float *ms_per_step, float *loss)
{
    return cnn_bench_impl(N, steps, warmup, read_loss_each_step ? 1 : 2, ms_per_step, loss);
}
#endif
}  // extern "C"
