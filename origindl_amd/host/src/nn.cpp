// Host glue above the operators: modules, layers, optimizers, device API (see origin/nn.h).
#include "origin/nn.h"

#include <typeinfo>

#include <cmath>
#include <random>

#include "odl_hip.h"

namespace origin
{
// ------------------------------------------------------------------------------------------- Module
std::vector<Parameter *> Module::parameters()
{
    std::vector<Parameter *> out;
    for (auto &p : parameters_)
        out.push_back(p.second);
    for (auto &m : modules_)
        for (auto *p : m.second->parameters())
            out.push_back(p);
    return out;
}

void Module::register_parameter(const std::string &name, Parameter &param)
{
    parameters_.emplace_back(name, &param);
}

void Module::register_module(const std::string &name, std::unique_ptr<Module> module)
{
    modules_.emplace_back(name, std::move(module));
}

void Module::train(bool mode)
{
    training_ = mode;
    for (auto &m : modules_)
        m.second->train(mode);
}

void Module::to(Device device)
{
    for (auto *p : parameters())
        if (p->defined() && p->device() != device)
        {
            Tensor moved = static_cast<const Tensor &>(*p).to(device);
            moved.impl_->requires_grad_ = true;
            *p = moved;
        }
}

void Module::zero_grad()
{
    for (auto *p : parameters())
        p->clear_grad();
}

std::unordered_map<std::string, Parameter *> Module::named_parameters(const std::string &prefix)
{
    std::unordered_map<std::string, Parameter *> named;
    for (auto &p : parameters_)
        named[prefix.empty() ? p.first : prefix + "." + p.first] = p.second;
    for (auto &m : modules_)
    {
        auto sub = m.second->named_parameters(prefix.empty() ? m.first : prefix + "." + m.first);
        named.insert(sub.begin(), sub.end());
    }
    return named;
}

std::unordered_map<std::string, const Parameter *> Module::named_parameters(const std::string &prefix) const
{
    std::unordered_map<std::string, const Parameter *> named;
    for (auto &p : const_cast<Module *>(this)->named_parameters(prefix))
        named[p.first] = p.second;
    return named;
}

Module::StateDict Module::state_dict() const
{
    StateDict sd;
    for (auto &p : named_parameters(""))
        sd[p.first] = static_cast<const Tensor &>(*p.second);
    return sd;
}

void Module::load_state_dict(const StateDict &state_dict, bool strict)
{
    std::unordered_map<std::string, bool> loaded;
    for (auto &[name, param] : named_parameters())
    {
        auto it = state_dict.find(name);
        if (it != state_dict.end())
        {
            if (param->shape() != it->second.shape())
                THROW_RUNTIME_ERROR("Shape mismatch for parameter '{}': expected {}, got {}", name,
                                    param->shape().to_string(), it->second.shape().to_string());
            *param = Parameter(it->second);
            loaded[name] = true;
        }
        else if (strict)
            THROW_RUNTIME_ERROR("Missing parameter '{}' in state_dict (strict mode)", name);
    }
    if (strict)
        for (const auto &kv : state_dict)
            if (!loaded.count(kv.first))
                THROW_RUNTIME_ERROR("Unexpected parameter '{}' in state_dict (strict mode)", kv.first);
}

void Module::load(const std::string &filepath, bool strict)
{
    load_state_dict(origin::load(filepath), strict);
}

namespace nn
{
BatchNormBase::BatchNormBase(const char *name, int num_dims, int num_features, float eps, float momentum)
    : name_(name), num_dims_(num_dims), num_features_(num_features), eps_(eps), momentum_(momentum)
{
    if (num_features <= 0)
        THROW_INVALID_ARG("{}: num_features must be positive, but got {}", name, num_features);
    reset_parameters();
    register_parameter("weight", gamma_);
    register_parameter("bias", beta_);
}

void BatchNormBase::reset_parameters()
{
    const Shape s{static_cast<size_t>(num_features_)};
    gamma_ = Parameter(Tensor::ones(s, TensorOptions(DataType::kFloat32).requires_grad(true)));
    beta_ = Parameter(Tensor::zeros(s, TensorOptions(DataType::kFloat32).requires_grad(true)));
    running_mean_ = Tensor::zeros(s, TensorOptions(DataType::kFloat32));
    running_var_ = Tensor::ones(s, TensorOptions(DataType::kFloat32));
}

void BatchNormBase::to(Device device)
{
    Module::to(device);
    if (running_mean_.device() != device)
        running_mean_ = running_mean_.to(device);
    if (running_var_.device() != device)
        running_var_ = running_var_.to(device);
}

Tensor BatchNormBase::forward(const Tensor &input)
{
    return run(input, false);
}

Tensor BatchNormBase::forward_relu(const Tensor &input)
{
    if (input.device().type() != DeviceType::kCUDA || input.dtype() != DataType::kFloat32)
        return functional::relu(run(input, false));
    return run(input, true);
}

Tensor BatchNormBase::run(const Tensor &input, bool relu)
{
    const Shape s = input.shape();
    if (s.size() != static_cast<size_t>(num_dims_))
        THROW_RUNTIME_ERROR("{} forward: input must be {}, but got shape {}", name_,
                            num_dims_ == 4 ? "4D (N, C, H, W)" : "2D (N, C)", s.to_string());
    if (s[1] != static_cast<size_t>(num_features_))
        THROW_RUNTIME_ERROR("{} forward: input feature size {} does not match num_features {}", name_, s[1],
                            num_features_);
    auto outs = (relu ? functional::batch_norm_relu_outputs : functional::batch_norm_outputs)(
        input, static_cast<const Tensor &>(gamma_), static_cast<const Tensor &>(beta_), running_mean_, running_var_,
        is_training(), eps_, momentum_, num_dims_);
    if (is_training() && outs.size() >= 3)
    {
        auto fold = [&](const Tensor &running, const Tensor &batch) {
            const auto &r = static_cast<const OriginMat &>(*running.impl_->data_);
            return Tensor(r.axpby(momentum_, 1.0f - momentum_, *batch.impl_->data_));
        };
        if (cuda::is_capturing())
        {
            // a recorded step must find the statistics at the same address on every replay
            static_cast<OriginMat &>(*running_mean_.impl_->data_).axpby_inplace(momentum_, 1.0f - momentum_, *outs[1].impl_->data_);
            static_cast<OriginMat &>(*running_var_.impl_->data_).axpby_inplace(momentum_, 1.0f - momentum_, *outs[2].impl_->data_);
        }
        else
        {
            running_mean_ = fold(running_mean_, outs[1]);
            running_var_ = fold(running_var_, outs[2]);
        }
    }
    return outs[0];
}
}  // namespace nn

Tensor Sequential::forward(const Tensor &input)
{
    // A Linear, Conv2d or batch normalisation that a ReLU follows runs together with it (the tensor between the two is not visible from
    // outside a Sequential); the values are those of the two modules run in turn.
    Tensor x = input;
    for (size_t i = 0; i < layers_.size(); ++i)
    {
        Module &l = *layers_[i];
        if (i + 1 < layers_.size() && typeid(*layers_[i + 1]) == typeid(nn::ReLU))
        {
            if (typeid(l) == typeid(nn::Linear))
            {
                x = static_cast<nn::Linear &>(l).forward_relu(x);
                ++i;
                continue;
            }
            if (typeid(l) == typeid(nn::BatchNorm2d) || typeid(l) == typeid(nn::BatchNorm1d))
            {
                x = static_cast<nn::BatchNormBase &>(l).forward_relu(x);
                ++i;
                continue;
            }
            if (typeid(l) == typeid(nn::Conv2d))
            {
                if (i + 2 < layers_.size() && typeid(*layers_[i + 2]) == typeid(nn::MaxPool2d))
                {
                    // ... and a MaxPool2d after the pair joins it: its gradient is masked by the ReLU as it is written
                    const auto &pool = static_cast<const nn::MaxPool2d &>(*layers_[i + 2]);
                    x = static_cast<nn::Conv2d &>(l).forward_relu_pool(x, pool.kernel_size(), pool.stride(), pool.pad());
                    i += 2;
                    continue;
                }
                x = static_cast<nn::Conv2d &>(l).forward_relu(x);
                ++i;
                continue;
            }
        }
        x = l.forward(x);
    }
    return x;
}

std::vector<Parameter *> Sequential::parameters()
{
    std::vector<Parameter *> out;
    for (auto &l : layers_)
        for (auto *p : l->parameters())
            out.push_back(p);
    return out;
}

void Sequential::to(Device device)
{
    for (auto &l : layers_)
        l->to(device);
}

// ------------------------------------------------------------------------------------------- layers
namespace
{
// randn * scale generated on the host (parameter initialisation is not a device kernel of this backend)
Parameter scaled_randn(const Shape &shape, float scale)
{
    static std::mt19937 gen{std::random_device{}()};
    std::normal_distribution<float> dist(0.f, 1.f);
    std::vector<float> host(shape.elements());
    for (auto &v : host)
        v = dist(gen) * scale;
    return Parameter(Tensor(host, shape, dtype(DataType::kFloat32).requires_grad(true)));
}
}  // namespace

namespace nn
{
Linear::Linear(int in_features, int out_features, bool bias)
    : in_features_(in_features), out_features_(out_features), use_bias_(bias)
{
    reset_parameters();
    register_parameter("weight", weight_);
    if (use_bias_)
        register_parameter("bias", bias_);
}

void Linear::reset_parameters()
{
    weight_ = scaled_randn(Shape{(size_t)in_features_, (size_t)out_features_}, std::sqrt(1.0f / (float)in_features_));
    if (use_bias_)
        bias_ = Parameter(Tensor::zeros(Shape{1, (size_t)out_features_}, dtype(DataType::kFloat32).requires_grad(true)));
}

Tensor Linear::forward(const Tensor &input)
{
    if (weight_.shape().elements() == 0)
        THROW_RUNTIME_ERROR("Weight is empty in forward! weight_.shape() = {}", weight_.shape().to_string());
    if (use_bias_ && input.shape().size() == 2 && input.device().type() == DeviceType::kCUDA)
        return functional::linear(input, static_cast<const Tensor &>(weight_), static_cast<const Tensor &>(bias_));
    auto output = functional::mat_mul(input, static_cast<const Tensor &>(weight_));
    if (use_bias_)
        output = output + functional::broadcast_to(bias_, output.shape());  // src/nn/layers/linear.cpp:96-102
    return output;
}

Tensor Linear::forward_relu(const Tensor &input)
{
    if (weight_.shape().elements() != 0 && use_bias_ && input.shape().size() == 2 &&
        input.device().type() == DeviceType::kCUDA && input.dtype() == DataType::kFloat32)
        return functional::linear_relu(input, static_cast<const Tensor &>(weight_), static_cast<const Tensor &>(bias_));
    return functional::relu(forward(input));
}

Conv2d::Conv2d(int in_channels, int out_channels, std::pair<int, int> kernel_size, std::pair<int, int> stride,
               std::pair<int, int> pad, bool bias)
    : in_channels_(in_channels), out_channels_(out_channels), kernel_(kernel_size), stride_(stride), pad_(pad),
      use_bias_(bias)
{
    if (in_channels <= 0)
        THROW_INVALID_ARG("Conv2d: in_channels must be positive, but got {}", in_channels);
    if (out_channels <= 0)
        THROW_INVALID_ARG("Conv2d: out_channels must be positive, but got {}", out_channels);
    if (kernel_size.first <= 0 || kernel_size.second <= 0)
        THROW_INVALID_ARG("Conv2d: kernel_size must be positive, but got ({}, {})", kernel_size.first, kernel_size.second);
    if (stride.first <= 0 || stride.second <= 0)
        THROW_INVALID_ARG("Conv2d: stride must be positive, but got ({}, {})", stride.first, stride.second);
    if (pad.first < 0 || pad.second < 0)
        THROW_INVALID_ARG("Conv2d: pad must be non-negative, but got ({}, {})", pad.first, pad.second);
    const float fan_in = (float)(in_channels * kernel_.first * kernel_.second);
    weight_ = scaled_randn(Shape{(size_t)out_channels, (size_t)in_channels, (size_t)kernel_.first, (size_t)kernel_.second},
                           std::sqrt(2.0f / fan_in));
    register_parameter("weight", weight_);
    if (use_bias_)
    {
        bias_ = Parameter(Tensor::zeros(Shape{(size_t)out_channels}, dtype(DataType::kFloat32).requires_grad(true)));
        register_parameter("bias", bias_);
    }
}

Conv2d::Conv2d(int in_channels, int out_channels, int kernel_size, int stride, int pad, bool bias)
    : Conv2d(in_channels, out_channels, pair(kernel_size), pair(stride), pair(pad), bias)
{}

Tensor Conv2d::forward(const Tensor &input)
{
    if (input.shape().size() != 4)
        THROW_RUNTIME_ERROR("Conv2d forward: input must be 4D (N, C, H, W), but got shape {}", input.shape().to_string());
    if (input.shape()[1] != (size_t)in_channels_)
        THROW_RUNTIME_ERROR("Conv2d forward: input channel mismatch - input has {} channels, but layer expects {} channels",
                            input.shape()[1], in_channels_);
    const Tensor *b = use_bias_ ? &static_cast<const Tensor &>(bias_) : nullptr;
    return functional::conv2d(input, static_cast<const Tensor &>(weight_), b, stride_, pad_);
}

Tensor Conv2d::forward_relu(const Tensor &input)
{
    if (input.shape().size() != 4 || input.shape()[1] != (size_t)in_channels_ ||
        input.device().type() != DeviceType::kCUDA || input.dtype() != DataType::kFloat32)
        return functional::relu(forward(input));
    const Tensor *b = use_bias_ ? &static_cast<const Tensor &>(bias_) : nullptr;
    return functional::conv2d_relu(input, static_cast<const Tensor &>(weight_), b, stride_, pad_);
}

Tensor Conv2d::forward_relu_pool(const Tensor &input, std::pair<int, int> pool_kernel, std::pair<int, int> pool_stride,
                                 std::pair<int, int> pool_pad)
{
    if (input.shape().size() != 4 || input.shape()[1] != (size_t)in_channels_ ||
        input.device().type() != DeviceType::kCUDA || input.dtype() != DataType::kFloat32)
        return functional::max_pool2d(functional::relu(forward(input)), pool_kernel, pool_stride, pool_pad);
    const Tensor *b = use_bias_ ? &static_cast<const Tensor &>(bias_) : nullptr;
    return functional::conv2d_relu_max_pool2d(input, static_cast<const Tensor &>(weight_), b, stride_, pad_, pool_kernel,
                                              pool_stride, pool_pad);
}

MaxPool2d::MaxPool2d(std::pair<int, int> kernel_size, std::pair<int, int> stride, std::pair<int, int> pad)
    : kernel_(kernel_size), stride_((stride.first == 0 && stride.second == 0) ? kernel_size : stride), pad_(pad)
{}

MaxPool2d::MaxPool2d(int kernel_size, int stride, int pad) : MaxPool2d(pair(kernel_size), pair(stride), pair(pad)) {}

MLP::MLP(const std::vector<int> &sizes, std::function<Tensor(const Tensor &)> activation)
    : activation_(activation ? std::move(activation) : [](const Tensor &x) { return functional::relu(x); }),
      default_relu_(!activation)
{
    if (sizes.size() < 2)
        THROW_INVALID_ARG("MLP needs at least an input and an output size");
    for (size_t i = 0; i + 1 < sizes.size(); ++i)
    {
        auto l = std::make_unique<Linear>(sizes[i], sizes[i + 1], true);
        layers_.push_back(l.get());
        register_module("layer_" + std::to_string(i), std::move(l));  // the names state_dict() keys are built from
    }
}

Tensor MLP::forward(const Tensor &input)
{
    Tensor x = input;
    for (size_t i = 0; i < layers_.size(); ++i)
    {
        // src/nn/models/mlp.cpp:43-61: every layer but the last is followed by the activation. With the default ReLU
        // the pair runs as one operator, as a Linear followed by a ReLU inside a Sequential does (the same bits).
        if (i + 1 < layers_.size() && default_relu_)
            x = layers_[i]->forward_relu(x);
        else
        {
            x = layers_[i]->forward(x);
            if (i + 1 < layers_.size())
                x = activation_(x);
        }
    }
    return x;
}
}  // namespace nn

// ---------------------------------------------------------------------------------------- optimizers
Optimizer::Optimizer(Module &target) : target_(&target), parameters_(target.parameters()) {}

void Optimizer::step()
{
    std::vector<Parameter *> with_grad;
    for (auto *p : parameters_)
        if (p->defined() && p->grad().defined())
            with_grad.push_back(p);
    // a lone WeightDecay hook in front of a one-launch step rides along in that launch
    const WeightDecayHook *decay = hooks_.size() == 1 ? hooks_[0].target<WeightDecayHook>() : nullptr;
    if (decay && decay->rate != 0.0f && step_all_takes_decay(with_grad))
    {
        hook_decay_ = decay->rate;
        try
        {
            step_all(with_grad);
        }
        catch (...)
        {
            hook_decay_ = 0.0f;
            throw;
        }
        hook_decay_ = 0.0f;
        return;
    }
    for (auto &h : hooks_)
        h(with_grad);
    step_all(with_grad);
}

void Optimizer::zero_grad()
{
    for (auto *p : parameters_)
        p->clear_grad();
}

namespace
{
const OriginMat &origin_mat(const Tensor &t)
{
    const auto *m = dynamic_cast<const OriginMat *>(t.impl_->data_.get());
    if (!m)
        THROW_RUNTIME_ERROR("optimizer: parameter is not backed by an OriginMat");
    return *m;
}

// The updated parameter starts a fresh graph: it must stay a leaf, otherwise every later backward would walk
// back through all earlier optimizer steps.
Parameter as_leaf(const Tensor &updated)
{
    Tensor t = updated.detach();
    t.impl_->requires_grad_ = true;
    return Parameter(t);
}
}  // namespace

SGD::SGD(Module &target, float lr, float momentum, float weight_decay, bool nesterov)
    : Optimizer(target), lr_(lr), momentum_(momentum), weight_decay_(weight_decay), nesterov_(nesterov)
{}

void SGD::step_one(Parameter &param)
{
    NoGradGuard guard;
    Tensor grad = param.grad();
    if (weight_decay_ > 0.0f)
        grad = grad + param * Scalar(weight_decay_);
    if (momentum_ > 0.0f)
    {
        auto it = momentum_buffers_.find(&param);
        if (it == momentum_buffers_.end())
            it = momentum_buffers_.emplace(&param, Tensor::zeros(grad.shape(), TensorOptions(grad.dtype()).device(grad.device()))).first;
        Tensor &buf = it->second;
        if (cuda::is_capturing())
            const_cast<OriginMat &>(origin_mat(buf)).copy_from(*(buf * Scalar(momentum_) + grad).impl_->data_);
        else
            buf = buf * Scalar(momentum_) + grad;
        grad = nesterov_ ? grad + buf * Scalar(momentum_) : buf;
    }
    // While a graph is being captured every persistent tensor is written where it lies (a later replay reads it
    // from that address), instead of being rebound to a new one.
    const bool in_place = cuda::is_capturing();
    if (weight_decay_ <= 0.0f && momentum_ <= 0.0f)
    {
        // plain step: one launch computing the same two roundings as param - grad * lr
        if (in_place)
            const_cast<OriginMat &>(origin_mat(param)).sgd_step_inplace(*grad.impl_->data_, lr_);
        else
            param = as_leaf(Tensor(origin_mat(param).sgd_step(*grad.impl_->data_, lr_)));
        return;
    }
    if (in_place)
        const_cast<OriginMat &>(origin_mat(param)).copy_from(*(param - grad * Scalar(lr_)).impl_->data_);
    else
        param = as_leaf(param - grad * Scalar(lr_));
}

namespace
{
// every parameter and its gradient float32 on the device, of one shape: what the one-launch steps and the hook's own
// one-launch form both ask for
bool all_on_device(const std::vector<Parameter *> &params)
{
    for (auto *p : params)
        if (!OriginMat::device_f32(*p->impl_->data_) || !OriginMat::device_f32(*p->grad().impl_->data_) ||
            p->grad().shape() != p->shape())
            return false;
    return true;
}
}  // namespace

bool SGD::step_all_takes_decay(const std::vector<Parameter *> &params) const
{
    return weight_decay_ <= 0.0f && momentum_ <= 0.0f && params.size() > 1 && all_on_device(params);
}

bool Adam::step_all_takes_decay(const std::vector<Parameter *> &params) const
{
    return params.size() > 1 && all_on_device(params);
}

// The plain step (no momentum, no weight decay) over device parameters: one launch for the whole list.
void SGD::step_all(std::vector<Parameter *> &params)
{
    bool fused = weight_decay_ <= 0.0f && momentum_ <= 0.0f && params.size() > 1;
    for (auto *p : params)
        fused = fused && OriginMat::device_f32(*p->impl_->data_) && OriginMat::device_f32(*p->grad().impl_->data_);
    if (!fused)
    {
        Optimizer::step_all(params);
        return;
    }
    NoGradGuard guard;
    std::vector<std::pair<const Mat *, const Mat *>> list;
    std::vector<Tensor> grads;  // keeps the gradients alive until the launch is queued
    for (auto *p : params)
    {
        grads.push_back(p->grad());
        list.emplace_back(p->impl_->data_.get(), grads.back().impl_->data_.get());
    }
    const bool in_place = cuda::is_capturing();
    auto updated = OriginMat::sgd_step_multi(list, lr_, in_place, hook_decay_);
    if (!in_place)
        for (size_t i = 0; i < params.size(); ++i)
            *params[i] = as_leaf(Tensor(std::move(updated[i])));
}

Adam::Adam(Module &target, float lr, float beta1, float beta2, float eps)
    : Optimizer(target), lr_(lr), beta1_(beta1), beta2_(beta2), eps_(eps)
{}

void Adam::step_one(Parameter &param)
{
    NoGradGuard guard;
    const Tensor grad = param.grad();
    auto zeros = [&] { return Tensor::zeros(grad.shape(), TensorOptions(grad.dtype()).device(grad.device())); };
    if (!m_buffers_.count(&param))
        m_buffers_.emplace(&param, zeros());
    if (!v_buffers_.count(&param))
        v_buffers_.emplace(&param, zeros());
    Tensor &m = m_buffers_.at(&param), &v = v_buffers_.at(&param);
    if (!replay_scales_.defined())  // two floats per parameter, read by recorded steps (see prepare_replay)
        replay_scales_ = Tensor::zeros(Shape{parameters_.size(), 2}, TensorOptions(DataType::kFloat32).device(grad.device()));
    if (cuda::is_capturing())
    {
        // recorded, not run: the step count moves in prepare_replay(), and the factors come from device memory
        if (!step_counts_.count(&param))
            THROW_RUNTIME_ERROR("Adam: run one ordinary step before capturing (the moment buffers must exist)");
        size_t index = 0;
        while (index < parameters_.size() && parameters_[index] != &param)
            ++index;
        const float *scales = static_cast<const OriginMat &>(*replay_scales_.impl_->data_).data_ptr<float>() + 2 * index;
        const_cast<OriginMat &>(origin_mat(param))
            .adam_step_inplace(*grad.impl_->data_, *m.impl_->data_, *v.impl_->data_, beta1_, beta2_, scales, eps_, lr_);
        replay_params_.push_back(&param);
        return;
    }
    int &t = step_counts_[&param];
    ++t;
    // same sequence of elementwise steps, each rounded to float, as src/optim/adam.cpp:52-113
    //   m = m*b1 + grad*(1-b1);  v = v*b2 + (grad*grad)*(1-b2);  m_hat = m*s1;  v_hat = v*s2;
    //   param = param - (m_hat / (pow(v_hat, 0.5) + eps)) * lr
    // fused into one launch per parameter (the reference issues ~15 whole-tensor ops and 10 scalar fills)
    const float b1p = std::pow(beta1_, static_cast<float>(t)), b2p = std::pow(beta2_, static_cast<float>(t));
    const float m_hat_scale = 1.0f / (1.0f - b1p), v_hat_scale = 1.0f / (1.0f - b2p);
    param = as_leaf(Tensor(origin_mat(param).adam_step(*grad.impl_->data_, *m.impl_->data_, *v.impl_->data_, beta1_, beta2_,
                                                       m_hat_scale, v_hat_scale, eps_, lr_)));
}

// Device parameters take one launch for the whole list; the bookkeeping per parameter (buffers, step counts, factors)
// is that of step_one.
void Adam::step_all(std::vector<Parameter *> &params)
{
    bool fused = params.size() > 1;
    for (auto *p : params)
        fused = fused && OriginMat::device_f32(*p->impl_->data_) && OriginMat::device_f32(*p->grad().impl_->data_);
    if (!fused)
    {
        Optimizer::step_all(params);
        return;
    }
    NoGradGuard guard;
    const bool capturing = cuda::is_capturing();
    std::vector<OriginMat::AdamItem> items;
    std::vector<Tensor> grads;
    for (auto *pp : params)
    {
        Parameter &param = *pp;
        grads.push_back(param.grad());
        const Tensor &grad = grads.back();
        auto zeros = [&] { return Tensor::zeros(grad.shape(), TensorOptions(grad.dtype()).device(grad.device())); };
        if (!m_buffers_.count(&param))
            m_buffers_.emplace(&param, zeros());
        if (!v_buffers_.count(&param))
            v_buffers_.emplace(&param, zeros());
        if (!replay_scales_.defined())
            replay_scales_ = Tensor::zeros(Shape{parameters_.size(), 2}, TensorOptions(DataType::kFloat32).device(grad.device()));
        OriginMat::AdamItem it{};
        it.param = param.impl_->data_.get(), it.grad = grad.impl_->data_.get();
        it.m = m_buffers_.at(&param).impl_->data_.get(), it.v = v_buffers_.at(&param).impl_->data_.get();
        if (capturing)
        {
            if (!step_counts_.count(&param))
                THROW_RUNTIME_ERROR("Adam: run one ordinary step before capturing (the moment buffers must exist)");
            size_t index = 0;
            while (index < parameters_.size() && parameters_[index] != &param)
                ++index;
            it.device_scales = static_cast<const OriginMat &>(*replay_scales_.impl_->data_).data_ptr<float>() + 2 * index;
            replay_params_.push_back(&param);
        }
        else
        {
            const int t = ++step_counts_[&param];
            const float b1p = std::pow(beta1_, static_cast<float>(t)), b2p = std::pow(beta2_, static_cast<float>(t));
            it.m_hat_scale = 1.0f / (1.0f - b1p), it.v_hat_scale = 1.0f / (1.0f - b2p);
        }
        items.push_back(it);
    }
    auto updated = OriginMat::adam_step_multi(items, beta1_, beta2_, eps_, lr_, capturing, hook_decay_);
    if (!capturing)
        for (size_t i = 0; i < params.size(); ++i)
            *params[i] = as_leaf(Tensor(std::move(updated[i])));
}

void Adam::prepare_replay()
{
    if (replay_params_.empty())
        return;
    std::vector<float> host(parameters_.size() * 2, 0.0f);
    for (Parameter *p : replay_params_)
    {
        size_t index = 0;
        while (index < parameters_.size() && parameters_[index] != p)
            ++index;
        const int t = ++step_counts_[p];
        const float b1p = std::pow(beta1_, static_cast<float>(t)), b2p = std::pow(beta2_, static_cast<float>(t));
        host[2 * index] = 1.0f / (1.0f - b1p), host[2 * index + 1] = 1.0f / (1.0f - b2p);
    }
    replay_scales_.upload(host.data(), host.size() * sizeof(float));
}

std::function<void(std::vector<Parameter *> &)> WeightDecay::hook() const
{
    return WeightDecayHook{rate_};
}

void WeightDecayHook::operator()(std::vector<Parameter *> &params) const
{
    {
        NoGradGuard guard;
        // grad += rate * param: one launch for all parameters that live on the device (the product is rounded, then
        // added — what the separate multiply and accumulate give)
        std::vector<std::pair<const Mat *, Mat *>> on_device;
        std::vector<Tensor> grads;
        for (auto *p : params)
        {
            if (!p)
                continue;
            Tensor g = p->grad();
            if (g.defined() && OriginMat::device_f32(*g.impl_->data_) && OriginMat::device_f32(*p->impl_->data_) &&
                g.shape() == p->shape())
            {
                grads.push_back(g);
                on_device.emplace_back(p->impl_->data_.get(), g.impl_->data_.get());
            }
            else
                p->accumulate_grad(static_cast<const Tensor &>(*p) * Scalar(rate));
        }
        if (!on_device.empty())
            OriginMat::axpy_multi(rate, on_device);
    }
}

// ----------------------------------------------------------------------------------------- device API
namespace cuda
{
int device_count()
{
    int n = 0;
    odl_hip_device_count(&n);
    return n;
}
bool is_available()
{
    return device_count() > 0;
}
int current_device()
{
    int d = 0;
    if (odl_hip_get_device(&d) != ODL_OK)
        THROW_RUNTIME_ERROR("{}", odl_hip_last_error());
    return d;
}
void set_device(int device)
{
    if (odl_hip_set_device(device) != ODL_OK)
        THROW_RUNTIME_ERROR("{}", odl_hip_last_error());
}
void device_info()
{
    const int n = device_count();
    for (int i = 0; i < n; ++i)
    {
        char buf[256];
        if (odl_hip_device_info(i, buf, sizeof(buf)) == ODL_OK)
            loga("Device {}: {}", i, buf);
    }
}
void synchronize()
{
    if (odl_hip_synchronize() != ODL_OK)
        THROW_RUNTIME_ERROR("{}", odl_hip_last_error());
}
}  // namespace cuda
}  // namespace origin

// ---- optimizer state (src/optim/adam.cpp:116-284, src/optim/sgd.cpp:77-157)
namespace origin
{
namespace
{
std::string name_of(const std::unordered_map<std::string, const Parameter *> &named, const Parameter *p)
{
    for (const auto &kv : named)
        if (kv.second == p)
            return kv.first;
    return "";
}

template <typename T>
void read_setting(const std::unordered_map<std::string, std::any> &sd, const char *key, T &dst)
{
    auto it = sd.find(key);
    if (it != sd.end())
        dst = std::any_cast<T>(it->second);
}

void read_buffers(const std::unordered_map<std::string, std::any> &sd, const char *key, const std::string &prefix,
                  std::unordered_map<std::string, Parameter *> &named, std::unordered_map<Parameter *, Tensor> &dst)
{
    auto it = sd.find(key);
    if (it == sd.end())
        return;
    const auto buffers = std::any_cast<StateDict>(it->second);
    dst.clear();
    for (const auto &kv : buffers)
        if (kv.first.size() > prefix.size() && kv.first.compare(0, prefix.size(), prefix) == 0)
        {
            auto p = named.find(kv.first.substr(prefix.size()));
            if (p != named.end())
                dst[p->second] = kv.second;
        }
}
}  // namespace

std::unordered_map<std::string, std::any> Adam::state_dict() const
{
    std::unordered_map<std::string, std::any> state;
    state["lr"] = lr_, state["beta1"] = beta1_, state["beta2"] = beta2_, state["eps"] = eps_;
    const auto named = static_cast<const Module *>(target_)->named_parameters("");
    StateDict m, v;
    std::unordered_map<std::string, int> steps;
    for (const auto &kv : m_buffers_)
        if (const std::string n = name_of(named, kv.first); !n.empty())
            m["m_" + n] = kv.second;
    for (const auto &kv : v_buffers_)
        if (const std::string n = name_of(named, kv.first); !n.empty())
            v["v_" + n] = kv.second;
    for (const auto &kv : step_counts_)
        if (const std::string n = name_of(named, kv.first); !n.empty())
            steps["step_" + n] = kv.second;
    state["m_buffers"] = m, state["v_buffers"] = v, state["step_counts"] = steps;
    return state;
}

void Adam::load_state_dict(const std::unordered_map<std::string, std::any> &sd)
{
    read_setting(sd, "lr", lr_), read_setting(sd, "beta1", beta1_), read_setting(sd, "beta2", beta2_);
    read_setting(sd, "eps", eps_);
    auto named = target_->named_parameters("");
    read_buffers(sd, "m_buffers", "m_", named, m_buffers_);
    read_buffers(sd, "v_buffers", "v_", named, v_buffers_);
    auto it = sd.find("step_counts");
    if (it != sd.end())
    {
        const auto steps = std::any_cast<std::unordered_map<std::string, int>>(it->second);
        step_counts_.clear();
        for (const auto &kv : steps)
            if (kv.first.size() > 5 && kv.first.compare(0, 5, "step_") == 0)
            {
                auto p = named.find(kv.first.substr(5));
                if (p != named.end())
                    step_counts_[p->second] = kv.second;
            }
    }
}

std::unordered_map<std::string, std::any> SGD::state_dict() const
{
    std::unordered_map<std::string, std::any> state;
    state["lr"] = lr_, state["momentum"] = momentum_, state["weight_decay"] = weight_decay_, state["nesterov"] = nesterov_;
    if (momentum_ > 0.0f)
    {
        const auto named = static_cast<const Module *>(target_)->named_parameters("");
        StateDict buffers;
        for (const auto &kv : momentum_buffers_)
            if (const std::string n = name_of(named, kv.first); !n.empty())
                buffers["momentum_" + n] = kv.second;
        state["momentum_buffers"] = buffers;
    }
    return state;
}

// The reference compares a ten-character prefix with the nine-character "momentum_" and so never restores a
// momentum buffer (sgd.cpp:146-148); here the buffers written by state_dict() are read back.
void SGD::load_state_dict(const std::unordered_map<std::string, std::any> &sd)
{
    read_setting(sd, "lr", lr_), read_setting(sd, "momentum", momentum_), read_setting(sd, "weight_decay", weight_decay_);
    read_setting(sd, "nesterov", nesterov_);
    if (momentum_ > 0.0f)
    {
        auto named = target_->named_parameters("");
        read_buffers(sd, "momentum_buffers", "momentum_", named, momentum_buffers_);
    }
}
}  // namespace origin
