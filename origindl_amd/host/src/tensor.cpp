// Autograd core: generation-ordered reverse walk with in-place gradient accumulation, as in the reference's
// src/core/tensor_impl.cpp:78-278 and src/operators/operator.cpp:9-36.
#include "origin/tensor.h"

#include <algorithm>
#include <set>

namespace origin
{
bool Config::enable_backprop = true;

void TensorImpl::set_creator(const std::shared_ptr<Operator> &func)
{
    creator_    = func;
    generation_ = func->generation_ + 1;
}

void TensorImpl::backward()
{
    if (!Config::enable_backprop)
        return;
    if (!requires_grad_)
        THROW_RUNTIME_ERROR("tensor does not require grad and does not have a grad_fn, can't run backward");
    if (!grad_)  // seed with ones of the output's shape
        grad_ = std::shared_ptr<Mat>(
            Mat_t::from_scalar(Scalar(1.0f), data_->shape(), TensorOptions(data_->dtype()).device(data_->device())));

    std::vector<std::shared_ptr<Operator>> queue;  // kept sorted by generation, the back is processed next
    std::set<Operator *> seen;
    auto push = [&](const std::shared_ptr<Operator> &f) {
        if (!f || !seen.insert(f.get()).second)
            return;
        auto pos = std::upper_bound(queue.begin(), queue.end(), f,
                                    [](const auto &a, const auto &b) { return a->generation_ < b->generation_; });
        queue.insert(pos, f);
    };
    push(creator_);

    std::vector<std::shared_ptr<Operator>> done;
    std::set<std::shared_ptr<TensorImpl>> touched;
    while (!queue.empty())
    {
        auto f = queue.back();
        queue.pop_back();
        std::vector<std::shared_ptr<TensorImpl>> outs;
        std::vector<Tensor> gys;
        for (const auto &w : f->outputs_)
            if (auto o = w.lock())
            {
                outs.push_back(o);
                touched.insert(o);
                gys.push_back(Tensor(o).grad());
            }
        if (gys.empty())
            continue;
        done.push_back(f);
        auto gxs = f->backward(gys);
        if (gxs.size() != f->inputs_.size())
            THROW_RUNTIME_ERROR("backward error!, gxs size {} inputs size {}", gxs.size(), f->inputs_.size());
        for (size_t i = 0; i < gxs.size(); ++i)
        {
            auto &x = f->inputs_[i];
            if (!x.impl_ || !gxs[i].impl_)
                continue;
            touched.insert(x.impl_);
            if (!x.impl_->grad_)
                x.impl_->grad_ = gxs[i].impl_->data_;  // the first gradient shares the Mat
            else
                x.impl_->grad_->add_inplace(*gxs[i].impl_->data_);
            push(x.impl_->creator_);
        }
    }

    // release the graph: inputs are forgotten, intermediate gradients dropped, leaf gradients kept
    std::set<std::shared_ptr<TensorImpl>> inputs;
    for (const auto &f : done)
        for (const auto &in : f->inputs_)
            if (in.impl_)
                inputs.insert(in.impl_);
    std::set<TensorImpl *> had_creator;
    for (const auto &t : touched)
        if (t->creator_)
            had_creator.insert(t.get());
    for (const auto &f : done)
        f->inputs_.clear();
    for (const auto &t : touched)
    {
        const bool is_input = inputs.count(t) != 0, is_root = (t.get() == this);
        t->creator_    = nullptr;
        t->generation_ = 0;
        if (!is_input && !is_root)
            t->grad_ = nullptr;
    }
    creator_    = nullptr;
    generation_ = 0;
}

std::vector<Tensor> Operator::operator()(const std::vector<Tensor> &inputs)
{
    auto outputs = this->forward(inputs);
    bool needs   = false;
    if (Config::enable_backprop)
        for (const auto &in : inputs)
            needs = needs || in.requires_grad();
    for (auto &out : outputs)
        if (out.impl_)
            out.impl_->requires_grad_ = needs;
    if (needs)
    {
        int gen = 0;
        for (const auto &in : inputs)
            gen = std::max(gen, in.impl_->generation_);
        generation_ = gen;
        inputs_     = inputs;
        outputs_.clear();
        for (auto &out : outputs)
            if (out.impl_)
            {
                out.set_creator(shared_from_this());
                outputs_.push_back(out.impl_);
            }
    }
    return outputs;
}

// ------------------------------------------------------------------------------------------------ Tensor
Tensor Tensor::zeros(const Shape &s, const TensorOptions &o)
{
    Tensor t(Mat_t::zeros(s, o));
    t.impl_->requires_grad_ = o.requires_grad();
    return t;
}
Tensor Tensor::ones(const Shape &s, const TensorOptions &o)
{
    Tensor t(Mat_t::ones(s, o));
    t.impl_->requires_grad_ = o.requires_grad();
    return t;
}
Tensor Tensor::randn(const Shape &s, const TensorOptions &o)
{
    Tensor t(Mat_t::randn(s, o));
    t.impl_->requires_grad_ = o.requires_grad();
    return t;
}
Tensor Tensor::full(const Shape &s, const Scalar &v, const TensorOptions &o)
{
    Tensor t(Mat_t::from_scalar(v, s, o));
    t.impl_->requires_grad_ = o.requires_grad();
    return t;
}

Tensor Tensor::from_blob(void *data, const Shape &s, const TensorOptions &o)
{
    if (!data)
        THROW_INVALID_ARG("from_blob: null data");
    Tensor t(Mat_t::from_memory(data, o.dtype(), s, o));
    t.impl_->requires_grad_ = o.requires_grad();
    return t;
}

void Tensor::upload(const void *host, size_t bytes)
{
    check_defined("upload");
    static_cast<OriginMat &>(*impl_->data_).upload(host, bytes);
}

Shape Tensor::shape() const
{
    check_defined("shape");  // src/core/tensor.cpp:82-86: metadata of an undefined tensor throws
    return impl_->data_->shape();
}
DataType Tensor::dtype() const
{
    check_defined("dtype");
    return impl_->data_->dtype();
}
Device Tensor::device() const
{
    check_defined("device");
    return impl_->data_->device();
}

Tensor Tensor::to(DataType target) const
{
    check_defined("to");
    Tensor t(impl_->data_->to(target));
    t.impl_->requires_grad_ = impl_->requires_grad_;
    return t;
}
Tensor Tensor::to(Device device) const
{
    check_defined("to");
    Tensor t(impl_->data_->to_device(device));
    t.impl_->requires_grad_ = impl_->requires_grad_;
    return t;
}
Tensor Tensor::to(const TensorOptions &options) const
{
    Tensor t = to(options.dtype()).to(options.device());
    t.impl_->requires_grad_ = impl_->requires_grad_ || options.requires_grad();
    return t;
}

Tensor Tensor::grad() const
{
    check_defined("grad");
    if (!impl_->grad_)
        return Tensor();
    return Tensor(std::make_shared<TensorImpl>(impl_->grad_));
}
void Tensor::set_creator(const std::shared_ptr<Operator> &func)
{
    impl_->set_creator(func);
}
void Tensor::backward()
{
    check_defined("backward");
    impl_->backward();
}
void Tensor::clear_grad()
{
    if (impl_)
        impl_->clear_grad();
}
void Tensor::accumulate_grad(const Tensor &g)
{
    check_defined("accumulate_grad");
    if (!g.defined())
        return;
    if (!impl_->grad_)
        impl_->grad_ = g.impl_->data_->clone();
    else
        impl_->grad_->add_inplace(*g.impl_->data_);
}
Tensor Tensor::detach() const
{
    check_defined("detach");
    return Tensor(std::make_shared<TensorImpl>(impl_->data_));  // shares the data, drops graph and grad
}
Tensor Tensor::clone() const
{
    check_defined("clone");
    Tensor t(impl_->data_->clone());
    t.impl_->requires_grad_ = impl_->requires_grad_;
    return t;
}
Tensor Tensor::contiguous() const
{
    check_defined("contiguous");
    return Tensor(impl_->data_->contiguous());
}
void Tensor::print(const std::string &desc) const
{
    check_defined("print");
    impl_->data_->print(desc);
}
}  // namespace origin
