// Tensor (value handle) -> TensorImpl (data, grad, creator, generation) -> Mat, and the Operator base that
// records the graph. Public surface and behaviour follow the reference's include/origin/core/{tensor,
// tensor_impl,operator,parameter,config}.h and src/core/tensor_impl.cpp:78-278 (generation-ordered backward,
// first gradient shares the Mat, later ones accumulate in place, graph released afterwards).
#pragma once
#include <functional>
#include <memory>
#include <string>
#include <vector>

#include "mat.h"

namespace origin
{
class Operator;
class Tensor;

struct Config
{
    static bool enable_backprop;
};

// RAII switch: `auto guard = no_grad();` disables graph construction until the guard dies
class NoGradGuard
{
public:
    NoGradGuard() : old_(Config::enable_backprop) { Config::enable_backprop = false; }
    ~NoGradGuard() { Config::enable_backprop = old_; }

private:
    bool old_;
};
inline NoGradGuard no_grad()
{
    return NoGradGuard();
}

class TensorImpl
{
public:
    std::shared_ptr<Mat> data_;
    std::shared_ptr<Mat> grad_;
    std::shared_ptr<Operator> creator_;
    int generation_     = 0;
    bool requires_grad_ = false;

    explicit TensorImpl(std::unique_ptr<Mat> m) : data_(std::move(m)) {}
    explicit TensorImpl(std::shared_ptr<Mat> m) : data_(std::move(m)) {}
    void set_creator(const std::shared_ptr<Operator> &func);
    void backward();
    void clear_grad() { grad_ = nullptr; }
    Shape shape() const { return data_->shape(); }
};

class Tensor
{
public:
    Tensor() = default;
    explicit Tensor(std::shared_ptr<TensorImpl> impl) : impl_(std::move(impl)) {}
    explicit Tensor(std::unique_ptr<Mat> mat) : impl_(std::make_shared<TensorImpl>(std::move(mat))) {}

    template <typename T>
    Tensor(const std::vector<T> &data, const Shape &shape) : Tensor(data, shape, TensorOptions(DataTypeTraits<T>::type))
    {}
    template <typename T>
    Tensor(const std::vector<T> &data, const Shape &shape, DataType dtype) : Tensor(data, shape, TensorOptions(dtype))
    {}
    template <typename T>
    Tensor(const std::vector<T> &data, const Shape &shape, const TensorOptions &options)
    {
        if (data.size() != shape.elements())
            throw std::invalid_argument("Data size (" + std::to_string(data.size()) + ") does not match shape elements (" +
                                        std::to_string(shape.elements()) + ")");
        check_extents(shape);
        init(Mat_t::from_memory(data.data(), DataTypeTraits<T>::type, shape, options), options);
    }
    template <typename T>
    Tensor(std::initializer_list<T> data, const Shape &shape) : Tensor(std::vector<T>(data), shape)
    {}
    template <typename T>
    Tensor(std::initializer_list<T> data, const Shape &shape, DataType dtype) : Tensor(std::vector<T>(data), shape, dtype)
    {}
    template <typename T>
    Tensor(std::initializer_list<T> data, const Shape &shape, const TensorOptions &options)
        : Tensor(std::vector<T>(data), shape, options)
    {}
    template <typename T, typename = std::enable_if_t<std::is_arithmetic<T>::value>>
    Tensor(T scalar, const Shape &shape) : Tensor(Scalar(scalar), shape, TensorOptions(DataTypeTraits<T>::type))
    {}
    template <typename T, typename = std::enable_if_t<std::is_arithmetic<T>::value>>
    Tensor(T scalar, const Shape &shape, const TensorOptions &options) : Tensor(Scalar(scalar), shape, options)
    {}
    Tensor(const Scalar &scalar, const Shape &shape, const TensorOptions &options)
    {
        check_extents(shape);
        init(Mat_t::from_scalar(scalar, shape, options), options);
    }

    static Tensor zeros(const Shape &shape, const TensorOptions &options = TensorOptions());
    static Tensor ones(const Shape &shape, const TensorOptions &options = TensorOptions());
    static Tensor randn(const Shape &shape, const TensorOptions &options = TensorOptions());
    static Tensor full(const Shape &shape, const Scalar &value, const TensorOptions &options = TensorOptions());
    // a tensor holding a copy of shape.elements() values of options.dtype() read from host memory (src/core/tensor.cpp:72-78)
    static Tensor from_blob(void *data, const Shape &shape, const TensorOptions &options = TensorOptions());

    Shape shape() const;
    size_t ndim() const { return shape().size(); }
    size_t elements() const { return shape().elements(); }
    size_t numel() const { return elements(); }
    size_t element_size() const { return dtype_size(dtype()); }
    size_t nbytes() const { return elements() * element_size(); }
    // the element buffer as it lies: host memory for a CPU tensor, device memory for a device tensor
    template <typename T>
    T *data_ptr()
    {
        check_defined("data_ptr");
        return static_cast<T *>(impl_->data_->data_ptr());
    }
    // one element by its coordinates; on the device a synchronising copy of that element
    template <typename T>
    T index(std::initializer_list<size_t> indices) const
    {
        check_defined("index");
        return impl_->data_->index(indices).template to<T>();
    }
    void index_put(std::initializer_list<size_t> indices, const Scalar &value)
    {
        check_defined("index_put");
        impl_->data_->index_put(indices, value);
    }
    DataType dtype() const;
    Device device() const;
    bool defined() const { return impl_ && impl_->data_; }
    bool requires_grad() const { return impl_ && impl_->requires_grad_; }

    template <typename T>
    T item() const
    {
        check_defined("item");
        if (elements() != 1)
            THROW_INVALID_ARG("item() needs a single-element tensor, shape is {}", shape().to_string());
        return to_vector<T>()[0];
    }
    template <typename T>
    std::vector<T> to_vector() const
    {
        check_defined("to_vector");
        return static_cast<const OriginMat &>(*impl_->data_).to_vector<T>();
    }

    // overwrites the elements in place from host memory (same byte count); the tensor keeps its address, which is
    // what a recorded graph reads from
    void upload(const void *host, size_t bytes);
    Tensor to(DataType target) const;
    Tensor to(Device device) const;
    Tensor to(const TensorOptions &options) const;
    Tensor grad() const;
    void set_creator(const std::shared_ptr<Operator> &func);
    void backward();
    void clear_grad();
    void accumulate_grad(const Tensor &grad_to_add);
    Tensor detach() const;
    Tensor clone() const;
    Tensor reshape(const Shape &shape) const;
    Tensor transpose() const;
    Tensor contiguous() const;
    void print(const std::string &desc = "") const;
    int backend_type() const { return ORIGIN_BACKEND_TYPE; }

    std::shared_ptr<TensorImpl> impl_;

private:
    void init(std::unique_ptr<Mat> m, const TensorOptions &options)
    {
        impl_                 = std::make_shared<TensorImpl>(std::move(m));
        impl_->requires_grad_ = options.requires_grad();
    }
    // a 0-dim shape is a scalar tensor; an extent of zero is refused (src/core/tensor.cpp:399-437)
    static void check_extents(const Shape &shape)
    {
        for (size_t i = 0; i < shape.size(); ++i)
            if (shape[i] == 0)
                THROW_INVALID_ARG("Tensor shape cannot have zero dimensions. Dimension {} is zero in shape {}", i,
                                  shape.to_string());
    }
    void check_defined(const char *who) const
    {
        if (!defined())
            THROW_RUNTIME_ERROR("{} called on an undefined Tensor", who);
    }
};

class Parameter : public Tensor
{
public:
    using Tensor::Tensor;
    Parameter() = default;
    Parameter(const Tensor &t) : Tensor(t) {}
    Parameter(Tensor &&t) : Tensor(std::move(t)) {}
    Parameter &operator=(const Tensor &t)
    {
        static_cast<Tensor &>(*this) = t;
        return *this;
    }
};

class Operator : public std::enable_shared_from_this<Operator>
{
public:
    virtual ~Operator() = default;
    Tensor operator()(const Tensor &input) { return (*this)(std::vector<Tensor>{input})[0]; }
    std::vector<Tensor> operator()(const std::vector<Tensor> &inputs);
    virtual std::vector<Tensor> forward(const std::vector<Tensor> &inputs)        = 0;
    virtual std::vector<Tensor> backward(const std::vector<Tensor> &grad_outputs) = 0;

    std::vector<Tensor> inputs_;
    std::vector<std::weak_ptr<TensorImpl>> outputs_;  // weak: outputs own the operator, not the reverse
    int generation_ = 0;

protected:
    static const Mat &mat(const Tensor &t)
    {
        if (!t.impl_ || !t.impl_->data_)
            THROW_RUNTIME_ERROR("mat() called on an undefined Tensor");
        return *t.impl_->data_;
    }
    static const OriginMat &omat(const Tensor &t) { return static_cast<const OriginMat &>(mat(t)); }
    static Tensor wrap(std::unique_ptr<Mat> m) { return Tensor(std::move(m)); }
};
}  // namespace origin
