// Host-side value types of the backend's C++ layer: DataType/Device/Shape/Scalar/TensorOptions, the exception
// macros and the {}-style log helpers. Same names and meaning as the reference's include/origin/mat/
// {basic_types,shape,scalar}.h, include/origin/core/tensor_options.h and include/origin/utils/{exception,log}.h,
// written from scratch; only what the hot path's callers touch is present.
#pragma once
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <initializer_list>
#include <iomanip>
#include <iostream>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace origin
{
// ---------------------------------------------------------------- {}-formatting (no external fmt library)
namespace detail
{
inline void format_rest(std::ostringstream &os, const char *f)
{
    os << f;
}

template <typename T, typename... R>
void format_rest(std::ostringstream &os, const char *f, const T &v, const R &...rest)
{
    for (; *f; ++f)
    {
        if (f[0] == '{')
        {
            const char *close = f;
            while (*close && *close != '}')
                ++close;
            if (*close == '}')
            {
                std::string spec(f + 1, close);  // "", ":.4f", ":6d" ...
                std::ostringstream one;
                const auto dot = spec.find('.');
                if (dot != std::string::npos)
                    one << std::fixed << std::setprecision(std::atoi(spec.c_str() + dot + 1));
                one << v;
                os << one.str();
                format_rest(os, close + 1, rest...);
                return;
            }
        }
        os << *f;
    }
}
}  // namespace detail

template <typename... A>
std::string format(const char *f, const A &...args)
{
    std::ostringstream os;
    detail::format_rest(os, f, args...);
    return os.str();
}

#define ODL_WHERE_ (std::string("[") + __FILE__ + ":" + __func__ + ":" + std::to_string(__LINE__) + "] ")
#define THROW_INVALID_ARG(...) throw std::invalid_argument(ODL_WHERE_ + ::origin::format(__VA_ARGS__))
#define THROW_RUNTIME_ERROR(...) throw std::runtime_error(ODL_WHERE_ + ::origin::format(__VA_ARGS__))

// loga = always printed (the reference's fmt::println); the levelled macros print at warn and above
#define loga(...) (std::cout << ::origin::format(__VA_ARGS__) << std::endl)
#define logw(...) (std::cerr << "[warn] " << ::origin::format(__VA_ARGS__) << std::endl)
#define loge(...) (std::cerr << "[error] " << ::origin::format(__VA_ARGS__) << std::endl)
#define logi(...) ((void)0)
#define logd(...) ((void)0)
#define logt(...) ((void)0)

// ---------------------------------------------------------------- dtypes and devices
enum class DataType
{
    kFloat32 = 0,
    kFloat64 = 1,
    kInt8    = 2,
    kInt32   = 3,
    kInt64   = 4,
    kUInt8   = 5,
};

// short names, as include/origin/mat/basic_types.h:29-34
constexpr auto Float32 = DataType::kFloat32;
constexpr auto Float64 = DataType::kFloat64;
constexpr auto Int8    = DataType::kInt8;
constexpr auto Int32   = DataType::kInt32;
constexpr auto Int64   = DataType::kInt64;
constexpr auto UInt8   = DataType::kUInt8;

inline size_t dtype_size(DataType t)
{
    switch (t)
    {
        case DataType::kFloat32: return 4;
        case DataType::kFloat64: return 8;
        case DataType::kInt8: return 1;
        case DataType::kInt32: return 4;
        case DataType::kInt64: return 8;
        default: return 1;
    }
}

inline std::string dtype_to_string(DataType t)
{
    switch (t)
    {
        case DataType::kFloat32: return "float32";
        case DataType::kFloat64: return "float64";
        case DataType::kInt8: return "int8";
        case DataType::kInt32: return "int32";
        case DataType::kInt64: return "int64";
        default: return "uint8";
    }
}

template <typename T>
struct DataTypeTraits;
template <> struct DataTypeTraits<float> { static constexpr DataType type = DataType::kFloat32; };
template <> struct DataTypeTraits<double> { static constexpr DataType type = DataType::kFloat64; };
template <> struct DataTypeTraits<int8_t> { static constexpr DataType type = DataType::kInt8; };
template <> struct DataTypeTraits<int32_t> { static constexpr DataType type = DataType::kInt32; };
template <> struct DataTypeTraits<int64_t> { static constexpr DataType type = DataType::kInt64; };
template <> struct DataTypeTraits<uint8_t> { static constexpr DataType type = DataType::kUInt8; };
template <> struct DataTypeTraits<unsigned long> { static constexpr DataType type = DataType::kInt64; };

// The device label stays kCUDA / "cuda:N": callers written for the reference construct
// Device(DeviceType::kCUDA, id) and must keep working; here it names a gfx950 GPU.
enum class DeviceType
{
    kCPU  = 0,
    kCUDA = 1,
};

class Device
{
public:
    Device(DeviceType type = DeviceType::kCPU, int index = 0) : type_(type), index_(index) {}
    DeviceType type() const { return type_; }
    int index() const { return index_; }
    bool operator==(const Device &o) const { return type_ == o.type_ && (type_ == DeviceType::kCPU || index_ == o.index_); }
    bool operator!=(const Device &o) const { return !(*this == o); }
    std::string to_string() const
    {
        return type_ == DeviceType::kCPU ? std::string("cpu") : "cuda:" + std::to_string(index_);
    }

private:
    DeviceType type_;
    int index_;
};

// ---------------------------------------------------------------- Shape
class Shape
{
public:
    Shape() = default;
    Shape(std::initializer_list<size_t> d) : dims_(d) {}
    explicit Shape(std::vector<size_t> d) : dims_(std::move(d)) {}
    size_t size() const { return dims_.size(); }
    size_t ndims() const { return dims_.size(); }
    size_t operator[](size_t i) const { return dims_.at(i); }
    size_t elements() const
    {
        size_t n = 1;  // a 0-dim shape holds one element
        for (size_t d : dims_)
            n *= d;
        return n;
    }
    const std::vector<size_t> &dims() const { return dims_; }
    bool is_scalar() const { return dims_.empty(); }  // a 0-dim shape
    bool operator==(const Shape &o) const { return dims_ == o.dims_; }
    bool operator!=(const Shape &o) const { return dims_ != o.dims_; }
    std::string to_string() const
    {
        std::string s = "{";
        for (size_t i = 0; i < dims_.size(); ++i)
            s += (i ? ", " : "") + std::to_string(dims_[i]);
        return s + "}";
    }

private:
    std::vector<size_t> dims_;
};

inline std::ostream &operator<<(std::ostream &os, const Shape &s)
{
    return os << s.to_string();
}

// ---------------------------------------------------------------- Scalar
class Scalar
{
public:
    Scalar() : dtype_(DataType::kFloat32), f_(0), i_(0) {}
    Scalar(float v) : dtype_(DataType::kFloat32), f_(v), i_((int64_t)v) {}
    Scalar(double v) : dtype_(DataType::kFloat64), f_(v), i_((int64_t)v) {}
    Scalar(int v) : dtype_(DataType::kInt32), f_(v), i_(v) {}
    Scalar(int64_t v) : dtype_(DataType::kInt64), f_((double)v), i_(v) {}
    Scalar(size_t v) : dtype_(DataType::kInt64), f_((double)v), i_((int64_t)v) {}
    DataType dtype() const { return dtype_; }
    float to_float32() const { return is_float() ? (float)f_ : (float)i_; }
    double to_float64() const { return is_float() ? f_ : (double)i_; }
    int32_t to_int32() const { return is_float() ? (int32_t)f_ : (int32_t)i_; }
    int64_t to_int64() const { return is_float() ? (int64_t)f_ : i_; }
    template <typename T>
    T to() const
    {
        return is_float() ? static_cast<T>(f_) : static_cast<T>(i_);
    }
    bool is_float() const { return dtype_ == DataType::kFloat32 || dtype_ == DataType::kFloat64; }

private:
    DataType dtype_;
    double f_;
    int64_t i_;
};

// ---------------------------------------------------------------- TensorOptions
class TensorOptions
{
public:
    TensorOptions() = default;
    TensorOptions(DataType d) : dtype_(d) {}
    TensorOptions &dtype(DataType d)
    {
        dtype_ = d;
        return *this;
    }
    TensorOptions &device(Device d)
    {
        device_ = d;
        return *this;
    }
    TensorOptions &device(DeviceType t, int index = 0)
    {
        device_ = Device(t, index);
        return *this;
    }
    TensorOptions &requires_grad(bool r)
    {
        requires_grad_ = r;
        return *this;
    }
    DataType dtype() const { return dtype_; }
    Device device() const { return device_; }
    bool requires_grad() const { return requires_grad_; }
    bool operator==(const TensorOptions &o) const
    {
        return dtype_ == o.dtype_ && device_ == o.device_ && requires_grad_ == o.requires_grad_;
    }
    bool operator!=(const TensorOptions &o) const { return !(*this == o); }

private:
    DataType dtype_     = DataType::kFloat32;
    Device device_      = Device(DeviceType::kCPU, 0);
    bool requires_grad_ = false;
};

inline TensorOptions dtype(DataType d)
{
    return TensorOptions(d);
}
inline TensorOptions device(Device d)
{
    return TensorOptions().device(d);
}
inline TensorOptions device(DeviceType t, int index = 0)
{
    return TensorOptions().device(Device(t, index));
}
inline TensorOptions requires_grad(bool r = true)
{
    return TensorOptions().requires_grad(r);
}

// (in + 2p - k) / s + 1, truncating — include/origin/utils/conv_utils.h
inline int get_conv_outsize(int input_size, int kernel_size, int stride, int pad)
{
    return (input_size + pad * 2 - kernel_size) / stride + 1;
}
inline std::pair<int, int> pair(int v)
{
    return {v, v};
}
inline std::pair<int, int> pair(std::pair<int, int> v)
{
    return v;
}
}  // namespace origin
