// The Mat plugin boundary and its gfx950 implementation.
//
// `Mat` keeps the reference's abstract interface (include/origin/mat/mat.h:20-806) for every virtual the hot
// path's callers use; `OriginMat` is the concrete class behind `Mat_t`. Where the reference's OriginMat
// dispatches a device Mat to origin::cuda::* kernels, this one calls the C ABI of libodl_hip.so
// (include/odl_hip.h). There is no CPU compute path: a Mat on the CPU can be created, copied, reshaped, read
// and moved to the device — arithmetic on it throws. The CPU backend of the reference is this project's
// oracle and is never linked into this library.
#pragma once
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include <atomic>
#include <cstring>

#include "base.h"

namespace origin
{
constexpr int ORIGIN_BACKEND_TYPE = 0;

// Owning buffer on the host or on the device (device memory comes from a caching pool over odl_hip_malloc,
// as the reference's Storage sits on its MemoryPool, src/mat/origin/memory/*).
class Storage : public std::enable_shared_from_this<Storage>
{
public:
    static std::shared_ptr<Storage> create(size_t bytes, DeviceType type, int index = 0);
    ~Storage();
    Storage(const Storage &)            = delete;
    Storage &operator=(const Storage &) = delete;
    // Handing out the address ends the validity of the host copy below: whoever holds the pointer may write through it.
    void *data() const
    {
        host_copy_valid_ = false;
        mirror_valid_    = false;
        if (fill_pending_)
            run_pending_fill();
        return data_;
    }
    // A device buffer that is to hold one value in all of its `n` elements (zeros, ones, full): the fill kernel is not
    // queued until the first data() call. Code that only needs to know the value (a gradient seed of ones read as a
    // scalar, zeros added to zeros) asks pending_fill() and never causes the launch.
    void set_pending_fill(int dtype_code, int64_t n, const void *element, size_t element_bytes) const;
    // true while the fill has not run; *dtype_code and the element's bytes (8 at most) are returned when asked for
    bool pending_fill(int *dtype_code = nullptr, void *element = nullptr) const
    {
        if (fill_pending_ && dtype_code)
            *dtype_code = fill_dtype_;
        if (fill_pending_ && element)
            std::memcpy(element, fill_element_, sizeof(fill_element_));
        return fill_pending_;
    }
    size_t size() const { return size_; }
    // A host copy of the first bytes of a small device buffer, kept by code that has just read them back anyway (the loss
    // scalar comes to the host once, for the bad-label check, and item() is then served from here instead of a second
    // synchronising copy). Valid until the next data() call.
    void set_host_copy(const void *bytes, size_t n) const
    {
        if (n <= sizeof(host_copy_))
        {
            std::memcpy(host_copy_, bytes, n);
            host_copy_bytes_ = n;
            host_copy_valid_ = true;
        }
    }
    bool host_copy(void *dst, size_t n) const
    {
        if (!host_copy_valid_ || n > host_copy_bytes_)
            return false;
        std::memcpy(dst, host_copy_, n);
        return true;
    }
    // The least and greatest element of an integer buffer that was uploaded from the host (found by a scan of the host
    // data on its way up): whoever needs to know whether class labels lie in range then needs no trip to the device.
    // Every in-place writer of the buffer calls forget_int_range().
    void set_int_range(int64_t lo, int64_t hi) const { int_lo_ = lo, int_hi_ = hi, int_range_valid_ = true; }
    void forget_int_range() const { int_range_valid_ = false; }
    bool int_range(int64_t *lo, int64_t *hi) const
    {
        if (!int_range_valid_)
            return false;
        *lo = int_lo_, *hi = int_hi_;
        return true;
    }
    // Pinned host words that the kernel which fills this buffer also writes (the loss and its bad-label flag): once the
    // device has been synchronised the host reads them there, with no copy queued. Set after the data() call that handed
    // the buffer to that kernel; like the host copy above it stops being trusted at the next data() call. A kernel
    // recorded into a graph keeps writing the words on every replay, so they are never given back (`recorded`).
    // `stream` is the stream of the kernel that writes the words: the slot goes back to that stream's free list only.
    // `event` (may be null): recorded right behind that kernel; a reader then waits for it alone, not for the work queued
    // after it.
    void set_mirror(void *pinned_words, bool recorded, void *stream, void *event = nullptr) const
    {
        mirror_ = pinned_words, mirror_stream_ = stream, mirror_recorded_ = recorded, mirror_event_ = event;
        mirror_valid_ = pinned_words != nullptr;
    }
    // waits for the kernel that writes the mirror (its event, or the whole device when there is none) and reads `n`
    // bytes from it; false when there is none to trust
    bool read_mirror(void *dst, size_t n) const;
    DeviceType device_type() const { return type_; }
    int device_index() const { return index_; }
    std::shared_ptr<Storage> to_device(DeviceType type, int index) const;  // synchronous copy, like the reference

private:
    Storage(void *p, size_t n, size_t cap, DeviceType t, int i) : data_(p), size_(n), capacity_(cap), type_(t), index_(i) {}
    void *data_;
    size_t size_, capacity_;
    DeviceType type_;
    int index_;
    // the three flags below are flipped inside const accessors that other host threads may call on a shared buffer
    mutable std::atomic<bool> host_copy_valid_{false};
    mutable size_t host_copy_bytes_ = 0;
    mutable unsigned char host_copy_[8] = {0};
    void run_pending_fill() const;
    mutable std::atomic<bool> fill_pending_{false};
    mutable bool fill_set_while_capturing_ = false;
    mutable int fill_dtype_ = 0;
    mutable int64_t fill_n_ = 0;
    mutable unsigned char fill_element_[8] = {0};
    mutable std::atomic<bool> int_range_valid_{false};
    mutable int64_t int_lo_ = 0, int_hi_ = 0;
    mutable void *mirror_ = nullptr, *mirror_stream_ = nullptr, *mirror_event_ = nullptr;
    mutable std::atomic<bool> mirror_valid_{false};
    mutable bool mirror_recorded_ = false;
};

class Mat
{
public:
    virtual ~Mat() = default;
    // ---- lifetime / shape
    virtual std::unique_ptr<Mat> clone() const                         = 0;
    virtual std::unique_ptr<Mat> view(const Shape &shape) const        = 0;
    virtual bool is_contiguous() const                                 = 0;
    virtual std::unique_ptr<Mat> contiguous() const                    = 0;
    virtual std::unique_ptr<Mat> reshape(const Shape &shape) const     = 0;
    virtual std::unique_ptr<Mat> transpose() const                     = 0;
    virtual Shape shape() const                                        = 0;
    virtual size_t elements() const                                    = 0;
    virtual bool is_scalar() const                                     = 0;
    virtual Scalar scalar_value() const                                = 0;
    virtual void *data_ptr()                                           = 0;
    virtual int backend_type() const                                   = 0;
    virtual DataType dtype() const                                     = 0;
    virtual std::unique_ptr<Mat> to(DataType target) const             = 0;
    virtual Device device() const                                      = 0;
    virtual std::unique_ptr<Mat> to_device(Device device) const        = 0;
    virtual void print(const std::string &desc = "") const             = 0;
    // ---- arithmetic (same shape, or one single-element operand)
    virtual std::unique_ptr<Mat> operator+(const Mat &other) const     = 0;
    virtual std::unique_ptr<Mat> operator-(const Mat &other) const     = 0;
    virtual std::unique_ptr<Mat> operator*(const Mat &other) const     = 0;
    virtual std::unique_ptr<Mat> operator/(const Mat &other) const     = 0;
    virtual std::unique_ptr<Mat> operator>(const Mat &other) const     = 0;
    virtual std::unique_ptr<Mat> operator==(const Mat &other) const    = 0;
    virtual std::unique_ptr<Mat> operator!=(const Mat &other) const    = 0;
    virtual std::unique_ptr<Mat> operator<(const Mat &other) const     = 0;
    virtual std::unique_ptr<Mat> operator<=(const Mat &other) const    = 0;
    virtual std::unique_ptr<Mat> operator>=(const Mat &other) const    = 0;
    virtual std::unique_ptr<Mat> operator-() const                     = 0;
    virtual void add_inplace(const Mat &other)                         = 0;
    virtual void sub_inplace(const Mat &other)                         = 0;
    virtual void mul_inplace(const Mat &other)                         = 0;
    virtual void div_inplace(const Mat &other)                         = 0;
    virtual void neg_inplace()                                         = 0;
    virtual void exp_inplace()                                         = 0;
    virtual void log_inplace()                                         = 0;
    virtual void square_inplace()                                      = 0;
    virtual void relu_inplace()                                        = 0;
    virtual Mat &operator+=(const Mat &other)                          = 0;
    virtual Mat &operator-=(const Mat &other)                          = 0;
    virtual Mat &operator*=(const Mat &other)                          = 0;
    virtual Mat &operator/=(const Mat &other)                          = 0;
    virtual std::unique_ptr<Mat> matmul(const Mat &other) const        = 0;
    // ---- reductions / broadcast
    virtual std::unique_ptr<Mat> broadcast_to(const Shape &shape) const           = 0;
    virtual std::unique_ptr<Mat> sum_to(const Shape &shape) const                 = 0;
    virtual std::unique_ptr<Mat> sum(int axis = -1, bool keepdim = false) const   = 0;
    virtual std::unique_ptr<Mat> max(int axis = -1) const                         = 0;
    // ---- math
    virtual std::unique_ptr<Mat> exp() const                           = 0;
    virtual std::unique_ptr<Mat> log() const                           = 0;
    virtual std::unique_ptr<Mat> sqrt() const                          = 0;
    virtual std::unique_ptr<Mat> square() const                        = 0;
    virtual std::unique_ptr<Mat> pow(const Scalar &exponent) const     = 0;
    virtual std::unique_ptr<Mat> relu() const                          = 0;
    virtual std::unique_ptr<Mat> sigmoid() const                       = 0;
    virtual std::unique_ptr<Mat> silu() const                          = 0;
    virtual std::unique_ptr<Mat> sigmoid_backward(const Mat &y) const  = 0;  // this = gy, y = sigmoid(x)
    virtual std::unique_ptr<Mat> silu_backward(const Mat &x) const     = 0;  // this = gy
    virtual std::unique_ptr<Mat> upsample_backward(const Mat &gy, const Shape &x_shape, int scale_h, int scale_w,
                                                   const std::string &mode = "nearest") const = 0;
    virtual std::vector<std::unique_ptr<Mat>> split(const std::vector<size_t> &split_sizes, int dim) const = 0;
    // ---- detector forward path (mat.h:719-797 of the reference)
    virtual std::unique_ptr<Mat> upsample(const Shape &output_shape, int scale_h, int scale_w,
                                          const std::string &mode = "nearest") const = 0;
    virtual std::unique_ptr<Mat> cat(const std::vector<const Mat *> &others, int dim) const = 0;
    virtual std::unique_ptr<Mat> yolo_detect_forward(const Mat &conv_weight, const Mat *conv_bias, const Mat &grid,
                                                     const Mat &anchor_grid, float stride, int32_t num_anchors,
                                                     int32_t num_classes) const = 0;
    // ---- batch normalisation (mat.h:584-649 of the reference); num_dims 2 = [N, C], 4 = [N, C, H, W]
    struct BatchNormResult
    {
        std::unique_ptr<Mat> y, mean, var, x_norm;
    };
    virtual BatchNormResult batch_norm_forward(const Mat &gamma, const Mat &beta, const Mat &running_mean,
                                               const Mat &running_var, bool training, float eps,
                                               int num_dims) const = 0;
    virtual std::unique_ptr<Mat> batch_norm(const Mat &gamma, const Mat &beta, const Mat &running_mean,
                                            const Mat &running_var, bool training, float eps, float momentum,
                                            int num_dims) const = 0;
    virtual std::vector<std::unique_ptr<Mat>> batch_norm_backward(const Mat &gy, const Mat &gamma, const Mat &saved_mean,
                                                                  const Mat &saved_var, const Mat &saved_x_norm,
                                                                  float eps, int num_dims) const = 0;
    // ---- convolution / pooling
    virtual std::unique_ptr<Mat> im2col(std::pair<int, int> kernel_size, std::pair<int, int> stride,
                                        std::pair<int, int> pad, bool to_matrix = true) const = 0;
    virtual std::unique_ptr<Mat> col2im(const Shape &input_shape, std::pair<int, int> kernel_size,
                                        std::pair<int, int> stride, std::pair<int, int> pad,
                                        bool to_matrix = true) const                           = 0;
    virtual std::unique_ptr<Mat> conv2d(const Mat &W, const Mat *b, std::pair<int, int> stride,
                                        std::pair<int, int> pad) const                         = 0;
    virtual std::vector<std::unique_ptr<Mat>> conv2d_backward(const Mat &gy, const Mat &x, const Mat &W, const Mat *b,
                                                              std::pair<int, int> stride,
                                                              std::pair<int, int> pad) const   = 0;
    virtual std::unique_ptr<Mat> max_pool2d(std::pair<int, int> kernel_size, std::pair<int, int> stride,
                                            std::pair<int, int> pad, std::vector<size_t> *indices = nullptr) const = 0;
    virtual std::unique_ptr<Mat> max_pool2d_backward(const Mat &gy, std::pair<int, int> kernel_size,
                                                     std::pair<int, int> stride, std::pair<int, int> pad,
                                                     const std::vector<size_t> &indices) const = 0;
    // ---- indexing
    // one element by its coordinates (src/mat/origin/origin_mat.cpp:970-1039): on the device a synchronising copy of
    // that element alone
    virtual Scalar index(std::initializer_list<size_t> indices) const                   = 0;
    virtual void index_put(std::initializer_list<size_t> indices, const Scalar &value) = 0;
    virtual std::unique_ptr<Mat> gather(const Mat &indices) const                   = 0;
    virtual std::unique_ptr<Mat> one_hot(const Mat &indices, int num_classes) const = 0;
};

class OriginMat : public Mat
{
public:
    OriginMat(const Shape &shape, DataType dtype, Device device = Device());
    OriginMat(std::shared_ptr<Storage> storage, const Shape &shape, DataType dtype);
    OriginMat(const OriginMat &) = default;  // shares the storage, like the reference's copy

    // factories required of Mat_t by the core (src/core/tensor_impl.cpp:20-43)
    static std::unique_ptr<Mat> from_scalar(const Scalar &scalar, const Shape &shape, const TensorOptions &options);
    static std::unique_ptr<Mat> from_memory(const void *data, DataType user_dtype, const Shape &shape,
                                            const TensorOptions &options);
    static std::unique_ptr<Mat> randn(const Shape &shape, const TensorOptions &options = TensorOptions());
    static std::unique_ptr<Mat> zeros(const Shape &shape, const TensorOptions &options = TensorOptions());
    static std::unique_ptr<Mat> ones(const Shape &shape, const TensorOptions &options = TensorOptions());
    static std::unique_ptr<Mat> full(const Shape &shape, float value, const TensorOptions &options = TensorOptions());

    std::unique_ptr<Mat> clone() const override;
    std::unique_ptr<Mat> view(const Shape &shape) const override;
    bool is_contiguous() const override { return true; }
    std::unique_ptr<Mat> contiguous() const override;
    std::unique_ptr<Mat> reshape(const Shape &shape) const override;
    std::unique_ptr<Mat> transpose() const override;
    Shape shape() const override { return shape_; }
    size_t elements() const override { return shape_.elements(); }
    bool is_scalar() const override { return shape_.elements() == 1; }
    Scalar index(std::initializer_list<size_t> indices) const override;
    void index_put(std::initializer_list<size_t> indices, const Scalar &value) override;
    Scalar scalar_value() const override;
    void *data_ptr() override { return storage_->data(); }
    int backend_type() const override { return ORIGIN_BACKEND_TYPE; }
    DataType dtype() const override { return dtype_; }
    std::unique_ptr<Mat> to(DataType target) const override;
    Device device() const override { return Device(storage_->device_type(), storage_->device_index()); }
    std::unique_ptr<Mat> to_device(Device device) const override;
    void print(const std::string &desc = "") const override;

    std::unique_ptr<Mat> operator+(const Mat &other) const override;
    std::unique_ptr<Mat> operator-(const Mat &other) const override;
    std::unique_ptr<Mat> operator*(const Mat &other) const override;
    std::unique_ptr<Mat> operator/(const Mat &other) const override;
    std::unique_ptr<Mat> operator>(const Mat &other) const override;
    std::unique_ptr<Mat> operator==(const Mat &other) const override;
    std::unique_ptr<Mat> operator!=(const Mat &other) const override;
    std::unique_ptr<Mat> operator<(const Mat &other) const override;
    std::unique_ptr<Mat> operator<=(const Mat &other) const override;
    std::unique_ptr<Mat> operator>=(const Mat &other) const override;
    std::unique_ptr<Mat> operator-() const override;
    void add_inplace(const Mat &other) override;
    void sub_inplace(const Mat &other) override;
    void mul_inplace(const Mat &other) override;
    void div_inplace(const Mat &other) override;
    void neg_inplace() override;
    void exp_inplace() override;
    void log_inplace() override;
    void square_inplace() override;
    void relu_inplace() override;
    Mat &operator+=(const Mat &other) override;
    Mat &operator-=(const Mat &other) override;
    Mat &operator*=(const Mat &other) override;
    Mat &operator/=(const Mat &other) override;
    std::unique_ptr<Mat> matmul(const Mat &other) const override;

    std::unique_ptr<Mat> broadcast_to(const Shape &shape) const override;
    std::unique_ptr<Mat> sum_to(const Shape &shape) const override;
    std::unique_ptr<Mat> sum(int axis = -1, bool keepdim = false) const override;
    std::unique_ptr<Mat> max(int axis = -1) const override;

    std::unique_ptr<Mat> exp() const override;
    std::unique_ptr<Mat> log() const override;
    std::unique_ptr<Mat> sqrt() const override;
    std::unique_ptr<Mat> square() const override;
    std::unique_ptr<Mat> pow(const Scalar &exponent) const override;
    std::unique_ptr<Mat> relu() const override;
    std::unique_ptr<Mat> sigmoid() const override;
    std::unique_ptr<Mat> silu() const override;
    std::unique_ptr<Mat> sigmoid_backward(const Mat &y) const override;
    std::unique_ptr<Mat> silu_backward(const Mat &x) const override;
    std::unique_ptr<Mat> upsample_backward(const Mat &gy, const Shape &x_shape, int scale_h, int scale_w,
                                           const std::string &mode = "nearest") const override;
    std::vector<std::unique_ptr<Mat>> split(const std::vector<size_t> &split_sizes, int dim) const override;
    std::unique_ptr<Mat> upsample(const Shape &output_shape, int scale_h, int scale_w,
                                  const std::string &mode = "nearest") const override;
    std::unique_ptr<Mat> cat(const std::vector<const Mat *> &others, int dim) const override;
    std::unique_ptr<Mat> yolo_detect_forward(const Mat &conv_weight, const Mat *conv_bias, const Mat &grid,
                                             const Mat &anchor_grid, float stride, int32_t num_anchors,
                                             int32_t num_classes) const override;

    BatchNormResult batch_norm_forward(const Mat &gamma, const Mat &beta, const Mat &running_mean, const Mat &running_var,
                                       bool training, float eps, int num_dims) const override;
    std::unique_ptr<Mat> batch_norm(const Mat &gamma, const Mat &beta, const Mat &running_mean, const Mat &running_var,
                                    bool training, float eps, float momentum, int num_dims) const override;
    std::vector<std::unique_ptr<Mat>> batch_norm_backward(const Mat &gy, const Mat &gamma, const Mat &saved_mean,
                                                          const Mat &saved_var, const Mat &saved_x_norm, float eps,
                                                          int num_dims) const override;
    std::unique_ptr<Mat> im2col(std::pair<int, int> kernel_size, std::pair<int, int> stride, std::pair<int, int> pad,
                                bool to_matrix = true) const override;
    std::unique_ptr<Mat> col2im(const Shape &input_shape, std::pair<int, int> kernel_size, std::pair<int, int> stride,
                                std::pair<int, int> pad, bool to_matrix = true) const override;
    std::unique_ptr<Mat> conv2d(const Mat &W, const Mat *b, std::pair<int, int> stride,
                                std::pair<int, int> pad) const override;
    std::vector<std::unique_ptr<Mat>> conv2d_backward(const Mat &gy, const Mat &x, const Mat &W, const Mat *b,
                                                      std::pair<int, int> stride,
                                                      std::pair<int, int> pad) const override;
    std::unique_ptr<Mat> max_pool2d(std::pair<int, int> kernel_size, std::pair<int, int> stride, std::pair<int, int> pad,
                                    std::vector<size_t> *indices = nullptr) const override;
    std::unique_ptr<Mat> max_pool2d_backward(const Mat &gy, std::pair<int, int> kernel_size, std::pair<int, int> stride,
                                             std::pair<int, int> pad,
                                             const std::vector<size_t> &indices) const override;
    std::unique_ptr<Mat> gather(const Mat &indices) const override;
    std::unique_ptr<Mat> one_hot(const Mat &indices, int num_classes) const override;

    // ---- beyond the reference's Mat: the fused kernels the operators above Mat may use on the device
    std::unique_ptr<Mat> softmax(int axis) const;
    float softmax_cross_entropy(const Mat &target) const;                      // loss value (host)
    std::unique_ptr<Mat> softmax_cross_entropy_backward(const Mat &target, float gy) const;
    // conv2d with an activation applied in the kernel's epilogue: -1 none, 0 relu, 7 silu. Bit-identical to conv2d()
    // followed by relu() / silu().
    // `packed` (optional): the filter copy conv2d_packed_weights made for an input of this shape — for weights that stay
    // the same from call to call, so that the forward does not re-order them every time
    std::unique_ptr<Mat> conv2d_packed_weights(const Mat &W, std::pair<int, int> stride, std::pair<int, int> pad) const;
    static std::unique_ptr<Mat> conv2d_packed_weights_for(const Shape &x_shape, const Mat &W, std::pair<int, int> stride,
                                                          std::pair<int, int> pad);
    std::unique_ptr<Mat> conv2d_act(const Mat &W, const Mat *b, std::pair<int, int> stride, std::pair<int, int> pad,
                                    int activation, const Mat *packed) const;
    std::unique_ptr<Mat> conv2d_act(const Mat &W, const Mat *b, std::pair<int, int> stride, std::pair<int, int> pad,
                                    int activation) const;
    // A run of channels [c0, c0 + channels) of an NCHW float32 device tensor: one input of a concatenation, written where
    // the concatenation would copy it and read from there by what follows. The operators below take and fill such
    // runs (a whole tensor is the run {t, 0, C}); their values are those of the dense operators.
    struct ChannelRun
    {
        const OriginMat *tensor;
        size_t c0, channels;
    };
    static ChannelRun whole(const Mat &m);
    // whether conv2d_fused covers a convolution over an input run of this [N, C, H, W]
    static bool conv2d_fused_ok(const Shape &x_run_shape, const Shape &w_shape, std::pair<int, int> stride,
                                std::pair<int, int> pad);
    // y = residual + act(conv(x, W) + b), W given as the copy conv2d_packed_weights made for this input shape
    static void conv2d_fused(const ChannelRun &x, const Mat &packed, const Shape &w_shape, const Mat *b,
                             std::pair<int, int> stride, std::pair<int, int> pad, int activation, const ChannelRun *residual,
                             const ChannelRun &y);
    // two convolutions over x as one launch: `packed` and b hold both filters / biases one after the other (w_shape: the
    // two together); the first y_first.channels filters fill y_first, the others y_second
    static void conv2d_fused_pair(const ChannelRun &x, const Mat &packed, const Shape &w_shape, const Mat *b,
                                  std::pair<int, int> stride, std::pair<int, int> pad, int activation, const ChannelRun &y_first,
                                  const ChannelRun &y_second);
    static void upsample_run(const ChannelRun &x, const ChannelRun &y, int scale_h, int scale_w);
    // y's channels [(j-1)*C, j*C) = the K x K / stride 1 / padding K/2 max pool applied j times to x, j = 1..count
    static void max_pool_chain(const ChannelRun &x, int K, int count, const ChannelRun &y);
    static void copy_run(const ChannelRun &src, const ChannelRun &dst);
    // the convolution of a detect stage (this = its output [N, A*(classes+5), H, W]) decoded into rows
    // [row0, row0 + A*H*W) of out[N, rows, classes+5]: the second half of yolo_detect_forward
    void yolo_decode_into(const Mat &grid, const Mat &anchor_grid, float stride, int32_t num_anchors, int32_t num_classes,
                          Mat &out, size_t row0) const;
    // yolo_detect_forward of every stage of a head in one launch: the stages' 1x1 convolutions (x[s] a run, packed[s] the
    // filter copy conv2d_packed_weights made for it, b[s] a bias or null) decoded in their epilogues into out[N, rows,
    // classes+5], stage s behind stage s - 1. stages_ok: whether the input shapes are covered
    static bool yolo_detect_stages_ok(const std::vector<Shape> &x_run_shapes, int32_t num_anchors, int32_t num_classes);
    static void yolo_detect_stages(const std::vector<ChannelRun> &x, const std::vector<const Mat *> &packed,
                                   const std::vector<const Mat *> &b, const std::vector<const Mat *> &grid,
                                   const std::vector<const Mat *> &anchor_grid, const std::vector<float> &stride, int32_t num_anchors,
                                   int32_t num_classes, Mat &out);
    // the same for every stage of a head in one launch: conv[s] into the rows that follow those of conv[s - 1], from row 0
    static void yolo_decode_stages_into(const std::vector<const Mat *> &conv, const std::vector<const Mat *> &grid,
                                        const std::vector<const Mat *> &anchor_grid, const std::vector<float> &stride,
                                        int32_t num_anchors, int32_t num_classes, Mat &out);
    // Max pooling with the window-local indices kept in device memory (uint64 per output). The Mat interface above
    // hands them to the caller as a host vector, which costs a device-to-host copy in forward and a host-to-device
    // copy in backward (the reference's device backend pays both); the pooling operator uses this pair instead.
    std::unique_ptr<Mat> max_pool2d_device(std::pair<int, int> kernel_size, std::pair<int, int> stride,
                                           std::pair<int, int> pad, std::shared_ptr<Storage> *indices) const;
    std::unique_ptr<Mat> max_pool2d_backward_device(const Mat &gy, std::pair<int, int> kernel_size,
                                                    std::pair<int, int> stride, std::pair<int, int> pad,
                                                    const Storage &indices) const;
    // ... and with the backward of the ReLU that produced this (the pooled) tensor applied in the same pass:
    // max_pool2d_backward_device(...)->relu_backward(*this), same floats
    std::unique_ptr<Mat> max_pool2d_backward_relu_device(const Mat &gy, std::pair<int, int> kernel_size,
                                                         std::pair<int, int> stride, std::pair<int, int> pad,
                                                         const Storage &indices) const;
    // The loss and its gradient without the host round trip of the pair above: the loss stays a device scalar and the
    // upstream gradient is read from device memory. For steps recorded into a graph; an out-of-range label is not
    // reported here (the flag stays on the device).
    // unit_grad (may be null): receives the gradient for an upstream gradient of 1, written by the loss's own launch where
    // the library has such a kernel (small batches of few classes), else stays empty
    std::unique_ptr<Mat> softmax_cross_entropy_device(const Mat &target, std::unique_ptr<Mat> *unit_grad = nullptr) const;
    // the device-resident loss, with the out-of-range-label flag read back and turned into the reference's exception
    // (one small device-to-host copy; no upload of the loss afterwards)
    std::unique_ptr<Mat> softmax_cross_entropy_checked(const Mat &target, std::unique_ptr<Mat> *unit_grad = nullptr) const;
    std::unique_ptr<Mat> softmax_cross_entropy_backward_device(const Mat &target, const Mat &gy) const;
    // include/origin/mat/origin/origin_mat.h:75: a dense copy with the dimensions in the order `dims`
    std::unique_ptr<Mat> permute(const std::vector<int> &dims) const;
    // a float32 tensor made by zeros / ones / full whose fill has not been queued yet: its one value, known on the host
    bool unwritten_constant(float *value) const
    {
        int code = -1;
        unsigned char element[8];
        if (!storage_ || dtype_ != DataType::kFloat32 || !storage_->pending_fill(&code, element) || code != 0)
            return false;
        std::memcpy(value, element, sizeof(float));
        return true;
    }
    // on a loss made by softmax_cross_entropy_device / _checked: the out-of-range-label flag that lies behind the loss
    // in device memory, read back now (one small device-to-host copy; synchronises). A recorded step cannot raise the
    // reference's exception for a bad label — it contributes nothing to the loss — so a caller that replays a graph on
    // new labels looks here after the replay. False for any other tensor.
    bool loss_bad_label_flag() const;
    // overwrites this tensor's elements from host memory (the copy is queued behind the work already on the current
    // stream, which may still read them, and has landed when the call returns)
    void upload(const void *host, size_t bytes);
    // the fused Adam step written over this parameter, bias-correction factors read from device memory
    void adam_step_inplace(const Mat &grad, Mat &m, Mat &v, float beta1, float beta2, const float *device_scales, float eps,
                           float lr);
    void sgd_step_inplace(const Mat &grad, float lr);
    // overwrites this tensor's elements with another's of the same shape (a device-to-device copy on the current
    // stream): how a recorded step stores a freshly computed tensor at the address later replays read it from
    void copy_from(const Mat &src);
    // Batch norm for an operator that keeps x anyway: the forward without the x_norm output (result.x_norm is null),
    // and the backward that forms x_norm again from x (this) and the saved statistics — the same floats, 4 bytes per
    // element less written in forward and one saved activation less.
    // relu / beta_for_relu (float32 only): the layer's output passes through a ReLU on its way out, and the backward
    // takes the gradient of that ReLU's output, forming the mask again from gamma * x_norm + beta.
    BatchNormResult batch_norm_forward_no_xnorm(const Mat &gamma, const Mat &beta, const Mat &running_mean,
                                                const Mat &running_var, bool training, float eps, int num_dims,
                                                bool relu = false) const;
    std::vector<std::unique_ptr<Mat>> batch_norm_backward_from_x(const Mat &gy, const Mat &gamma, const Mat &saved_mean,
                                                                 const Mat &saved_var, float eps, int num_dims,
                                                                 const Mat *beta_for_relu = nullptr) const;
    // gy (this) times the mask x > 0, in one launch: the two kernels of ReLU::backward, same products
    std::unique_ptr<Mat> relu_backward(const Mat &x) const;
    // x . W + b with the activation applied in the product's epilogue (-1 none, 0 relu): what linear() then relu() give
    std::unique_ptr<Mat> linear_act(const Mat &W, const Mat &b, int activation) const;
    // x (this) . W + b with the bias added in the product's epilogue: the three kernels of Linear::forward
    // (matmul, broadcast_to, add), same rounding (the sum is rounded to float before the bias is added)
    std::unique_ptr<Mat> linear(const Mat &W, const Mat &b) const;
    // this += b*other, one launch (the weight-decay hook's multiply and accumulate)
    void axpy_inplace(float b, const Mat &other);
    // this = a*this + b*other, written where this lies
    void axpby_inplace(float a, float b, const Mat &other);
    // a*this + b*other in one launch (each product rounded before the sum): the running-statistics update of the
    // BatchNorm layers
    std::unique_ptr<Mat> axpby(float a, float b, const Mat &other) const;
    // fused optimizer steps (one launch each; same per-element arithmetic as the op-by-op sequences of
    // src/optim/adam.cpp:52-113 and src/optim/sgd.cpp:18-75). m and v are updated in place.
    std::unique_ptr<Mat> adam_step(const Mat &grad, Mat &m, Mat &v, float beta1, float beta2, float m_hat_scale,
                                   float v_hat_scale, float eps, float lr) const;
    std::unique_ptr<Mat> sgd_step(const Mat &grad, float lr) const;
    // The same steps over a whole list of parameters in one launch (the walk over the parameters is launch-bound: most
    // are biases of a few hundred floats). Every tensor must be float32 on the device (device_f32 tells); in_place
    // writes each parameter where it lies and returns nothing, otherwise entry i of the result is the updated parameter.
    struct AdamItem
    {
        const Mat *param, *grad;
        Mat *m, *v;
        float m_hat_scale, v_hat_scale;
        const float *device_scales;  // the two factors in device memory instead (recorded steps), or null
    };
    // weight_decay != 0: the WeightDecay hook in the same pass — every gradient becomes g + weight_decay * p first (and
    // keeps that value), then the step runs on it
    static std::vector<std::unique_ptr<Mat>> adam_step_multi(const std::vector<AdamItem> &items, float beta1, float beta2,
                                                             float eps, float lr, bool in_place, float weight_decay = 0.0f);
    static std::vector<std::unique_ptr<Mat>> sgd_step_multi(const std::vector<std::pair<const Mat *, const Mat *>> &param_grad,
                                                            float lr, bool in_place, float weight_decay = 0.0f);
    // y += a*x for every (x, y) of the list
    static void axpy_multi(float a, const std::vector<std::pair<const Mat *, Mat *>> &x_y);
    static bool device_f32(const Mat &m);
    // {gy . w^T, x^T . gy} for 2-D operands, reading w and x in place (no transposed copies)
    static std::pair<std::unique_ptr<Mat>, std::unique_ptr<Mat>> matmul_backward_2d(const Mat &x, const Mat &w,
                                                                                   const Mat &gy);
    // Backward of Linear for 2-D inputs: matmul_backward_2d's two gradients and gy summed to bias_shape ({N} or {1, N}),
    // one library call (one launch for a classifier layer); the values of the separate operators
    // Conv2d + ReLU + MaxPool2d in one pass where the library has a kernel for the layer pair (conv_relu_pool_fused):
    // the pooled tensor and the indices of conv2d_act(relu) followed by max_pool2d_device; backward of the pooling and
    // the ReLU from the pooled tensor alone (this = the pooled tensor, input_shape = the shape of the convolution's output)
    static bool conv_relu_pool_fused(const Mat &x, const Mat &W, std::pair<int, int> s, std::pair<int, int> p,
                                     std::pair<int, int> pk, std::pair<int, int> ps, std::pair<int, int> pp);
    // (the indices of these three are one byte each: they never leave the operator that asks for them)
    std::unique_ptr<Mat> conv2d_relu_max_pool2d_device(const Mat &W, const Mat *b, std::pair<int, int> s, std::pair<int, int> p,
                                                       std::pair<int, int> pk, std::pair<int, int> ps, std::pair<int, int> pp,
                                                       std::shared_ptr<Storage> *indices) const;
    std::unique_ptr<Mat> max_pool2d_device_compact(std::pair<int, int> k, std::pair<int, int> s, std::pair<int, int> p,
                                                   std::shared_ptr<Storage> *indices) const;
    std::unique_ptr<Mat> max_pool2d_backward_relu_pooled_device(const Mat &gy, const Shape &input_shape, std::pair<int, int> k,
                                                                std::pair<int, int> s, std::pair<int, int> p,
                                                                const Storage &indices) const;
    static std::vector<std::unique_ptr<Mat>> linear_backward_2d(const Mat &x, const Mat &w, const Mat &gy, const Shape &bias_shape);
    float accuracy(const Mat &target_int32) const;

    // ---- OriginMat-only helpers used by callers (origin_mat.h:442-559 in the reference)
    const std::shared_ptr<Storage> &storage() const { return storage_; }
    template <typename T>
    T *data_ptr()
    {
        return static_cast<T *>(storage_->data());
    }
    template <typename T>
    const T *data_ptr() const
    {
        return static_cast<const T *>(storage_->data());
    }
    template <typename T>
    std::vector<T> to_vector() const
    {
        std::vector<double> d = to_doubles();
        return std::vector<T>(d.begin(), d.end());
    }
    std::vector<float> to_vector() const { return to_vector<float>(); }

private:
    std::vector<double> to_doubles() const;  // synchronous D2H when on the device
    Shape shape_;
    DataType dtype_;
    std::shared_ptr<Storage> storage_;
};

using Mat_t = OriginMat;

inline std::unique_ptr<Mat> create_mat(const void *data, DataType dtype, const Shape &shape, const TensorOptions &o)
{
    return OriginMat::from_memory(data, dtype, shape, o);
}
}  // namespace origin
