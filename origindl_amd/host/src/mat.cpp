// OriginMat over the C ABI of libodl_hip.so: every device operation below is one or two calls into
// include/odl_hip.h. Validation and error text follow the reference's CPU ops (src/mat/origin/cpu/**) so that
// callers see the same exceptions; the arithmetic itself lives in the HIP library only.
#include "origin/mat.h"

#include <cmath>
#include <cstring>
#include <map>
#include <memory>
#include <unordered_map>
#include <mutex>
#include <thread>
#include <random>

#include "odl_hip.h"
#include "origin/nn.h"

namespace origin
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

// ---- the stream every launch of this layer goes to, and graph capture (per host thread)
thread_local void *t_stream = nullptr;     // nullptr = the null stream, as in the reference
thread_local bool t_capturing = false;

void *cur()
{
    return t_stream;
}

// host <-> device copies are synchronous; they cannot be part of a recorded step
void no_capture(const char *what)
{
    if (t_capturing)
        THROW_RUNTIME_ERROR("{} while a graph is being captured: a captured step may not move data to or from the host",
                            what);
}

// Caching allocator for device memory: freed blocks are kept in size bins (powers of two from 256 B up to 1 MiB,
// whole MiB above) and handed out again. All work of a thread is queued on one stream at a time (switching streams
// synchronises the device), so a block freed by the host is reused only by work queued after every kernel that
// touched it.
// While a graph is being captured, blocks come from — and return to — an arena owned by that graph: the recorded
// kernels keep their addresses for as long as the graph lives, so those blocks must never be handed to anyone
// else, not even after the tensors of the capture run have died. Inside the capture they are reused freely (the
// graph replays its nodes in recording order).
class DevicePool
{
public:
    static DevicePool &get()
    {
        static DevicePool *p = new DevicePool();  // never destroyed: outlives every Storage
        return *p;
    }
    static size_t bin(size_t bytes)
    {
        if (bytes <= 256)
            return 256;
        if (bytes <= (1u << 20))
        {
            size_t b = 256;
            while (b < bytes)
                b <<= 1;
            return b;
        }
        return (bytes + (1u << 20) - 1) & ~(size_t)((1u << 20) - 1);
    }
    struct Arena
    {
        std::map<size_t, std::vector<void *>> free_;
        ~Arena() { DevicePool::get().absorb(*this); }
    };
    void *alloc(size_t cap)
    {
        std::shared_ptr<Arena> arena;
        {
            std::lock_guard<std::mutex> lk(mu_);
            if (capture_arena_ && capture_thread_ == std::this_thread::get_id())
                arena = capture_arena_;  // only the recording thread's blocks belong to the graph
            void *p = nullptr;
            if (arena)
                p = take(arena->free_, cap);
            if (!p)
                p = take(free_, cap);
            if (p)
            {
                if (arena)
                    owner_[p] = arena;
                return p;
            }
        }
        void *p = nullptr;
        if (odl_hip_malloc(&p, cap) != ODL_OK)
        {
            // out of device memory with blocks parked in the bins: give them back and try once more
            if (!arena && odl_hip_synchronize() == ODL_OK && trim() > 0)
                check(odl_hip_malloc(&p, cap));
            else
                check(ODL_ERR_RUNTIME);
        }
        if (arena)
        {
            std::lock_guard<std::mutex> lk(mu_);
            owner_[p] = arena;
        }
        return p;
    }
    void release(void *p, size_t cap)
    {
        std::lock_guard<std::mutex> lk(mu_);
        auto it = owner_.find(p);
        if (it != owner_.end())
        {
            if (auto arena = it->second.lock())
            {
                arena->free_[cap].push_back(p);
                return;
            }
            owner_.erase(it);  // its graph is gone: an ordinary block again
        }
        free_[cap].push_back(p);
    }
    std::shared_ptr<Arena> begin_capture()
    {
        std::lock_guard<std::mutex> lk(mu_);
        if (capture_arena_)
            THROW_RUNTIME_ERROR("a graph is already being captured");
        capture_arena_ = std::make_shared<Arena>();
        capture_thread_ = std::this_thread::get_id();
        return capture_arena_;
    }
    // frees every block of the ordinary bins (the caller has synchronised the device); returns how many
    size_t trim()
    {
        std::map<size_t, std::vector<void *>> bins;
        {
            std::lock_guard<std::mutex> lk(mu_);
            bins.swap(free_);
        }
        size_t n = 0;
        for (auto &bin : bins)
            for (void *p : bin.second)
            {
                (void)odl_hip_free(p);
                ++n;
            }
        return n;
    }
    void end_capture()
    {
        std::lock_guard<std::mutex> lk(mu_);
        capture_arena_.reset();
    }

private:
    static void *take(std::map<size_t, std::vector<void *>> &bins, size_t cap)
    {
        auto it = bins.find(cap);
        if (it == bins.end() || it->second.empty())
            return nullptr;
        void *p = it->second.back();
        it->second.pop_back();
        return p;
    }
    // a dying graph's free blocks become ordinary blocks; the ones still held by tensors follow when released
    void absorb(Arena &a)
    {
        std::lock_guard<std::mutex> lk(mu_);
        for (auto &bin : a.free_)
            for (void *p : bin.second)
            {
                owner_.erase(p);
                free_[bin.first].push_back(p);
            }
        a.free_.clear();
    }
    std::mutex mu_;
    std::map<size_t, std::vector<void *>> free_;
    std::shared_ptr<Arena> capture_arena_;
    std::thread::id capture_thread_;
    std::unordered_map<void *, std::weak_ptr<Arena>> owner_;
};

const OriginMat &as_origin(const Mat &m)
{
    const auto *p = dynamic_cast<const OriginMat *>(&m);
    if (!p)
        THROW_RUNTIME_ERROR("expected an OriginMat, got backend_type={}", m.backend_type());
    return *p;
}

// a float32 Mat living on the device: the only thing the kernels compute on
const OriginMat &dev_f32(const Mat &m, const char *who)
{
    const OriginMat &o = as_origin(m);
    if (o.device().type() != DeviceType::kCUDA)
        THROW_RUNTIME_ERROR("{}: tensor is on {}; this backend computes on the GPU only (move it with .to(device))", who,
                            o.device().to_string());
    if (o.dtype() != DataType::kFloat32)
        THROW_INVALID_ARG("{}: only float32 is supported on the device, got {}", who, dtype_to_string(o.dtype()));
    return o;
}

// the convolution operators also run on float64 tensors, as the reference's do (src/mat/origin/cuda/conv/conv2d.cu:412-664)
const OriginMat &dev_real(const Mat &m, const char *who)
{
    const OriginMat &o = as_origin(m);
    if (o.device().type() != DeviceType::kCUDA)
        THROW_RUNTIME_ERROR("{}: tensor is on {}; this backend computes on the GPU only (move it with .to(device))", who,
                            o.device().to_string());
    if (o.dtype() != DataType::kFloat32 && o.dtype() != DataType::kFloat64)
        THROW_INVALID_ARG("{}: only float32 and float64 are supported on the device, got {}", who, dtype_to_string(o.dtype()));
    return o;
}

void same_dtype(const OriginMat &a, const OriginMat &b, const char *who)
{
    if (a.dtype() != b.dtype())
        THROW_INVALID_ARG("{}: operands of different element types ({} and {})", who, dtype_to_string(a.dtype()),
                          dtype_to_string(b.dtype()));
}

const float *fp(const OriginMat &m)
{
    return m.data_ptr<float>();
}

// a Mat of any element type living on the device: the elementwise, conversion and sum kernels take all six types
const OriginMat &dev_any(const Mat &m, const char *who)
{
    const OriginMat &o = as_origin(m);
    if (o.device().type() != DeviceType::kCUDA)
        THROW_RUNTIME_ERROR("{}: tensor is on {}; this backend computes on the GPU only (move it with .to(device))", who,
                            o.device().to_string());
    return o;
}

// the C ABI's element type codes are the DataType enumerators
int code(DataType dt)
{
    return static_cast<int>(dt);
}

std::unique_ptr<OriginMat> new_like(const OriginMat &ref, const Shape &shape, DataType dt = DataType::kFloat32)
{
    return std::make_unique<OriginMat>(shape, dt, ref.device());
}

struct Workspace
{
    std::shared_ptr<Storage> s;
    size_t bytes = 0;
    explicit Workspace(size_t n, int index) : bytes(n)
    {
        if (n)
            s = Storage::create(n, DeviceType::kCUDA, index);
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

void same_dtype_device(const OriginMat &a, const OriginMat &b, const char *who)
{
    if (a.dtype() != b.dtype())
        THROW_INVALID_ARG("Data type mismatch in {}: expected {} but got {}", who, dtype_to_string(a.dtype()),
                          dtype_to_string(b.dtype()));
    if (a.device() != b.device())
        THROW_INVALID_ARG("Device mismatch in {}: {} vs {}", who, a.device().to_string(), b.device().to_string());
}

Shape broadcast_shape(const OriginMat &a, const OriginMat &b, const char *who)
{
    if (a.shape() == b.shape())
        return a.shape();
    if (b.elements() == 1)
        return a.shape();
    if (a.elements() == 1)
        return b.shape();
    THROW_RUNTIME_ERROR("Complex broadcasting not yet implemented for {} operation: {} vs {}", who,
                        a.shape().to_string(), b.shape().to_string());
}

std::unique_ptr<Mat> binary(int op, const char *who, const OriginMat &a, const Mat &other, OriginMat *out = nullptr)
{
    // arithmetic and comparisons run in any element type; the fused activation gradients (op > 9) are float32 kernels
    const OriginMat &x = op <= 9 ? dev_any(a, who) : dev_f32(a, who);
    const OriginMat &y = op <= 9 ? dev_any(other, who) : dev_f32(other, who);
    same_dtype_device(x, y, who);
    const Shape rs = broadcast_shape(x, y, who);
    std::unique_ptr<OriginMat> fresh;
    OriginMat *dst = out;
    if (!dst)
    {
        fresh = new_like(x, rs, x.dtype());
        dst   = fresh.get();
    }
    else if (dst->shape() != rs)
        THROW_INVALID_ARG("Output tensor mismatch. Expected shape={}, got shape={}", rs.to_string(),
                          dst->shape().to_string());
    else if (dst->dtype() != x.dtype())
        THROW_INVALID_ARG("Output tensor mismatch. Expected dtype={}, got dtype={}", dtype_to_string(x.dtype()),
                          dtype_to_string(dst->dtype()));
    dst->storage()->forget_int_range();
    check(odl_hip_binary_dtype(op, code(x.dtype()), x.storage()->data(), (int64_t)x.elements(), y.storage()->data(),
                               (int64_t)y.elements(), dst->storage()->data(), cur()));
    return fresh;
}

std::unique_ptr<Mat> unary(int op, const char *who, const OriginMat &a, OriginMat *out = nullptr)
{
    const OriginMat &x = dev_any(a, who);
    // exp, log, sqrt, sigmoid and silu exist for the floating-point types only, as in the reference
    const bool floating = x.dtype() == DataType::kFloat32 || x.dtype() == DataType::kFloat64;
    if (!floating && !(op == 0 || op == 3 || op == 4))
        THROW_INVALID_ARG("{}: only floating-point tensors are supported, got {}", who, dtype_to_string(x.dtype()));
    std::unique_ptr<OriginMat> fresh;
    OriginMat *dst = out;
    if (!dst)
    {
        fresh = new_like(x, x.shape(), x.dtype());
        dst   = fresh.get();
    }
    dst->storage()->forget_int_range();
    check(odl_hip_unary_dtype(op, code(x.dtype()), x.storage()->data(), (int64_t)x.elements(), dst->storage()->data(),
                              cur()));
    return fresh;
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
}  // namespace

// ------------------------------------------------------------------------------------------- Storage
std::shared_ptr<Storage> Storage::create(size_t bytes, DeviceType type, int index)
{
    if (type == DeviceType::kCPU)
    {
        const size_t cap = (bytes + 127) & ~(size_t)127;
        void *p          = cap ? std::aligned_alloc(128, cap) : nullptr;
        if (cap && !p)
            THROW_RUNTIME_ERROR("host allocation of {} bytes failed", bytes);
        return std::shared_ptr<Storage>(new Storage(p, bytes, cap, type, index));
    }
    check(odl_hip_set_device(index));
    const size_t cap = DevicePool::bin(bytes ? bytes : 1);
    void *p          = DevicePool::get().alloc(cap);
    return std::shared_ptr<Storage>(new Storage(p, bytes, cap, type, index));
}

// 16-byte slots of pinned host memory, carved from 4 KiB pieces that live as long as the process. A slot is given back
// while the kernel that writes it may still be queued, so free slots are kept per stream: the next kernel to get the
// slot is then queued behind that one, and a stale write can never land after a newer one.
class MirrorPool
{
public:
    static MirrorPool &get()
    {
        static MirrorPool *pool = new MirrorPool();
        return *pool;
    }
    void *take(void *stream)
    {
        std::lock_guard<std::mutex> lock(mutex_);
        auto &mine = free_[stream];
        if (mine.empty())
        {
            if (fresh_.empty())
            {
                void *piece = nullptr;
                check(odl_hip_host_alloc(&piece, 4096));
                for (size_t off = 0; off < 4096; off += 16)
                    fresh_.push_back(static_cast<char *>(piece) + off);
            }
            mine.push_back(fresh_.back());
            fresh_.pop_back();
        }
        void *slot = mine.back();
        mine.pop_back();
        return slot;
    }
    // the event that goes with a slot (made when first asked for, kept for the life of the process)
    void *event_of(void *slot)
    {
        std::lock_guard<std::mutex> lock(mutex_);
        void *&e = events_[slot];
        if (!e)
            check(odl_hip_event_create(&e));
        return e;
    }
    void give(void *slot, void *stream)
    {
        std::lock_guard<std::mutex> lock(mutex_);
        free_[stream].push_back(slot);
    }

private:
    std::mutex mutex_;
    std::vector<void *> fresh_;                    // never handed to a kernel yet
    std::map<void *, std::vector<void *>> free_;   // by the stream of the kernel that last wrote the slot
    std::map<void *, void *> events_;              // slot -> its event
};

// The buffers of this thread whose fill may still be pending. A capture must not record the fill of a buffer that was
// made before it (a replay would then reset the buffer every time), so begin_capture queues those fills first.
thread_local std::vector<std::weak_ptr<const Storage>> t_pending_fills;

void Storage::set_pending_fill(int dtype_code, int64_t n, const void *element, size_t element_bytes) const
{
    std::memset(fill_element_, 0, sizeof(fill_element_));
    std::memcpy(fill_element_, element, element_bytes < sizeof(fill_element_) ? element_bytes : sizeof(fill_element_));
    fill_dtype_ = dtype_code, fill_n_ = n;
    fill_set_while_capturing_ = t_capturing;
    fill_pending_ = n > 0;
    if (!fill_pending_ || t_capturing)
        return;
    if (t_pending_fills.size() >= 4096)
    {
        // drop the entries that are gone or done
        size_t kept = 0;
        for (auto &w : t_pending_fills)
        {
            auto st = w.lock();
            if (st && st->pending_fill())
                t_pending_fills[kept++] = w;
        }
        t_pending_fills.resize(kept);
    }
    t_pending_fills.push_back(weak_from_this());
}

void Storage::run_pending_fill() const
{
    // begin_capture runs the fills this thread had pending; one that is still pending here was made by another thread
    // (or dropped from the list). Recording it would make every replay reset the buffer.
    if (t_capturing && !fill_set_while_capturing_)
        THROW_RUNTIME_ERROR("a zeros/ones/full buffer made before the capture began (on another thread?) is first used "
                            "inside it: touch it before begin_capture");
    fill_pending_ = false;
    check(odl_hip_fill_dtype(data_, fill_dtype_, fill_n_, fill_element_, cur()));
}

static void run_pending_fills_of_this_thread()
{
    std::vector<std::weak_ptr<const Storage>> list;
    list.swap(t_pending_fills);
    for (auto &w : list)
        if (auto st = w.lock())
            if (st->pending_fill())
                (void)st->data();
}

bool Storage::read_mirror(void *dst, size_t n) const
{
    if (!mirror_valid_ || n > 8)
        return false;
    if (mirror_event_)
        check(odl_hip_event_synchronize(mirror_event_));  // the loss kernel is done; what was queued after it may still run
    else
        check(odl_hip_device_synchronize());
    std::memcpy(dst, mirror_, n);
    return true;
}

Storage::~Storage()
{
    if (mirror_ && !mirror_recorded_)
        MirrorPool::get().give(mirror_, mirror_stream_);
    if (!data_)
        return;
    if (type_ == DeviceType::kCPU)
        std::free(data_);
    else
        DevicePool::get().release(data_, capacity_);
}

std::shared_ptr<Storage> Storage::to_device(DeviceType type, int index) const
{
    auto dst = Storage::create(size_, type, index);
    if (size_ == 0)
        return dst;
    if (fill_pending_)
        run_pending_fill();
    if (type_ == DeviceType::kCPU && type == DeviceType::kCPU)
        std::memcpy(dst->data(), data_, size_);
    else if (type_ == DeviceType::kCPU)
    {
        no_capture("host-to-device copy");
        check(odl_hip_memcpy_h2d(dst->data(), data_, size_, cur()));
    }
    else if (type == DeviceType::kCPU)
    {
        no_capture("device-to-host copy");
        check(odl_hip_memcpy_d2h(dst->data(), data_, size_));
    }
    else
    {
        check(odl_hip_memcpy_d2d(dst->data(), data_, size_, cur()));
    }
    return dst;
}

// ------------------------------------------------------------------------------------------ factories
OriginMat::OriginMat(const Shape &shape, DataType dtype, Device device)
    : shape_(shape), dtype_(dtype), storage_(Storage::create(shape.elements() * dtype_size(dtype), device.type(),
                                                             device.index()))
{}

OriginMat::OriginMat(std::shared_ptr<Storage> storage, const Shape &shape, DataType dtype)
    : shape_(shape), dtype_(dtype), storage_(std::move(storage))
{}

namespace
{
// writes n values of `dt` converted from doubles into a host buffer
void store_as(void *dst, DataType dt, const double *src, size_t n)
{
    for (size_t i = 0; i < n; ++i)
    {
        switch (dt)
        {
            case DataType::kFloat32: static_cast<float *>(dst)[i] = (float)src[i]; break;
            case DataType::kFloat64: static_cast<double *>(dst)[i] = src[i]; break;
            case DataType::kInt8: static_cast<int8_t *>(dst)[i] = (int8_t)src[i]; break;
            case DataType::kInt32: static_cast<int32_t *>(dst)[i] = (int32_t)src[i]; break;
            case DataType::kInt64: static_cast<int64_t *>(dst)[i] = (int64_t)src[i]; break;
            default: static_cast<uint8_t *>(dst)[i] = (uint8_t)src[i]; break;
        }
    }
}

double load_as(const void *src, DataType dt, size_t i)
{
    switch (dt)
    {
        case DataType::kFloat32: return static_cast<const float *>(src)[i];
        case DataType::kFloat64: return static_cast<const double *>(src)[i];
        case DataType::kInt8: return static_cast<const int8_t *>(src)[i];
        case DataType::kInt32: return static_cast<const int32_t *>(src)[i];
        case DataType::kInt64: return (double)static_cast<const int64_t *>(src)[i];
        default: return static_cast<const uint8_t *>(src)[i];
    }
}

// class labels come up from the host as int32 / int64: their range is noted on the way
void note_int_range(const Storage &st, const void *host, DataType dt, size_t n)
{
    if ((dt != DataType::kInt32 && dt != DataType::kInt64) || n == 0)
        return;
    int64_t lo = INT64_MAX, hi = INT64_MIN;
    for (size_t i = 0; i < n; ++i)
    {
        const int64_t v = dt == DataType::kInt64 ? static_cast<const int64_t *>(host)[i] : static_cast<const int32_t *>(host)[i];
        lo = v < lo ? v : lo, hi = v > hi ? v : hi;
    }
    st.set_int_range(lo, hi);
}

std::unique_ptr<Mat> upload_new(const void *host, DataType dt, const Shape &shape, Device dev)
{
    auto m = std::make_unique<OriginMat>(shape, dt, dev);
    const size_t bytes = shape.elements() * dtype_size(dt);
    if (bytes == 0)
        return m;
    if (dev.type() == DeviceType::kCPU)
        std::memcpy(m->data_ptr(), host, bytes);
    else
    {
        no_capture("host-to-device copy");
        check(odl_hip_memcpy_h2d(m->data_ptr(), host, bytes, cur()));
        note_int_range(*m->storage(), host, dt, shape.elements());
    }
    return m;
}
}  // namespace

std::unique_ptr<Mat> OriginMat::from_memory(const void *data, DataType user_dtype, const Shape &shape,
                                            const TensorOptions &options)
{
    const size_t n = shape.elements();
    if (user_dtype == options.dtype())
        return upload_new(data, user_dtype, shape, options.device());
    std::vector<double> tmp(n);
    for (size_t i = 0; i < n; ++i)
        tmp[i] = load_as(data, user_dtype, i);
    std::vector<char> conv(n * dtype_size(options.dtype()));
    store_as(conv.data(), options.dtype(), tmp.data(), n);
    return upload_new(conv.data(), options.dtype(), shape, options.device());
}

std::unique_ptr<Mat> OriginMat::from_scalar(const Scalar &scalar, const Shape &shape, const TensorOptions &options)
{
    const size_t n = shape.elements();
    if (options.device().type() == DeviceType::kCUDA)
    {
        // one element converted on the host the way the host path below converts all of them, then a fill kernel
        auto m = std::make_unique<OriginMat>(shape, options.dtype(), options.device());
        const double v = scalar.to_float64();
        char element[8] = {0};
        if (options.dtype() == DataType::kInt64)
        {
            const int64_t w = scalar.to_int64();
            std::memcpy(element, &w, sizeof(w));
        }
        else
            store_as(element, options.dtype(), &v, 1);
        // the kernel is queued when the buffer is first asked for
        m->storage()->set_pending_fill(code(options.dtype()), (int64_t)n, element, dtype_size(options.dtype()));
        return m;
    }
    std::vector<double> tmp(n, scalar.to_float64());
    std::vector<char> conv(n * dtype_size(options.dtype()));
    store_as(conv.data(), options.dtype(), tmp.data(), n);
    return upload_new(conv.data(), options.dtype(), shape, options.device());
}

std::unique_ptr<Mat> OriginMat::randn(const Shape &shape, const TensorOptions &options)
{
    // like the reference (src/mat/origin/cpu/factory.cpp:27-56): mt19937 + normal_distribution on the host,
    // seeded from random_device — parameter initialisation, not part of the hot path
    static std::mt19937 gen{std::random_device{}()};
    std::normal_distribution<float> dist(0.f, 1.f);
    std::vector<float> host(shape.elements());
    for (auto &v : host)
        v = dist(gen);
    return from_memory(host.data(), DataType::kFloat32, shape, options);
}

std::unique_ptr<Mat> OriginMat::zeros(const Shape &shape, const TensorOptions &options)
{
    return from_scalar(Scalar(0.0f), shape, options);
}

std::unique_ptr<Mat> OriginMat::ones(const Shape &shape, const TensorOptions &options)
{
    return from_scalar(Scalar(1.0f), shape, options);
}

std::unique_ptr<Mat> OriginMat::full(const Shape &shape, float value, const TensorOptions &options)
{
    return from_scalar(Scalar(value), shape, options);
}

// ------------------------------------------------------------------------------------ lifetime / shape
std::unique_ptr<Mat> OriginMat::clone() const
{
    return std::make_unique<OriginMat>(storage_->to_device(storage_->device_type(), storage_->device_index()), shape_,
                                       dtype_);
}

std::unique_ptr<Mat> OriginMat::view(const Shape &shape) const
{
    if (shape.elements() != shape_.elements())
        THROW_INVALID_ARG("view: cannot view shape {} as {}", shape_.to_string(), shape.to_string());
    return std::make_unique<OriginMat>(storage_, shape, dtype_);  // zero-copy: same storage
}

std::unique_ptr<Mat> OriginMat::contiguous() const
{
    return std::make_unique<OriginMat>(*this);
}

std::unique_ptr<Mat> OriginMat::reshape(const Shape &shape) const
{
    if (shape.elements() != shape_.elements())
        THROW_INVALID_ARG("reshape: cannot reshape {} ({} elements) to {} ({} elements)", shape_.to_string(),
                          shape_.elements(), shape.to_string(), shape.elements());
    return view(shape);
}

std::unique_ptr<Mat> OriginMat::transpose() const
{
    if (shape_.size() < 2)
        return clone();
    if (dtype_ != DataType::kFloat32)
    {
        // every other element type: the same copy as a permutation of the last two dimensions
        std::vector<int> order(shape_.size());
        for (size_t i = 0; i < order.size(); ++i)
            order[i] = (int)i;
        std::swap(order[order.size() - 2], order[order.size() - 1]);
        return permute(order);
    }
    const OriginMat &x = dev_f32(*this, "transpose");
    std::vector<size_t> d = shape_.dims();
    const size_t rows = d[d.size() - 2], cols = d[d.size() - 1];
    std::swap(d[d.size() - 2], d[d.size() - 1]);
    auto out = new_like(x, Shape(d));
    const int64_t outer = (int64_t)(shape_.elements() / ((rows * cols) != 0 ? rows * cols : 1));
    check(odl_hip_transpose(fp(x), out->data_ptr<float>(), outer, (int64_t)rows, (int64_t)cols, cur()));
    return out;
}

std::vector<double> OriginMat::to_doubles() const
{
    const size_t n = shape_.elements();
    std::vector<double> out(n);
    if (n == 0)
        return out;
    std::vector<char> host;
    const void *src = nullptr;
    if (storage_->device_type() != DeviceType::kCPU && n == 1)
    {
        host.resize(dtype_size(dtype_));
        // a scalar that has been read back already, or one whose kernel also wrote it to pinned host memory
        if (storage_->host_copy(host.data(), host.size()) || (!t_capturing && storage_->read_mirror(host.data(), host.size())))
            src = host.data();
    }
    if (!src)
        src = storage_->data();
    if (storage_->device_type() != DeviceType::kCPU && src != host.data())
    {
        host.resize(n * dtype_size(dtype_));
        no_capture("device-to-host copy");
        check(odl_hip_memcpy_d2h(host.data(), storage_->data(), host.size()));
        src = host.data();
    }
    for (size_t i = 0; i < n; ++i)
        out[i] = load_as(src, dtype_, i);
    return out;
}

Scalar OriginMat::scalar_value() const
{
    if (shape_.elements() != 1)
        THROW_INVALID_ARG("scalar_value: tensor has {} elements", shape_.elements());
    const double v = to_doubles()[0];
    switch (dtype_)
    {
        case DataType::kFloat32: return Scalar((float)v);
        case DataType::kFloat64: return Scalar(v);
        case DataType::kInt64: return Scalar((int64_t)v);
        default: return Scalar((int)v);
    }
}

namespace
{
// element offset of a coordinate list in a contiguous tensor; the checks and messages of origin_mat.cpp:970-990
size_t element_offset(const Shape &shape, std::initializer_list<size_t> indices)
{
    if (indices.size() != shape.size())
        THROW_INVALID_ARG("Index count ({}) does not match tensor dimension ({}). Shape: {}", indices.size(), shape.size(),
                          shape.to_string());
    size_t offset = 0, i = 0;
    for (size_t idx : indices)
    {
        if (idx >= shape[i])
            THROW_INVALID_ARG("Index {} out of range for dimension {} (size: {}). Shape: {}", idx, i, shape[i],
                              shape.to_string());
        offset = offset * shape[i] + idx;
        ++i;
    }
    return offset;
}
}  // namespace

Scalar OriginMat::index(std::initializer_list<size_t> indices) const
{
    const size_t offset = element_offset(shape_, indices), width = dtype_size(dtype_);
    alignas(8) char element[8];
    const char *src = static_cast<const char *>(storage_->data()) + offset * width;
    if (storage_->device_type() == DeviceType::kCPU)
        std::memcpy(element, src, width);
    else
    {
        no_capture("device-to-host copy");
        check(odl_hip_synchronize());
        check(odl_hip_memcpy_d2h(element, src, width));
    }
    const double v = load_as(element, dtype_, 0);
    switch (dtype_)
    {
        case DataType::kFloat32: return Scalar((float)v);
        case DataType::kFloat64: return Scalar(v);
        case DataType::kInt64: return Scalar((int64_t)v);
        default: return Scalar((int)v);
    }
}

void OriginMat::index_put(std::initializer_list<size_t> indices, const Scalar &value)
{
    const size_t offset = element_offset(shape_, indices), width = dtype_size(dtype_);
    alignas(8) char element[8];
    const double v = value.to_float64();
    if (dtype_ == DataType::kInt64)  // keeps all 64 bits
    {
        const int64_t w = value.to_int64();
        std::memcpy(element, &w, sizeof(w));
    }
    else
        store_as(element, dtype_, &v, 1);
    storage_->forget_int_range();
    char *dst = static_cast<char *>(storage_->data()) + offset * width;
    if (storage_->device_type() == DeviceType::kCPU)
        std::memcpy(dst, element, width);
    else
    {
        no_capture("host-to-device copy");
        check(odl_hip_synchronize());
        check(odl_hip_memcpy_h2d(dst, element, width, cur()));
    }
}

std::unique_ptr<Mat> OriginMat::to(DataType target) const
{
    if (target == dtype_)
        return std::make_unique<OriginMat>(*this);
    if (device().type() == DeviceType::kCUDA)
    {
        // a cast kernel on the current stream: no host round trip, so it can sit inside a recorded step
        auto out = std::make_unique<OriginMat>(shape_, target, device());
        check(odl_hip_convert(storage_->data(), code(dtype_), out->storage()->data(), code(target), (int64_t)elements(),
                              cur()));
        return out;
    }
    const std::vector<double> d = to_doubles();
    std::vector<char> conv(d.size() * dtype_size(target));
    store_as(conv.data(), target, d.data(), d.size());
    return upload_new(conv.data(), target, shape_, device());
}

std::unique_ptr<Mat> OriginMat::to_device(Device dev) const
{
    if (dev == device())
        return std::make_unique<OriginMat>(*this);
    auto moved = storage_->to_device(dev.type(), dev.index());
    if (storage_->device_type() == DeviceType::kCPU && dev.type() == DeviceType::kCUDA)
        note_int_range(*moved, storage_->data(), dtype_, elements());
    return std::make_unique<OriginMat>(std::move(moved), shape_, dtype_);
}

void OriginMat::print(const std::string &desc) const
{
    const std::vector<double> d = to_doubles();
    std::cout << desc << (desc.empty() ? "" : " ") << "Mat" << shape_.to_string() << " " << dtype_to_string(dtype_) << " "
              << device().to_string() << " [";
    for (size_t i = 0; i < d.size() && i < 16; ++i)
        std::cout << (i ? ", " : "") << d[i];
    std::cout << (d.size() > 16 ? ", ...]" : "]") << std::endl;
}

// ------------------------------------------------------------------------------------------ arithmetic
std::unique_ptr<Mat> OriginMat::operator+(const Mat &o) const { return binary(0, "add", *this, o); }
std::unique_ptr<Mat> OriginMat::operator-(const Mat &o) const { return binary(1, "subtract", *this, o); }
std::unique_ptr<Mat> OriginMat::operator*(const Mat &o) const { return binary(2, "multiply", *this, o); }
std::unique_ptr<Mat> OriginMat::operator/(const Mat &o) const { return binary(3, "divide", *this, o); }
std::unique_ptr<Mat> OriginMat::operator>(const Mat &o) const { return binary(4, "gt", *this, o); }
std::unique_ptr<Mat> OriginMat::operator==(const Mat &o) const { return binary(5, "eq", *this, o); }
std::unique_ptr<Mat> OriginMat::operator!=(const Mat &o) const { return binary(6, "ne", *this, o); }
std::unique_ptr<Mat> OriginMat::operator<(const Mat &o) const { return binary(7, "lt", *this, o); }
std::unique_ptr<Mat> OriginMat::operator<=(const Mat &o) const { return binary(8, "le", *this, o); }
std::unique_ptr<Mat> OriginMat::operator>=(const Mat &o) const { return binary(9, "ge", *this, o); }
std::unique_ptr<Mat> OriginMat::operator-() const { return unary(3, "negate", *this); }

void OriginMat::add_inplace(const Mat &o)
{
    // zeros that have not been written yet, added to zeros that have not been written yet, are just that
    if (const auto *other = dynamic_cast<const OriginMat *>(&o))
    {
        int ca = 0, cb = 0;
        unsigned char ea[8], eb[8];
        const unsigned char none[8] = {0};
        if (storage_ && other->storage_ && shape_ == other->shape_ && dtype_ == other->dtype_ &&
            storage_->pending_fill(&ca, ea) && other->storage_->pending_fill(&cb, eb) && ca == cb &&
            std::memcmp(ea, none, 8) == 0 && std::memcmp(eb, none, 8) == 0)
            return;
    }
    binary(0, "add", *this, o, this);
}
void OriginMat::sub_inplace(const Mat &o) { binary(1, "subtract", *this, o, this); }
void OriginMat::mul_inplace(const Mat &o) { binary(2, "multiply", *this, o, this); }
void OriginMat::div_inplace(const Mat &o) { binary(3, "divide", *this, o, this); }
void OriginMat::neg_inplace() { unary(3, "negate", *this, this); }
void OriginMat::exp_inplace() { unary(1, "exp", *this, this); }
void OriginMat::log_inplace() { unary(2, "log", *this, this); }
void OriginMat::square_inplace() { unary(4, "square", *this, this); }
void OriginMat::relu_inplace() { unary(0, "relu", *this, this); }
Mat &OriginMat::operator+=(const Mat &o) { add_inplace(o); return *this; }
Mat &OriginMat::operator-=(const Mat &o) { sub_inplace(o); return *this; }
Mat &OriginMat::operator*=(const Mat &o) { mul_inplace(o); return *this; }
Mat &OriginMat::operator/=(const Mat &o) { div_inplace(o); return *this; }

std::unique_ptr<Mat> OriginMat::exp() const { return unary(1, "exp", *this); }
std::unique_ptr<Mat> OriginMat::log() const { return unary(2, "log", *this); }
std::unique_ptr<Mat> OriginMat::sqrt() const { return unary(5, "sqrt", *this); }
std::unique_ptr<Mat> OriginMat::square() const { return unary(4, "square", *this); }
std::unique_ptr<Mat> OriginMat::relu() const { return unary(0, "relu", *this); }
std::unique_ptr<Mat> OriginMat::sigmoid() const { return unary(6, "sigmoid", *this); }
std::unique_ptr<Mat> OriginMat::silu() const { return unary(7, "silu", *this); }

std::unique_ptr<Mat> OriginMat::sigmoid_backward(const Mat &y) const
{
    if (y.shape() != shape_)
        THROW_INVALID_ARG("sigmoid_backward: gy and y must have same shape and dtype");
    return binary(10, "sigmoid_backward", *this, y);
}

std::unique_ptr<Mat> OriginMat::silu_backward(const Mat &x) const
{
    if (x.shape() != shape_)
        THROW_INVALID_ARG("silu_backward: gy and x must have same shape and dtype");
    return binary(11, "silu_backward", *this, x);
}

std::unique_ptr<Mat> OriginMat::upsample_backward(const Mat &gym, const Shape &xs, int scale_h, int scale_w,
                                                  const std::string &) const
{
    const OriginMat &gy = dev_any(gym, "upsample_backward");
    if (gy.shape().size() != 4)
        THROW_INVALID_ARG("Upsample backward: gradient must be 4D (N, C, OH, OW), but got shape {}", gy.shape().to_string());
    if (xs.size() != 4)
        THROW_INVALID_ARG("Upsample backward: x_shape must be 4D (N, C, H, W), but got shape {}", xs.to_string());
    auto gx = new_like(gy, xs, gy.dtype());
    check(odl_hip_upsample_nearest_backward_dtype(code(gy.dtype()), gy.storage()->data(), (int64_t)xs[0], (int64_t)xs[1],
                                                  (int64_t)xs[2], (int64_t)xs[3], (int64_t)gy.shape()[2], (int64_t)gy.shape()[3],
                                                  scale_h, scale_w, gx->storage()->data(), cur()));
    return gx;
}

// ---- batch normalisation (src/mat/origin/cpu/normalization/batch_norm.cpp:31-258, 279-418: same checks, same text)
namespace
{
struct BnShape
{
    int64_t N, C, P;
};

BnShape bn_check(const char *who, const OriginMat &x, int num_dims, const Mat &gamma, const Mat &beta, const Mat &rm,
                 const Mat &rv)
{
    if (x.shape().size() != (size_t)num_dims)
        THROW_INVALID_ARG("{}: x must have {} dimensions, but got shape {}", who, num_dims, x.shape().to_string());
    if (num_dims != 2 && num_dims != 4)
        THROW_INVALID_ARG("{}: num_dims must be 2 or 4, but got {}", who, num_dims);
    const size_t C = x.shape()[1];
    if (gamma.shape() != Shape({C}) || beta.shape() != Shape({C}) || rm.shape() != Shape({C}) || rv.shape() != Shape({C}))
        THROW_INVALID_ARG("{}: gamma, beta, running_mean, running_var must have shape ({})", who, C);
    if (x.dtype() != DataType::kFloat32 && x.dtype() != DataType::kFloat64)
        THROW_INVALID_ARG("{}: input x must be float32 or float64, but got {}", who, static_cast<int>(x.dtype()));
    if (gamma.dtype() != x.dtype() || beta.dtype() != x.dtype() || rm.dtype() != x.dtype() || rv.dtype() != x.dtype())
        THROW_INVALID_ARG("{}: all inputs (x, gamma, beta, running_mean, running_var) must have the same "
                          "floating-point dtype", who);
    return BnShape{(int64_t)x.shape()[0], (int64_t)C,
                   num_dims == 4 ? (int64_t)(x.shape()[2] * x.shape()[3]) : (int64_t)1};
}

const double *dp(const OriginMat &m)
{
    return static_cast<const double *>(m.storage()->data());
}
double *dp(OriginMat &m)
{
    return static_cast<double *>(m.storage()->data());
}

// float64 tensors take the same path on doubles (src/mat/origin/cuda/normalization/batch_norm.cu:497-560)
Mat::BatchNormResult bn_forward_f64(const OriginMat &self, const BnShape &s, const Mat &gamma, const Mat &beta,
                                    const Mat &rm_, const Mat &rv_, bool training, float eps, bool with_x_norm)
{
    const OriginMat &x = dev_any(self, "batch_norm"), &g = dev_any(gamma, "batch_norm"), &b = dev_any(beta, "batch_norm");
    const OriginMat &rm = dev_any(rm_, "batch_norm"), &rv = dev_any(rv_, "batch_norm");
    Mat::BatchNormResult r;
    auto y = new_like(x, x.shape(), DataType::kFloat64);
    auto mean = new_like(x, Shape({(size_t)s.C}), DataType::kFloat64), var = new_like(x, Shape({(size_t)s.C}), DataType::kFloat64);
    std::unique_ptr<OriginMat> xn;
    if (with_x_norm)
        xn = new_like(x, x.shape(), DataType::kFloat64);
    check(odl_hip_batch_norm_forward_f64(dp(x), dp(g), dp(b), dp(rm), dp(rv), training ? 1 : 0, (double)eps, s.N, s.C, s.P,
                                         dp(*y), dp(*mean), dp(*var), xn ? dp(*xn) : nullptr, cur()));
    r.y = std::move(y), r.mean = std::move(mean), r.var = std::move(var);
    if (xn)
        r.x_norm = std::move(xn);
    return r;
}

std::vector<std::unique_ptr<Mat>> bn_backward_f64(const OriginMat &self, const Mat &gym, const Mat &xn_or_x, bool from_x,
                                                  const Mat &gamma, const Mat &saved_mean, const Mat &saved_var, float eps,
                                                  int num_dims)
{
    const OriginMat &x = dev_any(self, "batch_norm_backward"), &gy = dev_any(gym, "batch_norm_backward");
    const OriginMat &src = dev_any(xn_or_x, "batch_norm_backward"), &g = dev_any(gamma, "batch_norm_backward");
    const OriginMat &sm = dev_any(saved_mean, "batch_norm_backward"), &sv = dev_any(saved_var, "batch_norm_backward");
    const size_t C = x.shape()[1];
    const int64_t N = (int64_t)x.shape()[0], P = num_dims == 4 ? (int64_t)(x.shape()[2] * x.shape()[3]) : 1;
    auto gx = new_like(x, x.shape(), DataType::kFloat64);
    auto dgamma = new_like(x, Shape({C}), DataType::kFloat64), dbeta = new_like(x, Shape({C}), DataType::kFloat64);
    if (N > 0)
        check(odl_hip_batch_norm_backward_f64(dp(gy), dp(src), from_x ? 1 : 0, dp(g), dp(sm), dp(sv), (double)eps, N,
                                              (int64_t)C, P, dp(*gx), dp(*dgamma), dp(*dbeta), cur()));
    std::vector<std::unique_ptr<Mat>> outs;
    outs.push_back(std::move(gx)), outs.push_back(std::move(dgamma)), outs.push_back(std::move(dbeta));
    return outs;
}
}  // namespace

Mat::BatchNormResult OriginMat::batch_norm_forward(const Mat &gamma, const Mat &beta, const Mat &running_mean,
                                                   const Mat &running_var, bool training, float eps,
                                                   int num_dims) const
{
    const BnShape s = bn_check("batch_norm", *this, num_dims, gamma, beta, running_mean, running_var);
    if (dtype_ == DataType::kFloat64)
        return bn_forward_f64(*this, s, gamma, beta, running_mean, running_var, training, eps, true);
    const OriginMat &x = dev_f32(*this, "batch_norm");
    const OriginMat &g = dev_f32(gamma, "batch_norm"), &b = dev_f32(beta, "batch_norm");
    const OriginMat &rm = dev_f32(running_mean, "batch_norm"), &rv = dev_f32(running_var, "batch_norm");
    BatchNormResult r;
    auto y = new_like(x, shape_), xn = new_like(x, shape_);
    auto mean = new_like(x, Shape({(size_t)s.C})), var = new_like(x, Shape({(size_t)s.C}));
    Workspace ws(training ? odl_hip_batch_norm_workspace_bytes(s.N, s.C, s.P) : 0, device().index());
    check(odl_hip_batch_norm_forward(fp(x), fp(g), fp(b), fp(rm), fp(rv), training ? 1 : 0, eps, s.N, s.C, s.P,
                                     y->data_ptr<float>(), mean->data_ptr<float>(), var->data_ptr<float>(),
                                     xn->data_ptr<float>(), ws.ptr(), ws.bytes, cur()));
    r.y = std::move(y), r.mean = std::move(mean), r.var = std::move(var), r.x_norm = std::move(xn);
    return r;
}

Mat::BatchNormResult OriginMat::batch_norm_forward_no_xnorm(const Mat &gamma, const Mat &beta, const Mat &running_mean,
                                                            const Mat &running_var, bool training, float eps,
                                                            int num_dims, bool relu) const
{
    const BnShape s = bn_check("batch_norm", *this, num_dims, gamma, beta, running_mean, running_var);
    if (dtype_ == DataType::kFloat64)
    {
        if (relu)
            THROW_RUNTIME_ERROR("batch_norm: the form with the ReLU folded in takes float32 tensors only");
        return bn_forward_f64(*this, s, gamma, beta, running_mean, running_var, training, eps, false);
    }
    const OriginMat &x = dev_f32(*this, "batch_norm");
    const OriginMat &g = dev_f32(gamma, "batch_norm"), &b = dev_f32(beta, "batch_norm");
    const OriginMat &rm = dev_f32(running_mean, "batch_norm"), &rv = dev_f32(running_var, "batch_norm");
    BatchNormResult r;
    auto y = new_like(x, shape_);
    auto mean = new_like(x, Shape({(size_t)s.C})), var = new_like(x, Shape({(size_t)s.C}));
    Workspace ws(training ? odl_hip_batch_norm_workspace_bytes(s.N, s.C, s.P) : 0, device().index());
    if (relu)
        check(odl_hip_batch_norm_relu_forward(fp(x), fp(g), fp(b), fp(rm), fp(rv), training ? 1 : 0, eps, s.N, s.C, s.P,
                                              y->data_ptr<float>(), mean->data_ptr<float>(), var->data_ptr<float>(),
                                              ws.ptr(), ws.bytes, cur()));
    else
        check(odl_hip_batch_norm_forward(fp(x), fp(g), fp(b), fp(rm), fp(rv), training ? 1 : 0, eps, s.N, s.C, s.P,
                                         y->data_ptr<float>(), mean->data_ptr<float>(), var->data_ptr<float>(), nullptr,
                                         ws.ptr(), ws.bytes, cur()));
    r.y = std::move(y), r.mean = std::move(mean), r.var = std::move(var);
    return r;
}

std::vector<std::unique_ptr<Mat>> OriginMat::batch_norm_backward_from_x(const Mat &gym, const Mat &gamma,
                                                                        const Mat &saved_mean, const Mat &saved_var,
                                                                        float eps, int num_dims,
                                                                        const Mat *beta_for_relu) const
{
    if (shape_.size() != (size_t)num_dims || (num_dims != 2 && num_dims != 4))
        THROW_INVALID_ARG("batch_norm_backward: x must have {} dimensions (2 or 4), but got shape {}", num_dims,
                          shape_.to_string());
    const size_t C = shape_[1];
    if (gym.shape() != shape_ || gamma.shape() != Shape({C}) || saved_mean.shape() != Shape({C}) ||
        saved_var.shape() != Shape({C}))
        THROW_INVALID_ARG("batch_norm_backward: shape mismatch");
    if (beta_for_relu && beta_for_relu->shape() != Shape({C}))
        THROW_INVALID_ARG("batch_norm_backward: shape mismatch");
    if (dtype_ == DataType::kFloat64)
    {
        if (beta_for_relu)
            THROW_RUNTIME_ERROR("batch_norm_backward: the form with the ReLU folded in takes float32 tensors only");
        return bn_backward_f64(*this, gym, *this, true, gamma, saved_mean, saved_var, eps, num_dims);
    }
    const OriginMat &x = dev_f32(*this, "batch_norm_backward");
    const OriginMat &gy = dev_f32(gym, "batch_norm_backward"), &g = dev_f32(gamma, "batch_norm_backward");
    const OriginMat &sm = dev_f32(saved_mean, "batch_norm_backward"), &sv = dev_f32(saved_var, "batch_norm_backward");
    const int64_t N = (int64_t)shape_[0], P = num_dims == 4 ? (int64_t)(shape_[2] * shape_[3]) : 1;
    auto gx = new_like(x, shape_);
    auto dgamma = new_like(x, Shape({C})), dbeta = new_like(x, Shape({C}));
    Workspace ws(odl_hip_batch_norm_workspace_bytes(N, (int64_t)C, P), device().index());
    if (beta_for_relu)
        check(odl_hip_batch_norm_relu_backward_from_x(fp(gy), fp(x), fp(g), fp(dev_f32(*beta_for_relu, "batch_norm_backward")),
                                                      fp(sm), fp(sv), eps, N, (int64_t)C, P, gx->data_ptr<float>(),
                                                      dgamma->data_ptr<float>(), dbeta->data_ptr<float>(), ws.ptr(),
                                                      ws.bytes, cur()));
    else
        check(odl_hip_batch_norm_backward_from_x(fp(gy), fp(x), fp(g), fp(sm), fp(sv), eps, N, (int64_t)C, P,
                                                 gx->data_ptr<float>(), dgamma->data_ptr<float>(),
                                                 dbeta->data_ptr<float>(), ws.ptr(), ws.bytes, cur()));
    std::vector<std::unique_ptr<Mat>> outs;
    outs.push_back(std::move(gx)), outs.push_back(std::move(dgamma)), outs.push_back(std::move(dbeta));
    return outs;
}

std::unique_ptr<Mat> OriginMat::batch_norm(const Mat &gamma, const Mat &beta, const Mat &running_mean,
                                           const Mat &running_var, bool training, float eps, float, int num_dims) const
{
    const BnShape s = bn_check("batch_norm", *this, num_dims, gamma, beta, running_mean, running_var);
    if (dtype_ == DataType::kFloat64)
        return std::move(bn_forward_f64(*this, s, gamma, beta, running_mean, running_var, training, eps, false).y);
    const OriginMat &x = dev_f32(*this, "batch_norm");
    const OriginMat &g = dev_f32(gamma, "batch_norm"), &b = dev_f32(beta, "batch_norm");
    const OriginMat &rm = dev_f32(running_mean, "batch_norm"), &rv = dev_f32(running_var, "batch_norm");
    auto y = new_like(x, shape_);
    auto mean = new_like(x, Shape({(size_t)s.C})), var = new_like(x, Shape({(size_t)s.C}));
    Workspace ws(training ? odl_hip_batch_norm_workspace_bytes(s.N, s.C, s.P) : 0, device().index());
    check(odl_hip_batch_norm_forward(fp(x), fp(g), fp(b), fp(rm), fp(rv), training ? 1 : 0, eps, s.N, s.C, s.P,
                                     y->data_ptr<float>(), mean->data_ptr<float>(), var->data_ptr<float>(), nullptr,
                                     ws.ptr(), ws.bytes, cur()));
    return y;
}

std::vector<std::unique_ptr<Mat>> OriginMat::batch_norm_backward(const Mat &gym, const Mat &gamma, const Mat &saved_mean,
                                                                 const Mat &saved_var, const Mat &saved_x_norm, float eps,
                                                                 int num_dims) const
{
    if (shape_.size() != (size_t)num_dims)
        THROW_INVALID_ARG("batch_norm_backward: x must have {} dimensions, but got shape {}", num_dims, shape_.to_string());
    if (num_dims != 2 && num_dims != 4)
        THROW_INVALID_ARG("batch_norm_backward: num_dims must be 2 or 4, but got {}", num_dims);
    const size_t C = shape_[1];
    if (gym.shape() != shape_ || gamma.shape() != Shape({C}) || saved_mean.shape() != Shape({C}) ||
        saved_var.shape() != Shape({C}) || saved_x_norm.shape() != shape_)
        THROW_INVALID_ARG("batch_norm_backward: shape mismatch");
    if (dtype() != DataType::kFloat32 && dtype() != DataType::kFloat64)
        THROW_INVALID_ARG("batch_norm_backward: input x must be float32 or float64, but got {}", static_cast<int>(dtype()));
    if (gym.dtype() != dtype() || gamma.dtype() != dtype() || saved_mean.dtype() != dtype() ||
        saved_var.dtype() != dtype() || saved_x_norm.dtype() != dtype())
        THROW_INVALID_ARG("batch_norm_backward: all inputs (gy, x, gamma, saved_mean, saved_var, saved_x_norm) must "
                          "have the same floating-point dtype");
    if (dtype_ == DataType::kFloat64)
        return bn_backward_f64(*this, gym, saved_x_norm, false, gamma, saved_mean, saved_var, eps, num_dims);
    const OriginMat &x = dev_f32(*this, "batch_norm_backward");
    const OriginMat &gy = dev_f32(gym, "batch_norm_backward"), &g = dev_f32(gamma, "batch_norm_backward");
    const OriginMat &sv = dev_f32(saved_var, "batch_norm_backward"), &xn = dev_f32(saved_x_norm, "batch_norm_backward");
    const int64_t N = (int64_t)shape_[0], P = num_dims == 4 ? (int64_t)(shape_[2] * shape_[3]) : 1;
    auto gx = new_like(x, shape_);
    auto dgamma = new_like(x, Shape({C})), dbeta = new_like(x, Shape({C}));
    Workspace ws(odl_hip_batch_norm_workspace_bytes(N, (int64_t)C, P), device().index());
    check(odl_hip_batch_norm_backward(fp(gy), fp(g), fp(sv), fp(xn), eps, N, (int64_t)C, P, gx->data_ptr<float>(),
                                      dgamma->data_ptr<float>(), dbeta->data_ptr<float>(), ws.ptr(), ws.bytes, cur()));
    std::vector<std::unique_ptr<Mat>> outs;
    outs.push_back(std::move(gx)), outs.push_back(std::move(dgamma)), outs.push_back(std::move(dbeta));
    return outs;
}

std::unique_ptr<Mat> OriginMat::relu_backward(const Mat &x) const
{
    return binary(12, "relu_backward", dev_f32(*this, "relu_backward"), x);
}

std::unique_ptr<Mat> OriginMat::linear(const Mat &W_, const Mat &b_) const
{
    return linear_act(W_, b_, -1);
}

std::unique_ptr<Mat> OriginMat::linear_act(const Mat &W_, const Mat &b_, int activation) const
{
    const OriginMat &x = dev_f32(*this, "linear"), &W = dev_f32(W_, "linear"), &b = dev_f32(b_, "linear");
    if (shape_.size() != 2 || W.shape().size() != 2 || shape_[1] != W.shape()[0] || b.elements() != W.shape()[1])
        THROW_INVALID_ARG("linear: x {} . W {} + b {} do not fit", shape_.to_string(), W.shape().to_string(),
                          b.shape().to_string());
    const int64_t M = shape_[0], K = shape_[1], N = W.shape()[1];
    auto y = new_like(x, Shape{(size_t)M, (size_t)N});
    Workspace ws(odl_hip_sgemm_workspace_bytes(0, 0, M, N, K, 0), device().index());
    check(odl_hip_linear_act(fp(x), fp(W), fp(b), M, N, K, activation, y->data_ptr<float>(), ws.ptr(), ws.bytes, cur()));
    return y;
}

void OriginMat::axpby_inplace(float a, float b, const Mat &other)
{
    const OriginMat &x = dev_f32(*this, "axpby"), &y = dev_f32(other, "axpby");
    if (x.shape() != y.shape())
        THROW_INVALID_ARG("axpby: shape mismatch {} vs {}", x.shape().to_string(), y.shape().to_string());
    float *p = const_cast<float *>(fp(x));
    check(odl_hip_axpby(a, p, b, fp(y), (int64_t)elements(), p, cur()));
}

void OriginMat::axpy_inplace(float b, const Mat &other)
{
    const OriginMat &x = dev_f32(*this, "axpy"), &y = dev_f32(other, "axpy");
    if (x.shape() != y.shape())
        THROW_INVALID_ARG("axpy: shape mismatch {} vs {}", x.shape().to_string(), y.shape().to_string());
    float *p = const_cast<float *>(fp(x));
    check(odl_hip_axpby(1.0f, p, b, fp(y), (int64_t)elements(), p, cur()));
}

std::unique_ptr<Mat> OriginMat::axpby(float a, float b, const Mat &other) const
{
    const OriginMat &x = dev_f32(*this, "axpby"), &y = dev_f32(other, "axpby");
    if (x.shape() != y.shape())
        THROW_INVALID_ARG("axpby: shape mismatch {} vs {}", x.shape().to_string(), y.shape().to_string());
    auto o = new_like(x, shape_);
    check(odl_hip_axpby(a, fp(x), b, fp(y), (int64_t)elements(), o->data_ptr<float>(), cur()));
    return o;
}

std::vector<std::unique_ptr<Mat>> OriginMat::split(const std::vector<size_t> &sizes, int dim) const
{
    const OriginMat &x = dev_any(*this, "split");
    if (dim < 0 || (size_t)dim >= shape_.size())
        THROW_RUNTIME_ERROR("split: dimension {} out of range for {} dimensions", dim, shape_.size());
    size_t total = 0;
    for (size_t s : sizes)
        total += s;
    if (total != shape_[dim])
        THROW_RUNTIME_ERROR("split: sizes sum to {}, but dimension {} has {} elements", total, dim, shape_[dim]);
    int64_t outer, ax, inner;
    split_axis(shape_, dim, outer, ax, inner);
    std::vector<std::unique_ptr<Mat>> parts;
    int64_t off = 0;
    for (size_t sz : sizes)
    {
        std::vector<size_t> d = shape_.dims();
        d[dim] = sz;
        auto piece = new_like(x, Shape(d), x.dtype());
        check(odl_hip_slice_axis_dtype(code(x.dtype()), x.storage()->data(), outer, ax, inner, off, (int64_t)sz,
                                       piece->storage()->data(), cur()));
        off += (int64_t)sz;
        parts.push_back(std::move(piece));
    }
    return parts;
}

// ------------------------------------------------------------------------------------ detector forward path
std::unique_ptr<Mat> OriginMat::upsample(const Shape &output_shape, int scale_h, int scale_w, const std::string &) const
{
    const OriginMat &x = dev_any(*this, "upsample");
    if (shape_.size() != 4)
        THROW_INVALID_ARG("Upsample: input must be 4D (N, C, H, W), but got shape {}", shape_.to_string());
    if (output_shape.size() != 4)
        THROW_INVALID_ARG("Upsample: output_shape must be 4D (N, C, OH, OW), but got shape {}", output_shape.to_string());
    auto y = new_like(x, output_shape, x.dtype());
    check(odl_hip_upsample_nearest_dtype(code(x.dtype()), x.storage()->data(), (int64_t)shape_[0], (int64_t)shape_[1],
                                         (int64_t)shape_[2], (int64_t)shape_[3], (int64_t)output_shape[2], (int64_t)output_shape[3],
                                         scale_h, scale_w, y->storage()->data(), cur()));
    return y;
}

std::unique_ptr<Mat> OriginMat::cat(const std::vector<const Mat *> &others, int dim) const
{
    std::vector<const OriginMat *> in{&dev_any(*this, "cat")};
    for (const Mat *m : others)
    {
        if (!m)
            THROW_RUNTIME_ERROR("cat: null input");
        in.push_back(&dev_any(*m, "cat"));
        if (in.back()->dtype() != dtype())
            THROW_INVALID_ARG("cat: inputs of different element types ({} and {})", dtype_to_string(dtype()),
                              dtype_to_string(in.back()->dtype()));
    }
    if (in.size() == 1)
        return std::make_unique<OriginMat>(*this);  // shape/cat.cpp:29-33: a single input is returned as it is
    if (dim < 0 || (size_t)dim >= shape_.size())
        THROW_RUNTIME_ERROR("cat: dimension {} out of range for {} dimensions", dim, shape_.size());
    size_t total = 0;
    std::vector<const void *> ptrs;
    std::vector<int64_t> sizes;
    for (const OriginMat *m : in)
    {
        const Shape s = m->shape();
        if (s.size() != shape_.size())
            THROW_RUNTIME_ERROR("cat: all inputs must have same number of dimensions");
        for (size_t d = 0; d < s.size(); ++d)
            if (d != (size_t)dim && s[d] != shape_[d])
                THROW_RUNTIME_ERROR("cat: dimension {} mismatch: {} vs {}", d, s[d], shape_[d]);
        if (m->device() != device())
            THROW_INVALID_ARG("cat: inputs live on different devices");
        total += s[dim];
        ptrs.push_back(m->storage()->data());
        sizes.push_back((int64_t)s[dim]);
    }
    std::vector<size_t> od = shape_.dims();
    od[dim] = total;
    const Shape os(od);
    int64_t outer, ax, inner;
    split_axis(os, dim, outer, ax, inner);
    auto y = new_like(*in[0], os, dtype());
    check(odl_hip_cat_dtype(code(dtype()), ptrs.data(), sizes.data(), (int)ptrs.size(), outer, inner, y->storage()->data(), cur()));
    return y;
}

std::unique_ptr<Mat> OriginMat::yolo_detect_forward(const Mat &conv_weight, const Mat *conv_bias, const Mat &grid,
                                                    const Mat &anchor_grid, float stride, int32_t num_anchors,
                                                    int32_t num_classes) const
{
    const OriginMat &x = dev_f32(*this, "yolo_detect_forward");
    if (shape_.size() != 4)
        THROW_INVALID_ARG("yolo_detect_forward: input must be 4D (N, C, H, W), but got shape {}", shape_.to_string());
    const OriginMat &w = dev_f32(conv_weight, "yolo_detect_forward");
    const OriginMat *b = conv_bias ? &dev_f32(*conv_bias, "yolo_detect_forward") : nullptr;
    const OriginMat &g = dev_f32(grid, "yolo_detect_forward");
    const OriginMat &ag = dev_f32(anchor_grid, "yolo_detect_forward");
    const int64_t N = shape_[0], C = shape_[1], H = shape_[2], W = shape_[3];
    const int64_t CI = num_classes + 5;
    const Shape ws_ = w.shape();
    if (ws_.size() != 4 || (int64_t)ws_[0] != num_anchors * CI || (int64_t)ws_[1] != C || ws_[2] != 1 || ws_[3] != 1)
        THROW_INVALID_ARG("yolo_detect_forward: conv weight {} does not match [{}, {}, 1, 1]", ws_.to_string(),
                          num_anchors * CI, C);
    const Shape as = ag.shape();
    const int64_t aH = as.size() >= 3 ? (int64_t)as[2] : H, aW = as.size() >= 4 ? (int64_t)as[3] : W;
    auto y = new_like(x, Shape{(size_t)N, (size_t)(H * W * num_anchors), (size_t)CI});
    Workspace ws(odl_hip_yolo_detect_workspace_bytes(N, C, H, W, num_anchors, num_classes), device().index());
    check(odl_hip_yolo_detect_forward(fp(x), fp(w), b ? fp(*b) : nullptr, fp(g), (int64_t)g.elements(), fp(ag),
                                      (int64_t)ag.elements(), aH, aW, N, C, H, W, stride, num_anchors, num_classes,
                                      y->data_ptr<float>(), ws.ptr(), ws.bytes, cur()));
    return y;
}

namespace
{
struct RunPtr
{
    float *data;
    int64_t image_stride, N, C, H, W;
};

RunPtr run_ptr(const OriginMat::ChannelRun &r, const char *who)
{
    if (!r.tensor)
        THROW_INVALID_ARG("{}: null tensor in a channel run", who);
    const OriginMat &t = dev_f32(*r.tensor, who);
    const Shape &s = t.shape();
    if (s.size() != 4 || r.c0 + r.channels > s[1] || r.channels == 0)
        THROW_INVALID_ARG("{}: channels [{}, {}) do not lie in a 4D tensor of shape {}", who, r.c0, r.c0 + r.channels, s.to_string());
    const int64_t plane = (int64_t)(s[2] * s[3]);
    return RunPtr{const_cast<float *>(fp(t)) + (int64_t)r.c0 * plane, (int64_t)s[1] * plane, (int64_t)s[0], (int64_t)r.channels,
                  (int64_t)s[2], (int64_t)s[3]};
}
}  // namespace

OriginMat::ChannelRun OriginMat::whole(const Mat &m)
{
    const OriginMat &t = as_origin(m);
    return ChannelRun{&t, 0, t.shape().size() == 4 ? t.shape()[1] : 0};
}

bool OriginMat::conv2d_fused_ok(const Shape &xs, const Shape &ws, std::pair<int, int> s, std::pair<int, int> p)
{
    if (xs.size() != 4 || ws.size() != 4 || xs[1] != ws[1])
        return false;
    return odl_hip_conv2d_fused_ok((int64_t)xs[0], (int64_t)xs[1], (int64_t)xs[2], (int64_t)xs[3], (int64_t)ws[0], (int)ws[2],
                                   (int)ws[3], s.first, s.second, p.first, p.second) == 1;
}

void OriginMat::conv2d_fused(const ChannelRun &xr, const Mat &packed_m, const Shape &ws, const Mat *bm, std::pair<int, int> s,
                             std::pair<int, int> p, int activation, const ChannelRun *rr, const ChannelRun &yr)
{
    const RunPtr x = run_ptr(xr, "conv2d"), y = run_ptr(yr, "conv2d");
    if (ws.size() != 4 || (int64_t)ws[1] != x.C || (int64_t)ws[0] != y.C)
        THROW_INVALID_ARG("conv2d: filter {} does not map {} channels to {}", ws.to_string(), x.C, y.C);
    const int KH = (int)ws[2], KW = (int)ws[3];
    const int OH = get_conv_outsize((int)x.H, KH, s.first, p.first), OW = get_conv_outsize((int)x.W, KW, s.second, p.second);
    if (y.N != x.N || y.H != OH || y.W != OW)
        THROW_INVALID_ARG("conv2d: the output run is [{}, {}, {}, {}], the convolution gives [{}, {}, {}, {}]", y.N, y.C, y.H, y.W,
                          x.N, y.C, OH, OW);
    const OriginMat &pk = dev_f32(packed_m, "conv2d");
    const size_t want = odl_hip_conv2d_packed_weights_bytes(x.N, x.C, x.H, x.W, y.C, KH, KW, s.first, s.second, p.first, p.second);
    if (pk.elements() * sizeof(float) != want)
        THROW_INVALID_ARG("conv2d: the packed filter has {} bytes, this shape's kernel reads {}", pk.elements() * sizeof(float), want);
    const float *bias = nullptr;
    if (bm)
    {
        const OriginMat &b = dev_f32(*bm, "conv2d");
        if (b.shape().size() != 1 || (int64_t)b.shape()[0] != y.C)
            THROW_INVALID_ARG("conv2d: b must be 1D with size {}, but got shape {}", y.C, b.shape().to_string());
        bias = fp(b);
    }
    const float *res = nullptr;
    int64_t res_stride = 0;
    if (rr)
    {
        const RunPtr r = run_ptr(*rr, "conv2d");
        if (r.N != y.N || r.C != y.C || r.H != y.H || r.W != y.W)
            THROW_INVALID_ARG("conv2d: the residual run does not have the output's shape");
        res = r.data, res_stride = r.image_stride;
    }
    check(odl_hip_conv2d_fused(x.data, x.image_stride, fp(pk), bias, x.N, x.C, x.H, x.W, y.C, KH, KW, s.first, s.second, p.first,
                               p.second, activation, res, res_stride, y.data, y.image_stride, cur()));
}

void OriginMat::conv2d_fused_pair(const ChannelRun &xr, const Mat &packed_m, const Shape &ws, const Mat *bm, std::pair<int, int> s,
                                  std::pair<int, int> p, int activation, const ChannelRun &y1r, const ChannelRun &y2r)
{
    const RunPtr x = run_ptr(xr, "conv2d"), y1 = run_ptr(y1r, "conv2d"), y2 = run_ptr(y2r, "conv2d");
    if (ws.size() != 4 || (int64_t)ws[1] != x.C || (int64_t)ws[0] != y1.C + y2.C)
        THROW_INVALID_ARG("conv2d: filters {} do not map {} channels to {} + {}", ws.to_string(), x.C, y1.C, y2.C);
    const int KH = (int)ws[2], KW = (int)ws[3];
    const int OH = get_conv_outsize((int)x.H, KH, s.first, p.first), OW = get_conv_outsize((int)x.W, KW, s.second, p.second);
    if (y1.N != x.N || y1.H != OH || y1.W != OW || y2.N != x.N || y2.H != OH || y2.W != OW)
        THROW_INVALID_ARG("conv2d: an output run does not have the convolution's [{}, *, {}, {}]", x.N, OH, OW);
    const OriginMat &pk = dev_f32(packed_m, "conv2d");
    const int64_t OC = (int64_t)ws[0];
    const size_t want = odl_hip_conv2d_packed_weights_bytes(x.N, x.C, x.H, x.W, OC, KH, KW, s.first, s.second, p.first, p.second);
    if (pk.elements() * sizeof(float) != want)
        THROW_INVALID_ARG("conv2d: the packed filter has {} bytes, this shape's kernel reads {}", pk.elements() * sizeof(float), want);
    const float *bias = nullptr;
    if (bm)
    {
        const OriginMat &b = dev_f32(*bm, "conv2d");
        if (b.shape().size() != 1 || (int64_t)b.shape()[0] != OC)
            THROW_INVALID_ARG("conv2d: b must be 1D with size {}, but got shape {}", OC, b.shape().to_string());
        bias = fp(b);
    }
    check(odl_hip_conv2d_fused_pair(x.data, x.image_stride, fp(pk), bias, x.N, x.C, x.H, x.W, OC, y1.C, KH, KW, s.first, s.second,
                                    p.first, p.second, activation, y1.data, y1.image_stride, y2.data, y2.image_stride, cur()));
}

void OriginMat::upsample_run(const ChannelRun &xr, const ChannelRun &yr, int sh, int sw)
{
    const RunPtr x = run_ptr(xr, "upsample"), y = run_ptr(yr, "upsample");
    if (x.N != y.N || x.C != y.C)
        THROW_INVALID_ARG("upsample: the runs differ in batch or channels");
    check(odl_hip_upsample_nearest_view(x.data, x.image_stride, x.N, x.C, x.H, x.W, y.H, y.W, sh, sw, y.data, y.image_stride, cur()));
}

void OriginMat::max_pool_chain(const ChannelRun &xr, int K, int count, const ChannelRun &yr)
{
    const RunPtr x = run_ptr(xr, "max_pool2d"), y = run_ptr(yr, "max_pool2d");
    if (x.N != y.N || x.C * count != y.C || x.H != y.H || x.W != y.W)
        THROW_INVALID_ARG("max_pool2d: the output run must hold {} stages of the input run's shape", count);
    check(odl_hip_max_pool2d_chain(x.data, x.image_stride, x.N, x.C, x.H, x.W, K, count, y.data, y.image_stride, cur()));
}

void OriginMat::copy_run(const ChannelRun &sr, const ChannelRun &dr)
{
    const RunPtr s = run_ptr(sr, "cat"), d = run_ptr(dr, "cat");
    if (s.N != d.N || s.C != d.C || s.H != d.H || s.W != d.W)
        THROW_INVALID_ARG("cat: the runs differ in shape");
    check(odl_hip_copy_images(s.data, s.image_stride, d.data, d.image_stride, s.N, s.C * s.H * s.W, cur()));
}

void OriginMat::yolo_decode_into(const Mat &grid, const Mat &anchor_grid, float stride, int32_t num_anchors, int32_t num_classes,
                                 Mat &out_m, size_t row0) const
{
    const OriginMat &conv = dev_f32(*this, "yolo_detect_forward");
    const OriginMat &g = dev_f32(grid, "yolo_detect_forward");
    const OriginMat &ag = dev_f32(anchor_grid, "yolo_detect_forward");
    const OriginMat &out = dev_f32(out_m, "yolo_detect_forward");
    const int64_t CI = num_classes + 5;
    if (shape_.size() != 4 || (int64_t)shape_[1] != num_anchors * CI)
        THROW_INVALID_ARG("yolo_detect_forward: the stage's convolution must be [N, {}, H, W], got {}", num_anchors * CI, shape_.to_string());
    const int64_t N = shape_[0], H = shape_[2], W = shape_[3];
    const Shape &os = out.shape();
    if (os.size() != 3 || (int64_t)os[0] != N || (int64_t)os[2] != CI || row0 + (size_t)(num_anchors * H * W) > os[1])
        THROW_INVALID_ARG("yolo_detect_forward: rows [{}, {}) do not lie in an output of shape {}", row0, row0 + num_anchors * H * W,
                          os.to_string());
    const Shape as = ag.shape();
    const int64_t aH = as.size() >= 3 ? (int64_t)as[2] : H, aW = as.size() >= 4 ? (int64_t)as[3] : W;
    check(odl_hip_yolo_decode(fp(conv), fp(g), (int64_t)g.elements(), fp(ag), (int64_t)ag.elements(), aH, aW, N, H, W, stride,
                              num_anchors, num_classes, const_cast<float *>(fp(out)) + (int64_t)row0 * CI, (int64_t)(os[1] * os[2]),
                              cur()));
}

bool OriginMat::yolo_detect_stages_ok(const std::vector<Shape> &xs, int32_t num_anchors, int32_t num_classes)
{
    const size_t S = xs.size();
    if (S == 0 || S > 4)
        return false;
    int64_t C[4], H[4], W[4];
    for (size_t s = 0; s < S; ++s)
    {
        if (xs[s].size() != 4 || xs[s][0] != xs[0][0])
            return false;
        C[s] = xs[s][1], H[s] = xs[s][2], W[s] = xs[s][3];
    }
    return odl_hip_yolo_detect_stages_ok((int)S, (int64_t)xs[0][0], C, H, W, num_anchors, num_classes) == 1;
}

void OriginMat::yolo_detect_stages(const std::vector<ChannelRun> &xr, const std::vector<const Mat *> &packed,
                                   const std::vector<const Mat *> &bm, const std::vector<const Mat *> &grid,
                                   const std::vector<const Mat *> &anchor_grid, const std::vector<float> &stride, int32_t num_anchors,
                                   int32_t num_classes, Mat &out_m)
{
    const size_t S = xr.size();
    if (S == 0 || S > 4 || packed.size() != S || bm.size() != S || grid.size() != S || anchor_grid.size() != S || stride.size() != S)
        THROW_INVALID_ARG("yolo_detect_forward: 1 to 4 stages with a filter copy, a bias (or null), a grid, an anchor grid and a stride each, got {}", S);
    const OriginMat &out = dev_f32(out_m, "yolo_detect_forward");
    const int64_t CI = num_classes + 5, OC = num_anchors * CI;
    const Shape &os = out.shape();
    if (os.size() != 3 || (int64_t)os[2] != CI)
        THROW_INVALID_ARG("yolo_detect_forward: the output must be [N, rows, {}], got {}", CI, os.to_string());
    const int64_t N = os[0];
    const float *xp[4], *pp[4], *bp[4], *gp[4], *ap[4];
    float *op[4];
    int64_t xs[4], ge[4], ae[4], aH[4], aW[4], C[4], H[4], W[4];
    size_t row0 = 0;
    for (size_t s = 0; s < S; ++s)
    {
        const RunPtr x = run_ptr(xr[s], "yolo_detect_forward");
        if (x.N != N)
            THROW_INVALID_ARG("yolo_detect_forward: stage {} has {} images, the output {}", s, x.N, N);
        if (!packed[s] || !grid[s] || !anchor_grid[s])
            THROW_INVALID_ARG("yolo_detect_forward: stage {} lacks one of filter copy / grid / anchor grid", s);
        const OriginMat &pk = dev_f32(*packed[s], "yolo_detect_forward");
        const size_t want = odl_hip_conv2d_packed_weights_bytes(x.N, x.C, x.H, x.W, OC, 1, 1, 1, 1, 0, 0);
        if (want == 0 || pk.elements() * sizeof(float) != want)
            THROW_INVALID_ARG("yolo_detect_forward: the packed filter has {} bytes, this shape's kernel reads {}", pk.elements() * sizeof(float), want);
        bp[s] = nullptr;
        if (bm[s])
        {
            const OriginMat &b = dev_f32(*bm[s], "yolo_detect_forward");
            if (b.shape().size() != 1 || (int64_t)b.shape()[0] != OC)
                THROW_INVALID_ARG("yolo_detect_forward: b must be 1D with size {}, but got shape {}", OC, b.shape().to_string());
            bp[s] = fp(b);
        }
        const OriginMat &g = dev_f32(*grid[s], "yolo_detect_forward");
        const OriginMat &ag = dev_f32(*anchor_grid[s], "yolo_detect_forward");
        if (row0 + (size_t)(num_anchors * x.H * x.W) > os[1])
            THROW_INVALID_ARG("yolo_detect_forward: rows [{}, {}) do not lie in an output of shape {}", row0,
                              row0 + num_anchors * x.H * x.W, os.to_string());
        const Shape as = ag.shape();
        aH[s] = as.size() >= 3 ? (int64_t)as[2] : x.H, aW[s] = as.size() >= 4 ? (int64_t)as[3] : x.W;
        xp[s] = x.data, xs[s] = x.image_stride, pp[s] = fp(pk), gp[s] = fp(g), ap[s] = fp(ag);
        ge[s] = (int64_t)g.elements(), ae[s] = (int64_t)ag.elements(), C[s] = x.C, H[s] = x.H, W[s] = x.W;
        op[s] = const_cast<float *>(fp(out)) + (int64_t)row0 * CI;
        row0 += (size_t)(num_anchors * x.H * x.W);
    }
    check(odl_hip_yolo_detect_stages_forward((int)S, xp, xs, pp, bp, gp, ge, ap, ae, aH, aW, N, C, H, W, stride.data(), num_anchors,
                                             num_classes, op, (int64_t)(os[1] * os[2]), cur()));
}

void OriginMat::yolo_decode_stages_into(const std::vector<const Mat *> &conv_m, const std::vector<const Mat *> &grid,
                                        const std::vector<const Mat *> &anchor_grid, const std::vector<float> &stride,
                                        int32_t num_anchors, int32_t num_classes, Mat &out_m)
{
    const size_t S = conv_m.size();
    if (S == 0 || S > 4 || grid.size() != S || anchor_grid.size() != S || stride.size() != S)
        THROW_INVALID_ARG("yolo_detect_forward: 1 to 4 stages with a grid, an anchor grid and a stride each, got {}", S);
    const OriginMat &out = dev_f32(out_m, "yolo_detect_forward");
    const int64_t CI = num_classes + 5;
    const Shape &os = out.shape();
    if (os.size() != 3 || (int64_t)os[2] != CI)
        THROW_INVALID_ARG("yolo_detect_forward: the output must be [N, rows, {}], got {}", CI, os.to_string());
    const int64_t N = os[0];
    const float *cp[4], *gp[4], *ap[4];
    float *op[4];
    int64_t ge[4], ae[4], aH[4], aW[4], H[4], W[4];
    size_t row0 = 0;
    for (size_t s = 0; s < S; ++s)
    {
        const OriginMat &conv = dev_f32(*conv_m[s], "yolo_detect_forward");
        const OriginMat &g = dev_f32(*grid[s], "yolo_detect_forward");
        const OriginMat &ag = dev_f32(*anchor_grid[s], "yolo_detect_forward");
        const Shape &cs = conv.shape();
        if (cs.size() != 4 || (int64_t)cs[0] != N || (int64_t)cs[1] != num_anchors * CI)
            THROW_INVALID_ARG("yolo_detect_forward: the stage's convolution must be [{}, {}, H, W], got {}", N, num_anchors * CI,
                              cs.to_string());
        H[s] = cs[2], W[s] = cs[3];
        if (row0 + (size_t)(num_anchors * H[s] * W[s]) > os[1])
            THROW_INVALID_ARG("yolo_detect_forward: rows [{}, {}) do not lie in an output of shape {}", row0,
                              row0 + num_anchors * H[s] * W[s], os.to_string());
        const Shape as = ag.shape();
        aH[s] = as.size() >= 3 ? (int64_t)as[2] : H[s], aW[s] = as.size() >= 4 ? (int64_t)as[3] : W[s];
        cp[s] = fp(conv), gp[s] = fp(g), ap[s] = fp(ag), ge[s] = (int64_t)g.elements(), ae[s] = (int64_t)ag.elements();
        op[s] = const_cast<float *>(fp(out)) + (int64_t)row0 * CI;
        row0 += (size_t)(num_anchors * H[s] * W[s]);
    }
    check(odl_hip_yolo_decode_stages((int)S, cp, gp, ge, ap, ae, aH, aW, N, H, W, stride.data(), num_anchors, num_classes, op,
                                     (int64_t)(os[1] * os[2]), cur()));
}

std::unique_ptr<Mat> OriginMat::pow(const Scalar &exponent) const
{
    const OriginMat &x = dev_any(*this, "pow");
    if (x.dtype() != DataType::kFloat32 && x.dtype() != DataType::kFloat64)
        THROW_INVALID_ARG("pow: only floating-point tensors are supported on the device, got {}", dtype_to_string(x.dtype()));
    auto out = new_like(x, shape_, x.dtype());
    // float32: powf with the exponent rounded to float, as the reference's float kernel sees it
    const double e = x.dtype() == DataType::kFloat32 ? (double)exponent.to_float32() : exponent.to_float64();
    check(odl_hip_pow_scalar_dtype(code(x.dtype()), x.storage()->data(), (int64_t)elements(), e, out->storage()->data(),
                                   cur()));
    return out;
}

std::unique_ptr<Mat> OriginMat::matmul(const Mat &other) const
{
    // float64 x float64 goes to the FP64 matrix cores; everything else is the float32 product
    const bool f64 = dtype_ == DataType::kFloat64 && other.dtype() == DataType::kFloat64;
    const OriginMat &a = f64 ? dev_any(*this, "matmul") : dev_f32(*this, "matmul");
    const OriginMat &b = f64 ? dev_any(other, "matmul") : dev_f32(other, "matmul");
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
    if (f64)
    {
        auto c = new_like(a, rs, DataType::kFloat64);
        check(odl_hip_dgemm(0, 0, M, N, K, static_cast<const double *>(a.storage()->data()), K,
                            static_cast<const double *>(b.storage()->data()), N, static_cast<double *>(c->storage()->data()), N,
                            batch, M * K, b_batched ? K * N : 0, M * N, cur()));
        return c;
    }
    auto c = new_like(a, rs);
    Workspace ws(odl_hip_matmul_workspace_bytes(batch, M, N, K, b_batched), device().index());
    check(odl_hip_matmul(fp(a), fp(b), c->data_ptr<float>(), batch, M, N, K, b_batched, ws.ptr(), ws.bytes, cur()));
    return c;
}

// -------------------------------------------------------------------------------- reductions / broadcast
std::unique_ptr<Mat> OriginMat::broadcast_to(const Shape &shape) const
{
    const OriginMat &x = dev_any(*this, "broadcast_to");
    auto out = new_like(x, shape, x.dtype());
    const auto sd = dims64(shape_), dd = dims64(shape);
    check(odl_hip_broadcast_to_dtype(code(x.dtype()), x.storage()->data(), sd.data(), (int)shape_.size(), dd.data(),
                                     (int)shape.size(), out->storage()->data(), cur()));
    return out;
}

std::unique_ptr<Mat> OriginMat::sum_to(const Shape &shape) const
{
    if (shape_ == shape)
        return std::make_unique<OriginMat>(*this);  // storage-sharing copy, src/mat/origin/cpu/math/sum_to.cpp:14-18
    const OriginMat &x = dev_any(*this, "sum_to");
    const int dt = code(x.dtype());
    const auto sd = dims64(shape_), td = dims64(shape);
    Workspace ws(odl_hip_sum_to_dtype_workspace_bytes(dt, sd.data(), (int)shape_.size(), td.data(), (int)shape.size()),
                 device().index());
    auto out = new_like(x, shape, x.dtype());
    check(odl_hip_sum_to_dtype(dt, x.storage()->data(), sd.data(), (int)shape_.size(), td.data(), (int)shape.size(),
                               out->storage()->data(), ws.ptr(), ws.bytes, cur()));
    return out;
}

std::unique_ptr<Mat> OriginMat::sum(int axis, bool keepdim) const
{
    const OriginMat &x = dev_any(*this, "sum");
    const int dt = code(x.dtype());
    if (axis == -1)
    {
        const Shape rs = keepdim ? Shape(std::vector<size_t>(shape_.size(), 1)) : Shape{1};
        auto out = new_like(x, rs, x.dtype());
        // the reference's whole-tensor sum goes back into the element type through a float (sum.cpp:18-35)
        Workspace ws(odl_hip_sum_axis_dtype_workspace_bytes(dt, 1, (int64_t)elements(), 1), device().index());
        check(odl_hip_sum_axis_dtype(dt, x.storage()->data(), 1, (int64_t)elements(), 1, 1, out->storage()->data(), ws.ptr(),
                                     ws.bytes, cur()));
        return out;
    }
    if (axis < 0 || axis >= (int)shape_.size())
        THROW_INVALID_ARG("Invalid axis {} for sum operation. Tensor has {} dimensions", axis, shape_.size());
    std::vector<size_t> rd;
    for (size_t i = 0; i < shape_.size(); ++i)
    {
        if ((int)i != axis)
            rd.push_back(shape_[i]);
        else if (keepdim)
            rd.push_back(1);
    }
    int64_t outer, ax, inner;
    split_axis(shape_, axis, outer, ax, inner);
    auto out = new_like(x, Shape(rd), x.dtype());
    Workspace ws(odl_hip_sum_axis_dtype_workspace_bytes(dt, outer, ax, inner), device().index());
    check(odl_hip_sum_axis_dtype(dt, x.storage()->data(), outer, ax, inner, 0, out->storage()->data(), ws.ptr(), ws.bytes,
                                 cur()));
    return out;
}

std::unique_ptr<Mat> OriginMat::max(int axis) const
{
    const OriginMat &x = dev_any(*this, "max");
    const int dt = code(x.dtype());
    if (axis == -1)
    {
        auto out = new_like(x, Shape{1}, x.dtype());
        check(odl_hip_max_all_dtype(dt, x.storage()->data(), (int64_t)elements(), out->storage()->data(), cur()));
        return out;
    }
    if (axis < 0 || axis >= (int)shape_.size())
        THROW_INVALID_ARG("Invalid axis {} for max operation. Tensor has {} dimensions", axis, shape_.size());
    std::vector<size_t> rd;
    for (size_t i = 0; i < shape_.size(); ++i)
        if ((int)i != axis)
            rd.push_back(shape_[i]);
    int64_t outer, ax, inner;
    split_axis(shape_, axis, outer, ax, inner);
    auto out = new_like(x, Shape(rd), x.dtype());
    check(odl_hip_max_axis_dtype(dt, x.storage()->data(), outer, ax, inner, out->storage()->data(), cur()));
    return out;
}

// ----------------------------------------------------------------------------------- convolution / pooling
std::unique_ptr<Mat> OriginMat::im2col(std::pair<int, int> k, std::pair<int, int> s, std::pair<int, int> p,
                                       bool to_matrix) const
{
    const OriginMat &x = dev_real(*this, "im2col");
    if (shape_.size() != 4)
        THROW_INVALID_ARG("im2col: input must be 4D (N, C, H, W), but got shape {}", shape_.to_string());
    const int64_t N = shape_[0], C = shape_[1], H = shape_[2], W = shape_[3];
    const int OH = get_conv_outsize((int)H, k.first, s.first, p.first);
    const int OW = get_conv_outsize((int)W, k.second, s.second, p.second);
    if (OH <= 0 || OW <= 0)
        THROW_INVALID_ARG("im2col: invalid output size OH={}, OW={} for input H={}, W={}", OH, OW, H, W);
    const Shape cs = to_matrix ? Shape{(size_t)(N * OH * OW), (size_t)(C * k.first * k.second)}
                               : Shape{(size_t)N, (size_t)C, (size_t)k.first, (size_t)k.second, (size_t)OH, (size_t)OW};
    auto col = new_like(x, cs, x.dtype());
    if (x.dtype() == DataType::kFloat64)
        check(odl_hip_im2col_f64(x.data_ptr<double>(), N, C, H, W, k.first, k.second, s.first, s.second, p.first, p.second,
                                 to_matrix ? 1 : 0, col->data_ptr<double>(), cur()));
    else
        check(odl_hip_im2col(fp(x), N, C, H, W, k.first, k.second, s.first, s.second, p.first, p.second, to_matrix ? 1 : 0,
                             col->data_ptr<float>(), cur()));
    return col;
}

std::unique_ptr<Mat> OriginMat::col2im(const Shape &is, std::pair<int, int> k, std::pair<int, int> s,
                                       std::pair<int, int> p, bool to_matrix) const
{
    const OriginMat &col = dev_real(*this, "col2im");
    if (is.size() != 4)
        THROW_INVALID_ARG("col2im: input_shape must be 4D (N, C, H, W), but got shape {}", is.to_string());
    const int64_t N = is[0], C = is[1], H = is[2], W = is[3];
    const int OH = get_conv_outsize((int)H, k.first, s.first, p.first);
    const int OW = get_conv_outsize((int)W, k.second, s.second, p.second);
    const Shape want = to_matrix ? Shape{(size_t)(N * OH * OW), (size_t)(C * k.first * k.second)}
                                 : Shape{(size_t)N, (size_t)C, (size_t)k.first, (size_t)k.second, (size_t)OH, (size_t)OW};
    if (OH <= 0 || OW <= 0 || shape_ != want)
        THROW_INVALID_ARG("col2im: invalid col shape {} for input_shape {}", shape_.to_string(), is.to_string());
    auto img = new_like(col, is, col.dtype());
    if (col.dtype() == DataType::kFloat64)
        check(odl_hip_col2im_f64(col.data_ptr<double>(), N, C, H, W, k.first, k.second, s.first, s.second, p.first, p.second,
                                 to_matrix ? 1 : 0, img->data_ptr<double>(), cur()));
    else
        check(odl_hip_col2im(fp(col), N, C, H, W, k.first, k.second, s.first, s.second, p.first, p.second, to_matrix ? 1 : 0,
                             img->data_ptr<float>(), cur()));
    return img;
}

std::unique_ptr<Mat> OriginMat::conv2d(const Mat &Wm, const Mat *bm, std::pair<int, int> s, std::pair<int, int> p) const
{
    return conv2d_act(Wm, bm, s, p, -1);
}

std::unique_ptr<Mat> OriginMat::conv2d_act(const Mat &Wm, const Mat *bm, std::pair<int, int> s, std::pair<int, int> p,
                                           int activation) const
{
    return conv2d_act(Wm, bm, s, p, activation, nullptr);
}

// null when a forward over an input of this shape reads the filter as it lies
std::unique_ptr<Mat> OriginMat::conv2d_packed_weights(const Mat &Wm, std::pair<int, int> s, std::pair<int, int> p) const
{
    dev_f32(*this, "conv2d");
    return conv2d_packed_weights_for(shape_, Wm, s, p);
}

std::unique_ptr<Mat> OriginMat::conv2d_packed_weights_for(const Shape &shape_, const Mat &Wm, std::pair<int, int> s,
                                                          std::pair<int, int> p)
{
    const OriginMat &w = dev_f32(Wm, "conv2d");
    const OriginMat &x = w;  // the copy lives where the filter does
    if (shape_.size() != 4 || w.shape().size() != 4)
        return nullptr;
    const int64_t OC = w.shape()[0], C = w.shape()[1];
    const int KH = (int)w.shape()[2], KW = (int)w.shape()[3];
    const size_t bytes = odl_hip_conv2d_packed_weights_bytes((int64_t)shape_[0], (int64_t)shape_[1], (int64_t)shape_[2],
                                                             (int64_t)shape_[3], OC, KH, KW, s.first, s.second, p.first,
                                                             p.second);
    if (bytes == 0 || (int64_t)shape_[1] != C)
        return nullptr;
    auto packed = new_like(x, Shape{bytes / sizeof(float)});  // whole tiles of output channels for some kernels
    check(odl_hip_conv2d_pack_weights(fp(w), (int64_t)shape_[0], C, (int64_t)shape_[2], (int64_t)shape_[3], OC, KH, KW, s.first,
                                      s.second, p.first, p.second, packed->data_ptr<float>(), cur()));
    return packed;
}

std::unique_ptr<Mat> OriginMat::conv2d_act(const Mat &Wm, const Mat *bm, std::pair<int, int> s, std::pair<int, int> p,
                                           int activation, const Mat *packed_m) const
{
    const OriginMat &x = dev_real(*this, "conv2d");
    const OriginMat &w = dev_real(Wm, "conv2d");
    same_dtype(x, w, "conv2d");
    const bool f64 = x.dtype() == DataType::kFloat64;
    if (shape_.size() != 4)
        THROW_INVALID_ARG("conv2d: x must be 4D (N, C, H, W), but got shape {}", shape_.to_string());
    if (w.shape().size() != 4)
        THROW_INVALID_ARG("conv2d: W must be 4D (OC, C, KH, KW), but got shape {}", w.shape().to_string());
    const int64_t N = shape_[0], C = shape_[1], H = shape_[2], W = shape_[3];
    const int64_t OC = w.shape()[0];
    const int KH = (int)w.shape()[2], KW = (int)w.shape()[3];
    if ((int64_t)w.shape()[1] != C)
        THROW_INVALID_ARG("conv2d: channel mismatch - x has {} channels, but W expects {} channels", C, w.shape()[1]);
    const int OH = get_conv_outsize((int)H, KH, s.first, p.first), OW = get_conv_outsize((int)W, KW, s.second, p.second);
    if (OH <= 0 || OW <= 0)
        THROW_INVALID_ARG("conv2d: invalid output size OH={}, OW={} for input H={}, W={}, kernel=({},{})", OH, OW, H, W,
                          KH, KW);
    const float *bias = nullptr;
    const double *bias64 = nullptr;
    if (bm)
    {
        const OriginMat &b = dev_real(*bm, "conv2d");
        same_dtype(x, b, "conv2d");
        if (b.shape().size() != 1 || (int64_t)b.shape()[0] != OC)
            THROW_INVALID_ARG("conv2d: b must be 1D with size {}, but got shape {}", OC, b.shape().to_string());
        if (f64)
            bias64 = b.data_ptr<double>();
        else
            bias = fp(b);
    }
    auto y = new_like(x, Shape{(size_t)N, (size_t)OC, (size_t)OH, (size_t)OW}, x.dtype());
    if (f64)
    {
        // float64: the products on the FP64 matrix cores, an activation that follows as a pass of its own
        Workspace ws64(odl_hip_conv2d_f64_workspace_bytes(N, C, H, W, OC, KH, KW, s.first, s.second, p.first, p.second),
                       device().index());
        check(odl_hip_conv2d_f64(x.data_ptr<double>(), w.data_ptr<double>(), bias64, N, C, H, W, OC, KH, KW, s.first, s.second,
                                 p.first, p.second, y->data_ptr<double>(), ws64.ptr(), ws64.bytes, cur()));
        if (activation >= 0)
            check(odl_hip_unary_dtype(activation, code(DataType::kFloat64), y->storage()->data(), (int64_t)y->elements(),
                                      y->storage()->data(), cur()));
        return y;
    }
    Workspace ws(odl_hip_conv2d_workspace_bytes(N, C, H, W, OC, KH, KW, s.first, s.second, p.first, p.second),
                 device().index());
    const float *packed = nullptr;
    if (packed_m)
    {
        const OriginMat &pk = dev_f32(*packed_m, "conv2d");
        const size_t want = odl_hip_conv2d_packed_weights_bytes(N, C, H, W, OC, KH, KW, s.first, s.second, p.first, p.second);
        if (pk.elements() * sizeof(float) != want)
            THROW_INVALID_ARG("conv2d: the packed filter has {} bytes, this shape's kernel reads {}", pk.elements() * sizeof(float),
                              want);
        packed = fp(pk);
    }
    check(odl_hip_conv2d_act_packed(fp(x), fp(w), packed, bias, N, C, H, W, OC, KH, KW, s.first, s.second, p.first,
                                    p.second, activation, y->data_ptr<float>(), ws.ptr(), ws.bytes, cur()));
    return y;
}

std::vector<std::unique_ptr<Mat>> OriginMat::conv2d_backward(const Mat &gym, const Mat &xm, const Mat &Wm, const Mat *bm,
                                                             std::pair<int, int> s, std::pair<int, int> p) const
{
    const OriginMat &gy = dev_real(gym, "conv2d_backward");
    const OriginMat &x  = dev_real(xm, "conv2d_backward");
    const OriginMat &w  = dev_real(Wm, "conv2d_backward");
    same_dtype(x, gy, "conv2d_backward");
    same_dtype(x, w, "conv2d_backward");
    if (gy.shape().size() != 4)
        THROW_INVALID_ARG("conv2d_backward: gy must be 4D (N, OC, OH, OW), but got shape {}", gy.shape().to_string());
    if (x.shape().size() != 4)
        THROW_INVALID_ARG("conv2d_backward: x must be 4D (N, C, H, W), but got shape {}", x.shape().to_string());
    if (w.shape().size() != 4)
        THROW_INVALID_ARG("conv2d_backward: W must be 4D (OC, C, KH, KW), but got shape {}", w.shape().to_string());
    const int64_t N = x.shape()[0], C = x.shape()[1], H = x.shape()[2], W = x.shape()[3];
    const int64_t OC = w.shape()[0];
    const int KH = (int)w.shape()[2], KW = (int)w.shape()[3];
    auto gx = new_like(x, x.shape(), x.dtype());
    auto gw = new_like(x, w.shape(), x.dtype());
    std::unique_ptr<OriginMat> gb;
    if (bm)
        gb = new_like(x, Shape{(size_t)OC}, x.dtype());
    if (x.dtype() == DataType::kFloat64)
    {
        Workspace ws64(odl_hip_conv2d_backward_f64_workspace_bytes(N, C, H, W, OC, KH, KW, s.first, s.second, p.first, p.second),
                       device().index());
        check(odl_hip_conv2d_backward_f64(gy.data_ptr<double>(), x.data_ptr<double>(), w.data_ptr<double>(), N, C, H, W, OC, KH,
                                          KW, s.first, s.second, p.first, p.second, gx->data_ptr<double>(),
                                          gw->data_ptr<double>(), gb ? gb->data_ptr<double>() : nullptr, ws64.ptr(), ws64.bytes,
                                          cur()));
    }
    else
    {
        Workspace ws(odl_hip_conv2d_backward_workspace_bytes(N, C, H, W, OC, KH, KW, s.first, s.second, p.first, p.second),
                     device().index());
        check(odl_hip_conv2d_backward(fp(gy), fp(x), fp(w), N, C, H, W, OC, KH, KW, s.first, s.second, p.first, p.second,
                                      gx->data_ptr<float>(), gw->data_ptr<float>(), gb ? gb->data_ptr<float>() : nullptr,
                                      ws.ptr(), ws.bytes, cur()));
    }
    std::vector<std::unique_ptr<Mat>> grads;  // {gx, gW, [gb]}
    grads.push_back(std::move(gx));
    grads.push_back(std::move(gw));
    if (gb)
        grads.push_back(std::move(gb));
    return grads;
}

std::unique_ptr<Mat> OriginMat::max_pool2d_device(std::pair<int, int> k, std::pair<int, int> s, std::pair<int, int> p,
                                                  std::shared_ptr<Storage> *indices) const
{
    const OriginMat &x = dev_f32(*this, "max_pool2d");
    if (shape_.size() != 4)
        THROW_INVALID_ARG("max_pool2d: x must be 4D (N, C, H, W), but got shape {}", shape_.to_string());
    const int64_t N = shape_[0], C = shape_[1], H = shape_[2], W = shape_[3];
    const int OH = get_conv_outsize((int)H, k.first, s.first, p.first);
    const int OW = get_conv_outsize((int)W, k.second, s.second, p.second);
    if (OH <= 0 || OW <= 0)
        THROW_INVALID_ARG("max_pool2d: invalid output size OH={}, OW={} for input H={}, W={}", OH, OW, H, W);
    auto y = new_like(x, Shape{(size_t)N, (size_t)C, (size_t)OH, (size_t)OW});
    std::shared_ptr<Storage> idx;
    if (indices)
        idx = Storage::create(y->elements() * sizeof(uint64_t), DeviceType::kCUDA, device().index());
    check(odl_hip_max_pool2d(fp(x), N, C, H, W, k.first, k.second, s.first, s.second, p.first, p.second,
                             y->data_ptr<float>(), idx ? static_cast<uint64_t *>(idx->data()) : nullptr, cur()));
    if (indices)
        *indices = idx;
    return y;
}

std::unique_ptr<Mat> OriginMat::max_pool2d(std::pair<int, int> k, std::pair<int, int> s, std::pair<int, int> p,
                                           std::vector<size_t> *indices) const
{
    std::shared_ptr<Storage> idx;
    auto y = max_pool2d_device(k, s, p, indices ? &idx : nullptr);
    if (indices)
    {
        // the interface hands the window-local indices to the caller as a host vector (mat.h:560-566)
        static_assert(sizeof(size_t) == sizeof(uint64_t), "size_t must be 64-bit");
        indices->resize(y->elements());
        no_capture("device-to-host copy");
        check(odl_hip_memcpy_d2h(indices->data(), idx->data(), y->elements() * sizeof(uint64_t)));
    }
    return y;
}

std::unique_ptr<Mat> OriginMat::max_pool2d_backward_device(const Mat &gym, std::pair<int, int> k, std::pair<int, int> s,
                                                           std::pair<int, int> p, const Storage &indices) const
{
    const OriginMat &gy = dev_f32(gym, "max_pool2d_backward");
    if (gy.shape().size() != 4)
        THROW_INVALID_ARG("max_pool2d_backward: gy must be 4D (N, C, OH, OW), but got shape {}", gy.shape().to_string());
    if (indices.size() < gy.elements() * sizeof(uint64_t) || indices.device_type() != DeviceType::kCUDA)
        THROW_INVALID_ARG("max_pool2d_backward: indices size mismatch. Expected {}, got {}", gy.elements(),
                          indices.size() / sizeof(uint64_t));
    const int64_t N = shape_[0], C = shape_[1], H = shape_[2], W = shape_[3];
    auto gx = new_like(gy, shape_);
    check(odl_hip_max_pool2d_backward(fp(gy), static_cast<const uint64_t *>(indices.data()), N, C, H, W, k.first, k.second,
                                      s.first, s.second, p.first, p.second, gx->data_ptr<float>(), cur()));
    return gx;
}

std::unique_ptr<Mat> OriginMat::max_pool2d_backward_relu_device(const Mat &gym, std::pair<int, int> k, std::pair<int, int> s,
                                                                std::pair<int, int> p, const Storage &indices) const
{
    const OriginMat &gy = dev_f32(gym, "max_pool2d_backward");
    const OriginMat &x  = dev_f32(*this, "max_pool2d_backward");
    if (gy.shape().size() != 4)
        THROW_INVALID_ARG("max_pool2d_backward: gy must be 4D (N, C, OH, OW), but got shape {}", gy.shape().to_string());
    if (indices.size() < gy.elements() * sizeof(uint64_t) || indices.device_type() != DeviceType::kCUDA)
        THROW_INVALID_ARG("max_pool2d_backward: indices size mismatch. Expected {}, got {}", gy.elements(),
                          indices.size() / sizeof(uint64_t));
    const int64_t N = shape_[0], C = shape_[1], H = shape_[2], W = shape_[3];
    auto gx = new_like(gy, shape_);
    check(odl_hip_max_pool2d_backward_relu(fp(gy), static_cast<const uint64_t *>(indices.data()), fp(x), N, C, H, W, k.first,
                                           k.second, s.first, s.second, p.first, p.second, gx->data_ptr<float>(), cur()));
    return gx;
}

bool OriginMat::conv_relu_pool_fused(const Mat &xm, const Mat &Wm, std::pair<int, int> s, std::pair<int, int> p,
                                     std::pair<int, int> pk, std::pair<int, int> ps, std::pair<int, int> pp)
{
    if (!device_f32(xm) || !device_f32(Wm) || xm.shape().size() != 4 || Wm.shape().size() != 4 || xm.shape()[1] != Wm.shape()[1])
        return false;
    const Shape xs = xm.shape(), ws = Wm.shape();
    return odl_hip_conv2d_relu_max_pool2d_ok((int64_t)xs[0], (int64_t)xs[1], (int64_t)xs[2], (int64_t)xs[3], (int64_t)ws[0],
                                             (int)ws[2], (int)ws[3], s.first, s.second, p.first, p.second, pk.first, pk.second,
                                             ps.first, ps.second, pp.first, pp.second) == 1;
}

std::unique_ptr<Mat> OriginMat::conv2d_relu_max_pool2d_device(const Mat &Wm, const Mat *bm, std::pair<int, int> s,
                                                              std::pair<int, int> p, std::pair<int, int> pk,
                                                              std::pair<int, int> ps, std::pair<int, int> pp,
                                                              std::shared_ptr<Storage> *indices) const
{
    const OriginMat &x = dev_f32(*this, "conv2d"), &w = dev_f32(Wm, "conv2d");
    const int64_t N = shape_[0], C = shape_[1], H = shape_[2], W = shape_[3], OC = w.shape()[0];
    const float *bias = nullptr;
    if (bm)
    {
        const OriginMat &b = dev_f32(*bm, "conv2d");
        if (b.shape().size() != 1 || (int64_t)b.shape()[0] != OC)
            THROW_INVALID_ARG("conv2d: b must be 1D with size {}, but got shape {}", OC, b.shape().to_string());
        bias = fp(b);
    }
    auto y = new_like(x, Shape{(size_t)N, (size_t)OC, (size_t)(H / 2), (size_t)(W / 2)});
    std::shared_ptr<Storage> idx;
    if (indices)
    {
        idx = Storage::create(y->elements() * sizeof(uint8_t), DeviceType::kCUDA, device().index());
        check(odl_hip_conv2d_relu_max_pool2d_compact(fp(x), fp(w), bias, N, C, H, W, OC, (int)w.shape()[2], (int)w.shape()[3],
                                                     s.first, s.second, p.first, p.second, pk.first, pk.second, ps.first,
                                                     ps.second, pp.first, pp.second, y->data_ptr<float>(),
                                                     static_cast<uint8_t *>(idx->data()), cur()));
        *indices = idx;
    }
    else
        check(odl_hip_conv2d_relu_max_pool2d(fp(x), fp(w), bias, N, C, H, W, OC, (int)w.shape()[2], (int)w.shape()[3], s.first,
                                             s.second, p.first, p.second, pk.first, pk.second, ps.first, ps.second, pp.first,
                                             pp.second, y->data_ptr<float>(), nullptr, cur()));
    return y;
}

std::unique_ptr<Mat> OriginMat::max_pool2d_backward_relu_pooled_device(const Mat &gym, const Shape &input_shape,
                                                                       std::pair<int, int> k, std::pair<int, int> s,
                                                                       std::pair<int, int> p, const Storage &indices) const
{
    const OriginMat &gy = dev_f32(gym, "max_pool2d_backward");
    const OriginMat &y  = dev_f32(*this, "max_pool2d_backward");
    if (gy.shape().size() != 4 || input_shape.size() != 4 || !(gy.shape() == y.shape()))
        THROW_INVALID_ARG("max_pool2d_backward: gy {} and the pooled tensor {} must be 4D of one shape", gy.shape().to_string(),
                          y.shape().to_string());
    if (indices.size() < gy.elements() * sizeof(uint8_t) || indices.device_type() != DeviceType::kCUDA)
        THROW_INVALID_ARG("max_pool2d_backward: indices size mismatch. Expected {}, got {}", gy.elements(), indices.size());
    auto gx = new_like(gy, input_shape);
    check(odl_hip_max_pool2d_backward_relu_pooled_compact(fp(gy), static_cast<const uint8_t *>(indices.data()), fp(y),
                                                          (int64_t)input_shape[0], (int64_t)input_shape[1],
                                                          (int64_t)input_shape[2], (int64_t)input_shape[3], k.first, k.second,
                                                          s.first, s.second, p.first, p.second, gx->data_ptr<float>(), cur()));
    return gx;
}

std::unique_ptr<Mat> OriginMat::max_pool2d_device_compact(std::pair<int, int> k, std::pair<int, int> s, std::pair<int, int> p,
                                                          std::shared_ptr<Storage> *indices) const
{
    const OriginMat &x = dev_f32(*this, "max_pool2d");
    if (shape_.size() != 4)
        THROW_INVALID_ARG("max_pool2d: x must be 4D (N, C, H, W), but got shape {}", shape_.to_string());
    const int64_t N = shape_[0], C = shape_[1], H = shape_[2], W = shape_[3];
    const int OH = get_conv_outsize((int)H, k.first, s.first, p.first);
    const int OW = get_conv_outsize((int)W, k.second, s.second, p.second);
    if (OH <= 0 || OW <= 0)
        THROW_INVALID_ARG("max_pool2d: invalid output size OH={}, OW={} for input H={}, W={}", OH, OW, H, W);
    auto y   = new_like(x, Shape{(size_t)N, (size_t)C, (size_t)OH, (size_t)OW});
    auto idx = Storage::create(y->elements() * sizeof(uint8_t), DeviceType::kCUDA, device().index());
    check(odl_hip_max_pool2d_compact(fp(x), N, C, H, W, k.first, k.second, s.first, s.second, p.first, p.second,
                                     y->data_ptr<float>(), static_cast<uint8_t *>(idx->data()), cur()));
    *indices = idx;
    return y;
}

std::unique_ptr<Mat> OriginMat::max_pool2d_backward(const Mat &gym, std::pair<int, int> k, std::pair<int, int> s,
                                                    std::pair<int, int> p, const std::vector<size_t> &indices) const
{
    const OriginMat &gy = dev_f32(gym, "max_pool2d_backward");
    if (indices.size() != gy.elements())
        THROW_INVALID_ARG("max_pool2d_backward: indices size mismatch. Expected {}, got {}", gy.elements(),
                          indices.size());
    auto idx = Storage::create(indices.size() * sizeof(uint64_t), DeviceType::kCUDA, gy.device().index());
    no_capture("host-to-device copy");
    check(odl_hip_memcpy_h2d(idx->data(), indices.data(), indices.size() * sizeof(uint64_t), cur()));
    return max_pool2d_backward_device(gym, k, s, p, *idx);
}

// -------------------------------------------------------------------------------------------- indexing
std::unique_ptr<Mat> OriginMat::gather(const Mat &indices) const
{
    const OriginMat &x   = dev_any(*this, "gather");
    const OriginMat &idx = as_origin(indices);
    if (shape_.size() != 2)
        THROW_INVALID_ARG("gather: input must be 2D (N, C), but got shape {}", shape_.to_string());
    if (idx.shape().size() != 1)
        THROW_INVALID_ARG("gather: indices must be 1D (N,), but got shape {}", idx.shape().to_string());
    if (shape_[0] != idx.shape()[0])
        THROW_INVALID_ARG("gather: batch size mismatch. input has {} samples, indices has {} samples", shape_[0],
                          idx.shape()[0]);
    if (idx.device() != device())
        THROW_INVALID_ARG("gather: input and indices must be on the same device");
    const int is64 = label_kind(idx, "gather");
    auto out = new_like(x, Shape{shape_[0]}, x.dtype());
    check(odl_hip_gather_dtype(code(x.dtype()), x.storage()->data(), idx.storage()->data(), is64, (int64_t)shape_[0],
                               (int64_t)shape_[1], out->storage()->data(), cur()));
    return out;
}

std::unique_ptr<Mat> OriginMat::one_hot(const Mat &indices, int num_classes) const
{
    const OriginMat &idx = as_origin(indices);
    if (idx.shape().size() != 1)
        THROW_INVALID_ARG("one_hot: indices must be 1D (N,), but got shape {}", idx.shape().to_string());
    if (num_classes <= 0)
        THROW_INVALID_ARG("one_hot: num_classes must be positive, but got {}", num_classes);
    if (idx.device().type() != DeviceType::kCUDA)
        THROW_RUNTIME_ERROR("one_hot: indices are on {}; this backend computes on the GPU only", idx.device().to_string());
    const int is64 = label_kind(idx, "one_hot");
    auto out = std::make_unique<OriginMat>(Shape{idx.shape()[0], (size_t)num_classes}, DataType::kFloat32, idx.device());
    check(odl_hip_one_hot(idx.storage()->data(), is64, (int64_t)idx.shape()[0], num_classes, out->data_ptr<float>(),
                          cur()));
    return out;
}

// ------------------------------------------------------------------------ fused paths above the Mat set
std::unique_ptr<Mat> OriginMat::softmax(int axis) const
{
    if (dtype() == DataType::kFloat64)
    {
        // float64: the reference's own composition (src/operators/activation/softmax.cpp:34-76) out of operators that
        // take every element type — max along the axis, subtract, exp, sum along the axis, divide
        dev_any(*this, "softmax");
        std::vector<size_t> kd = shape_.dims();
        kd[axis] = 1;
        const Shape keep(kd);
        auto shifted = *this - *max(axis)->reshape(keep)->broadcast_to(shape_);
        auto e = shifted->exp();
        return *e / *e->sum(axis, false)->reshape(keep)->broadcast_to(shape_);
    }
    const OriginMat &x = dev_f32(*this, "softmax");
    int64_t outer, ax, inner;
    split_axis(shape_, axis, outer, ax, inner);
    auto y = new_like(x, shape_);
    check(odl_hip_softmax(fp(x), outer, ax, inner, y->data_ptr<float>(), cur()));
    return y;
}

float OriginMat::softmax_cross_entropy(const Mat &target) const
{
    const OriginMat &x = dev_f32(*this, "softmax_cross_entropy");
    const OriginMat &t = as_origin(target);
    const int is64     = label_kind(t, "gather");
    const int64_t N = shape_[0], C = shape_[1];
    Workspace ws(odl_hip_softmax_ce_loss_workspace_bytes(N), device().index());
    float loss = 0.f;
    check(odl_hip_softmax_ce_loss(fp(x), t.storage()->data(), is64, N, C, &loss, ws.ptr(), ws.bytes, cur()));
    return loss;
}

std::unique_ptr<Mat> OriginMat::softmax_cross_entropy_backward(const Mat &target, float gy) const
{
    const OriginMat &x = dev_f32(*this, "softmax_cross_entropy");
    const OriginMat &t = as_origin(target);
    const int is64     = label_kind(t, "one_hot");
    auto gx = new_like(x, shape_);
    check(odl_hip_softmax_ce_grad(fp(x), t.storage()->data(), is64, (int64_t)shape_[0], (int64_t)shape_[1], gy,
                                  gx->data_ptr<float>(), cur()));
    return gx;
}

std::unique_ptr<Mat> OriginMat::softmax_cross_entropy_device(const Mat &target, std::unique_ptr<Mat> *unit_grad) const
{
    const OriginMat &x = dev_f32(*this, "softmax_cross_entropy");
    const OriginMat &t = as_origin(target);
    const int is64     = label_kind(t, "gather");
    const int64_t N = shape_[0], C = shape_[1];
    Workspace ws(odl_hip_softmax_ce_loss_workspace_bytes(N), device().index());
    // two words: the loss, and the bad-label flag behind it; the Mat is the scalar in front
    auto storage = Storage::create(2 * sizeof(float), DeviceType::kCUDA, device().index());
    void *mirror = MirrorPool::get().take(cur());
    if (unit_grad && odl_hip_softmax_ce_loss_grad_ok(N, C) == 1)
    {
        auto gx = new_like(x, shape_);
        check(odl_hip_softmax_ce_loss_grad_device(fp(x), t.storage()->data(), is64, N, C, static_cast<float *>(storage->data()),
                                                  mirror, gx->data_ptr<float>(), ws.ptr(), ws.bytes, cur()));
        *unit_grad = std::move(gx);
    }
    else
        check(odl_hip_softmax_ce_loss_device(fp(x), t.storage()->data(), is64, N, C, static_cast<float *>(storage->data()),
                                             mirror, ws.ptr(), ws.bytes, cur()));
    // outside a capture an event behind the kernel lets the host read the loss without waiting for the backward pass
    void *event = nullptr;
    if (!t_capturing)
    {
        event = MirrorPool::get().event_of(mirror);
        check(odl_hip_event_record(event, cur()));
    }
    storage->set_mirror(mirror, t_capturing, cur(), event);
    return std::make_unique<OriginMat>(std::move(storage), Shape{}, DataType::kFloat32);
}

std::unique_ptr<Mat> OriginMat::softmax_cross_entropy_checked(const Mat &target, std::unique_ptr<Mat> *unit_grad) const
{
    // labels that came up from the host carry their range: an out-of-range label is reported without asking the device,
    // and a batch in range needs no check at all (the step then has no stop in its middle)
    int64_t lo = 0, hi = 0;
    if (as_origin(target).storage()->int_range(&lo, &hi))
    {
        if (lo < 0 || hi >= (int64_t)shape_[1])
            THROW_INVALID_ARG("gather: index out of range [0, {})", shape_[1]);
        return softmax_cross_entropy_device(target, unit_grad);
    }
    auto loss = softmax_cross_entropy_device(target, unit_grad);
    // the loss word and the bad-label flag behind it come back together (this synchronises, as the reference's host-side
    // divide does); the loss itself stays on the device for the operators that follow
    unsigned words[2] = {0, 0};
    no_capture("device-to-host copy");
    const auto &st = as_origin(*loss).storage();
    if (!st->read_mirror(words, sizeof(words)))
        check(odl_hip_memcpy_d2h(words, st->data(), sizeof(words)));
    if (words[1] != 0)
        THROW_INVALID_ARG("gather: index out of range [0, {})", shape_[1]);
    st->set_host_copy(words, sizeof(words));  // item() on the loss needs no second trip
    return loss;
}

std::unique_ptr<Mat> OriginMat::permute(const std::vector<int> &dims) const
{
    if (dims.size() != shape_.size())
        THROW_INVALID_ARG("permute: dims size {} does not match input dimension {}", dims.size(), shape_.size());
    std::vector<size_t> od;
    for (int d : dims)
    {
        if (d < 0 || d >= (int)shape_.size())
            THROW_INVALID_ARG("permute: invalid dimension {} (must be in [0, {}))", d, shape_.size());
        od.push_back(shape_[d]);
    }
    const OriginMat &x = dev_any(*this, "permute");
    auto out = new_like(x, Shape(od), dtype_);
    const std::vector<int64_t> in = dims64(shape_);
    check(odl_hip_permute(x.storage()->data(), code(dtype_), in.data(), (int)shape_.size(), dims.data(),
                          out->storage()->data(), cur()));
    return out;
}

bool OriginMat::loss_bad_label_flag() const
{
    if (device().type() != DeviceType::kCUDA || dtype_ != DataType::kFloat32 || elements() != 1 || !storage_ ||
        storage_->size() != 2 * sizeof(float))
        return false;
    unsigned words[2] = {0, 0};
    no_capture("device-to-host copy");
    if (!storage_->read_mirror(words, sizeof(words)))
        check(odl_hip_memcpy_d2h(words, storage_->data(), sizeof(words)));
    return words[1] != 0;
}

std::unique_ptr<Mat> OriginMat::softmax_cross_entropy_backward_device(const Mat &target, const Mat &gy) const
{
    const OriginMat &x = dev_f32(*this, "softmax_cross_entropy");
    const OriginMat &t = as_origin(target);
    const OriginMat &g = dev_f32(gy, "softmax_cross_entropy");
    const int is64     = label_kind(t, "one_hot");
    auto gx = new_like(x, shape_);
    check(odl_hip_softmax_ce_grad_device(fp(x), t.storage()->data(), is64, (int64_t)shape_[0], (int64_t)shape_[1], fp(g),
                                         gx->data_ptr<float>(), cur()));
    return gx;
}

void OriginMat::upload(const void *host, size_t bytes)
{
    if (bytes != elements() * dtype_size(dtype_))
        THROW_INVALID_ARG("upload: {} bytes given for a tensor of {} bytes", bytes, elements() * dtype_size(dtype_));
    if (bytes == 0)
        return;
    if (device().type() == DeviceType::kCPU)
    {
        std::memcpy(storage_->data(), host, bytes);
        return;
    }
    no_capture("host-to-device copy");
    // queued behind everything on the current stream that still reads the old contents
    check(odl_hip_memcpy_h2d(storage_->data(), host, bytes, cur()));
    storage_->forget_int_range();
    note_int_range(*storage_, host, dtype_, elements());
}

void OriginMat::adam_step_inplace(const Mat &grad, Mat &m, Mat &v, float beta1, float beta2, const float *device_scales,
                                  float eps, float lr)
{
    const OriginMat &p = dev_f32(*this, "adam_step");
    const OriginMat &g = dev_f32(grad, "adam_step");
    const OriginMat &mm = dev_f32(m, "adam_step");
    const OriginMat &vv = dev_f32(v, "adam_step");
    if (g.shape() != shape_ || mm.shape() != shape_ || vv.shape() != shape_)
        THROW_INVALID_ARG("adam_step: parameter, gradient and moments must have one shape");
    float *pp = const_cast<float *>(fp(p));
    check(odl_hip_adam_step_device_scales(pp, fp(g), const_cast<float *>(fp(mm)), const_cast<float *>(fp(vv)),
                                          (int64_t)elements(), beta1, beta2, device_scales, eps, lr, pp, cur()));
}

void OriginMat::copy_from(const Mat &src)
{
    const OriginMat &o = as_origin(src);
    if (o.shape() != shape_ || o.dtype() != dtype_ || o.device() != device())
        THROW_INVALID_ARG("copy_from: shape, dtype and device must match");
    storage_->forget_int_range();
    if (device().type() == DeviceType::kCPU)
        std::memcpy(storage_->data(), o.storage()->data(), elements() * dtype_size(dtype_));
    else
        check(odl_hip_memcpy_d2d(storage_->data(), o.storage()->data(), elements() * dtype_size(dtype_), cur()));
}

void OriginMat::sgd_step_inplace(const Mat &grad, float lr)
{
    const OriginMat &p = dev_f32(*this, "sgd_step");
    const OriginMat &g = dev_f32(grad, "sgd_step");
    if (g.shape() != shape_)
        THROW_INVALID_ARG("sgd_step: parameter and gradient must have one shape");
    float *pp = const_cast<float *>(fp(p));
    check(odl_hip_sgd_step(pp, fp(g), (int64_t)elements(), lr, pp, cur()));
}

std::unique_ptr<Mat> OriginMat::adam_step(const Mat &grad, Mat &m, Mat &v, float beta1, float beta2, float m_hat_scale,
                                          float v_hat_scale, float eps, float lr) const
{
    const OriginMat &p = dev_f32(*this, "adam_step");
    const OriginMat &g = dev_f32(grad, "adam_step");
    const OriginMat &mm = dev_f32(m, "adam_step");
    const OriginMat &vv = dev_f32(v, "adam_step");
    if (g.elements() != elements() || mm.elements() != elements() || vv.elements() != elements())
        THROW_INVALID_ARG("adam_step: parameter, gradient and moment sizes differ");
    auto out = new_like(p, shape_);
    check(odl_hip_adam_step(fp(p), fp(g), const_cast<float *>(fp(mm)), const_cast<float *>(fp(vv)), (int64_t)elements(),
                            beta1, beta2, m_hat_scale, v_hat_scale, eps, lr, out->data_ptr<float>(), cur()));
    return out;
}

bool OriginMat::device_f32(const Mat &m)
{
    const auto *o = dynamic_cast<const OriginMat *>(&m);
    return o && o->device().type() == DeviceType::kCUDA && o->dtype() == DataType::kFloat32;
}

std::vector<std::unique_ptr<Mat>> OriginMat::adam_step_multi(const std::vector<AdamItem> &items, float beta1, float beta2,
                                                             float eps, float lr, bool in_place, float weight_decay)
{
    const size_t count = items.size();
    std::vector<const float *> p(count), g(count), scales(count);
    std::vector<float *> m(count), v(count), out(count);
    std::vector<float> s1(count), s2(count);
    std::vector<int64_t> n(count);
    std::vector<std::unique_ptr<Mat>> results;
    for (size_t i = 0; i < count; ++i)
    {
        const OriginMat &pm = dev_f32(*items[i].param, "adam_step"), &gm = dev_f32(*items[i].grad, "adam_step");
        const OriginMat &mm = dev_f32(*items[i].m, "adam_step"), &vm = dev_f32(*items[i].v, "adam_step");
        if (gm.elements() != pm.elements() || mm.elements() != pm.elements() || vm.elements() != pm.elements())
            THROW_INVALID_ARG("adam_step: parameter, gradient and moment sizes differ");
        p[i] = fp(pm), g[i] = fp(gm), m[i] = const_cast<float *>(fp(mm)), v[i] = const_cast<float *>(fp(vm));
        s1[i] = items[i].m_hat_scale, s2[i] = items[i].v_hat_scale, scales[i] = items[i].device_scales;
        n[i] = (int64_t)pm.elements();
        if (in_place)
            out[i] = const_cast<float *>(p[i]);
        else
        {
            auto o = new_like(pm, pm.shape());
            out[i] = o->data_ptr<float>();
            results.push_back(std::move(o));
        }
    }
    if (weight_decay != 0.0f)
        check(odl_hip_adam_step_multi_decay((int)count, p.data(), const_cast<float *const *>(g.data()), m.data(), v.data(),
                                            n.data(), weight_decay, beta1, beta2, s1.data(), s2.data(), scales.data(), eps,
                                            lr, out.data(), cur()));
    else
        check(odl_hip_adam_step_multi((int)count, p.data(), g.data(), m.data(), v.data(), n.data(), beta1, beta2, s1.data(),
                                      s2.data(), scales.data(), eps, lr, out.data(), cur()));
    return results;
}

std::vector<std::unique_ptr<Mat>> OriginMat::sgd_step_multi(const std::vector<std::pair<const Mat *, const Mat *>> &param_grad,
                                                            float lr, bool in_place, float weight_decay)
{
    const size_t count = param_grad.size();
    std::vector<const float *> p(count), g(count);
    std::vector<float *> out(count);
    std::vector<int64_t> n(count);
    std::vector<std::unique_ptr<Mat>> results;
    for (size_t i = 0; i < count; ++i)
    {
        const OriginMat &pm = dev_f32(*param_grad[i].first, "sgd_step"), &gm = dev_f32(*param_grad[i].second, "sgd_step");
        if (gm.elements() != pm.elements())
            THROW_INVALID_ARG("sgd_step: parameter and gradient sizes differ");
        p[i] = fp(pm), g[i] = fp(gm), n[i] = (int64_t)pm.elements();
        if (in_place)
            out[i] = const_cast<float *>(p[i]);
        else
        {
            auto o = new_like(pm, pm.shape());
            out[i] = o->data_ptr<float>();
            results.push_back(std::move(o));
        }
    }
    if (weight_decay != 0.0f)
        check(odl_hip_sgd_step_multi_decay((int)count, p.data(), const_cast<float *const *>(g.data()), n.data(), weight_decay,
                                           lr, out.data(), cur()));
    else
        check(odl_hip_sgd_step_multi((int)count, p.data(), g.data(), n.data(), lr, out.data(), cur()));
    return results;
}

void OriginMat::axpy_multi(float a, const std::vector<std::pair<const Mat *, Mat *>> &x_y)
{
    const size_t count = x_y.size();
    std::vector<const float *> x(count);
    std::vector<float *> y(count);
    std::vector<int64_t> n(count);
    for (size_t i = 0; i < count; ++i)
    {
        const OriginMat &xm = dev_f32(*x_y[i].first, "axpy"), &ym = dev_f32(*x_y[i].second, "axpy");
        if (xm.shape() != ym.shape())
            THROW_INVALID_ARG("axpy: shape mismatch {} vs {}", xm.shape().to_string(), ym.shape().to_string());
        x[i] = fp(xm), y[i] = const_cast<float *>(fp(ym)), n[i] = (int64_t)xm.elements();
    }
    check(odl_hip_axpy_multi((int)count, a, x.data(), y.data(), n.data(), cur()));
}

std::unique_ptr<Mat> OriginMat::sgd_step(const Mat &grad, float lr) const
{
    const OriginMat &p = dev_f32(*this, "sgd_step");
    const OriginMat &g = dev_f32(grad, "sgd_step");
    if (g.elements() != elements())
        THROW_INVALID_ARG("sgd_step: parameter and gradient sizes differ");
    auto out = new_like(p, shape_);
    check(odl_hip_sgd_step(fp(p), fp(g), (int64_t)elements(), lr, out->data_ptr<float>(), cur()));
    return out;
}

std::pair<std::unique_ptr<Mat>, std::unique_ptr<Mat>> OriginMat::matmul_backward_2d(const Mat &x_, const Mat &w_,
                                                                                    const Mat &gy_)
{
    const bool f64 = x_.dtype() == DataType::kFloat64 && w_.dtype() == DataType::kFloat64 && gy_.dtype() == DataType::kFloat64;
    const OriginMat &x = f64 ? dev_any(x_, "matmul") : dev_f32(x_, "matmul");
    const OriginMat &w = f64 ? dev_any(w_, "matmul") : dev_f32(w_, "matmul");
    const OriginMat &gy = f64 ? dev_any(gy_, "matmul") : dev_f32(gy_, "matmul");
    const Shape xs = x.shape(), ws_ = w.shape(), gs = gy.shape();
    if (xs.size() != 2 || ws_.size() != 2 || gs.size() != 2 || xs[1] != ws_[0] || gs[0] != xs[0] || gs[1] != ws_[1])
        THROW_INVALID_ARG("matmul backward: shapes {} {} {} do not form x[M,K] w[K,N] gy[M,N]", xs.to_string(),
                          ws_.to_string(), gs.to_string());
    const int64_t M = xs[0], K = xs[1], N = ws_[1];
    if (f64)
    {
        // gx[M,K] = gy[M,N] . w[K,N]^T and gw[K,N] = x[M,K]^T . gy[M,N], both operands read where they lie
        auto gx = new_like(x, xs, DataType::kFloat64);
        auto gw = new_like(w, ws_, DataType::kFloat64);
        const double *xp = static_cast<const double *>(x.storage()->data()), *wp = static_cast<const double *>(w.storage()->data());
        const double *gp = static_cast<const double *>(gy.storage()->data());
        check(odl_hip_dgemm(0, 1, M, K, N, gp, N, wp, N, static_cast<double *>(gx->storage()->data()), K, 1, 0, 0, 0, cur()));
        check(odl_hip_dgemm(1, 0, K, N, M, xp, K, gp, N, static_cast<double *>(gw->storage()->data()), N, 1, 0, 0, 0, cur()));
        return {std::move(gx), std::move(gw)};
    }
    auto gx = new_like(x, xs);
    auto gw = new_like(w, ws_);
    Workspace ws(odl_hip_matmul_backward_workspace_bytes(M, K, N), x.device().index());
    check(odl_hip_matmul_backward(fp(x), fp(w), fp(gy), gx->data_ptr<float>(), gw->data_ptr<float>(), M, K, N, ws.ptr(),
                                  ws.bytes, cur()));
    return {std::move(gx), std::move(gw)};
}

std::vector<std::unique_ptr<Mat>> OriginMat::linear_backward_2d(const Mat &x_, const Mat &w_, const Mat &gy_, const Shape &bias_shape)
{
    std::vector<std::unique_ptr<Mat>> out;
    const bool f32 = x_.dtype() == DataType::kFloat32 && w_.dtype() == DataType::kFloat32 && gy_.dtype() == DataType::kFloat32;
    const Shape gs = gy_.shape();
    const bool row_bias = gs.size() == 2 && (bias_shape.size() == 1 || (bias_shape.size() == 2 && bias_shape[0] == 1)) &&
                          bias_shape[bias_shape.size() - 1] == gs[1] && gs[0] > 0 && gs[1] > 0;
    if (!f32 || !row_bias)
    {
        // other element types, or a bias of another shape: the operators one after the other
        auto g = matmul_backward_2d(x_, w_, gy_);
        out.push_back(std::move(g.first)), out.push_back(std::move(g.second));
        out.push_back(gy_.sum_to(bias_shape));
        return out;
    }
    const OriginMat &x = dev_f32(x_, "matmul"), &w = dev_f32(w_, "matmul"), &gy = dev_f32(gy_, "matmul");
    const Shape xs = x.shape(), ws_ = w.shape();
    if (xs.size() != 2 || ws_.size() != 2 || xs[1] != ws_[0] || gs[0] != xs[0] || gs[1] != ws_[1])
        THROW_INVALID_ARG("matmul backward: shapes {} {} {} do not form x[M,K] w[K,N] gy[M,N]", xs.to_string(),
                          ws_.to_string(), gs.to_string());
    const int64_t M = xs[0], K = xs[1], N = ws_[1];
    auto gx = new_like(x, xs);
    auto gw = new_like(w, ws_);
    auto gb = new_like(gy, bias_shape);
    Workspace ws(odl_hip_linear_backward_workspace_bytes(M, K, N), x.device().index());
    check(odl_hip_linear_backward(fp(x), fp(w), fp(gy), gx->data_ptr<float>(), gw->data_ptr<float>(), gb->data_ptr<float>(), M,
                                  K, N, ws.ptr(), ws.bytes, cur()));
    out.push_back(std::move(gx)), out.push_back(std::move(gw)), out.push_back(std::move(gb));
    return out;
}

float OriginMat::accuracy(const Mat &target_int32) const
{
    const OriginMat &y = dev_f32(*this, "accuracy");
    const OriginMat &t = as_origin(target_int32);
    if (t.dtype() != DataType::kInt32 || t.device() != device())
        THROW_INVALID_ARG("accuracy: target must be int32 on the same device");
    Workspace ws(odl_hip_accuracy_workspace_bytes((int64_t)shape_[0]), device().index());
    float acc = 0.f;
    check(odl_hip_accuracy(fp(y), t.data_ptr<int32_t>(), (int64_t)shape_[0], (int64_t)shape_[1], &acc, ws.ptr(),
                           ws.bytes, cur()));
    return acc;
}

// ----------------------------------------------------------------------------------- streams and graphs
namespace cuda
{
void *create_stream()
{
    void *s = nullptr;
    check(odl_hip_stream_create(&s));
    return s;
}

void destroy_stream(void *stream)
{
    if (stream && stream == t_stream)
        set_stream(nullptr);
    check(odl_hip_stream_destroy(stream));
}

void set_stream(void *stream)
{
    if (t_capturing)
        THROW_RUNTIME_ERROR("the stream cannot be changed while a graph is being captured");
    if (stream == t_stream)
        return;
    check(odl_hip_synchronize());  // memory freed under the old stream may be handed out under the new one
    t_stream = stream;
}

void *current_stream()
{
    return t_stream;
}

bool is_capturing()
{
    return t_capturing;
}

void empty_cache()
{
    check(odl_hip_synchronize());
    DevicePool::get().trim();
}

Graph::~Graph()
{
    // a Graph destroyed in the middle of its capture (an exception unwound past it) must not leave the thread recording
    if (began_)
        abort_capture();
    if (exec_)
    {
        (void)odl_hip_synchronize();  // no replay may still be running when its memory is handed back
        (void)odl_hip_graph_destroy(exec_);
    }
}

void Graph::begin_capture()
{
    if (exec_)
        THROW_RUNTIME_ERROR("this graph has been captured already");
    if (!t_stream)
        THROW_RUNTIME_ERROR("graph capture needs a created stream (cuda::set_stream): the null stream cannot be captured");
    run_pending_fills_of_this_thread();
    check(odl_hip_stream_synchronize(t_stream));
    arena_ = DevicePool::get().begin_capture();
    if (odl_hip_graph_capture_begin(t_stream) != ODL_OK)
    {
        DevicePool::get().end_capture();
        arena_.reset();
        THROW_RUNTIME_ERROR("{}", odl_hip_last_error());
    }
    t_capturing = true;
    began_ = true;
}

void Graph::abort_capture()
{
    if (!began_)
        return;
    began_ = false;
    t_capturing = false;
    DevicePool::get().end_capture();
    (void)odl_hip_graph_capture_abort(t_stream);
    (void)odl_hip_stream_synchronize(t_stream);
    arena_.reset();  // the blocks of the capture run return to the ordinary pool as their tensors die
}

void Graph::end_capture()
{
    if (!t_capturing)
        THROW_RUNTIME_ERROR("end_capture without begin_capture");
    if (!began_)
        THROW_RUNTIME_ERROR("end_capture on a Graph that did not begin the capture in progress");
    began_ = false;
    t_capturing = false;
    DevicePool::get().end_capture();
    void *exec = nullptr;
    if (odl_hip_graph_capture_end(t_stream, &exec) != ODL_OK)
    {
        arena_.reset();
        THROW_RUNTIME_ERROR("{}", odl_hip_last_error());
    }
    exec_ = exec;
    int64_t nodes = 0;
    if (odl_hip_graph_last_node_count(&nodes) == ODL_OK)
        nodes_ = (size_t)nodes;
}

void Graph::launch()
{
    if (!exec_)
        THROW_RUNTIME_ERROR("this graph has not been captured");
    check(odl_hip_graph_launch(exec_, t_stream));
}
}  // namespace cuda
}  // namespace origin
