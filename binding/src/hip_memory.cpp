// The memory layer of OriginDL with its device branch on the gfx950 backend: this one translation unit stands where the
// reference's src/mat/origin/memory/{allocator,storage,memory_pool_manager}.cpp stand (their device branches are CUDA
// runtime calls), against the reference's own class declarations (include/origin/mat/origin/memory/*.h). MemoryPool
// (memory_pool.cpp) has no device code and is the reference's own object.
//
//   Allocator::allocate / deallocate   allocator.cpp:53-107   -> odl_hip_set_device + odl_hip_malloc / odl_hip_free
//   Storage::to_device                 storage.cpp:69-145     -> odl_hip_memcpy_{h2d,d2h,d2d} (synchronous, like cudaMemcpy)
//   MemoryPoolManager::initialize      memory_pool_manager.cpp:28-52 -> odl_hip_device_count
#include <cstdlib>
#include <cstring>

#include "odl_hip.h"
#include "origin/mat/origin/memory/allocator.h"
#include "origin/mat/origin/memory/memory_pool.h"
#include "origin/mat/origin/memory/memory_pool_manager.h"
#include "origin/mat/origin/memory/storage.h"
#include "origin/utils/exception.h"

namespace origin
{
namespace
{
constexpr size_t kAlign = 128;  // sizes are rounded to whole 128-byte lines on both sides, as in the reference

void device_call(int rc, const char *what)
{
    if (rc == ODL_OK)
        return;
    if (rc == ODL_ERR_INVALID_ARG)
        THROW_INVALID_ARG("{}: {}", what, odl_hip_last_error());
    THROW_RUNTIME_ERROR("{}: {}", what, odl_hip_last_error());
}
}  // namespace

// ---- allocators
void *CPUAllocator::allocate(size_t size)
{
    const size_t bytes = (size + kAlign - 1) / kAlign * kAlign;
    void *p = std::aligned_alloc(kAlign, bytes ? bytes : kAlign);
    if (!p)
        throw std::bad_alloc();
    return p;
}

void CPUAllocator::deallocate(void *ptr)
{
    std::free(ptr);
}

void *CUDAAllocator::allocate(size_t size)
{
    device_call(odl_hip_set_device(device_index_), "set device");
    const size_t bytes = (size + kAlign - 1) / kAlign * kAlign;
    void *p = nullptr;
    if (odl_hip_malloc(&p, bytes ? bytes : kAlign) != ODL_OK)
    {
        size_t free_b = 0, total_b = 0;
        (void)odl_hip_mem_info(&free_b, &total_b);
        THROW_RUNTIME_ERROR("device memory allocation failed: {} (requested {} bytes on device {}; free {} of {} bytes)",
                            odl_hip_last_error(), size, device_index_, free_b, total_b);
    }
    return p;
}

void CUDAAllocator::deallocate(void *ptr)
{
    if (!ptr)
        return;
    device_call(odl_hip_set_device(device_index_), "set device");
    device_call(odl_hip_free(ptr), "device memory release");
}

std::unique_ptr<Allocator> AllocatorFactory::create_allocator(DeviceType device_type, int device_index)
{
    if (device_type == DeviceType::kCPU)
        return std::make_unique<CPUAllocator>();
    if (device_type == DeviceType::kCUDA)
        return std::make_unique<CUDAAllocator>(device_index);
    THROW_INVALID_ARG("Unsupported device type: {}", static_cast<int>(device_type));
}

// ---- one pool per device, the host's last
MemoryPoolManager::MemoryPoolManager() : max_cuda_devices_(0)
{
    initialize_pools();
}

MemoryPoolManager &MemoryPoolManager::get_instance()
{
    static MemoryPoolManager manager;
    return manager;
}

void MemoryPoolManager::initialize_pools()
{
    if (!pools_.empty())
        return;
    int n = 0;
    max_cuda_devices_ = odl_hip_device_count(&n) == ODL_OK ? n : 0;
    pools_.resize((size_t)max_cuda_devices_ + 1);
}

int MemoryPoolManager::get_pool_index(DeviceType device_type, int device_index) const
{
    if (device_type == DeviceType::kCPU)
        return (int)pools_.size() - 1;
    if (device_type != DeviceType::kCUDA)
        THROW_INVALID_ARG("Unsupported device type: {}", static_cast<int>(device_type));
    if (device_index < 0 || device_index >= max_cuda_devices_)
        THROW_INVALID_ARG("Invalid CUDA device index: {}, max devices: {}", device_index, max_cuda_devices_);
    return device_index;
}

MemoryPool *MemoryPoolManager::get_memory_pool(DeviceType device_type, int device_index)
{
    std::lock_guard<std::mutex> lock(mutex_);
    const int i = get_pool_index(device_type, device_index);
    if (!pools_[i])
        pools_[i] = std::make_unique<MemoryPool>(device_type, device_index);
    return pools_[i].get();
}

// ---- storage
Storage::Storage(size_t size, DeviceType device_type, int device_index)
    : data_(nullptr), size_(size), device_type_(device_type), device_index_(device_index),
      pool_(MemoryPoolManager::get_instance().get_memory_pool(device_type, device_index))
{
    data_ = pool_->malloc(size_);
}

Storage::~Storage()
{
    if (data_)
        pool_->free(data_);
}

Storage::Storage(Storage &&o) noexcept
    : data_(o.data_), size_(o.size_), device_type_(o.device_type_), device_index_(o.device_index_), pool_(o.pool_)
{
    o.data_ = nullptr, o.size_ = 0;
}

Storage &Storage::operator=(Storage &&o) noexcept
{
    if (this != &o)
    {
        if (data_)
            pool_->free(data_);
        data_ = o.data_, size_ = o.size_, device_type_ = o.device_type_, device_index_ = o.device_index_, pool_ = o.pool_;
        o.data_ = nullptr, o.size_ = 0;
    }
    return *this;
}

std::shared_ptr<Storage> Storage::create(size_t size, DeviceType device_type, int device_index)
{
    return std::shared_ptr<Storage>(new Storage(size, device_type, device_index));
}

// A copy on the target device. Copies that touch the host are synchronous and wait for the device first, as the
// reference's are (storage.cpp:100-106): whoever reads the host copy finds the results of every kernel queued before.
std::shared_ptr<Storage> Storage::to_device(DeviceType target_type, int target_index) const
{
    if (target_type != DeviceType::kCPU && target_type != DeviceType::kCUDA)
        THROW_RUNTIME_ERROR("Unsupported device transfer from {} to {}", Device(device_type_, device_index_).to_string(),
                            Device(target_type, target_index).to_string());
    auto dst = create(size_, target_type, target_type == DeviceType::kCPU ? 0 : target_index);
    if (size_ == 0)
        return dst;
    const bool from_host = device_type_ == DeviceType::kCPU, to_host = target_type == DeviceType::kCPU;
    if (from_host && to_host)
        std::memcpy(dst->data(), data_, size_);
    else if (from_host)
        device_call(odl_hip_memcpy_h2d(dst->data(), data_, size_, nullptr), "host-to-device copy");
    else if (to_host)
        device_call(odl_hip_memcpy_d2h(dst->data(), data_, size_), "device-to-host copy");
    else
        device_call(odl_hip_memcpy_d2d(dst->data(), data_, size_, nullptr), "device-to-device copy");
    return dst;
}
}  // namespace origin
