// Device runtime entry points of the C ABI: device selection, memory, copies, error text.
// They stand where the reference's CUDAAllocator / Storage / origin::cuda::* device API make their
// runtime calls (src/mat/origin/memory/allocator.cpp:53-107, storage.cpp:69-145, cuda/cuda_utils.cu:37-91).
#include <cstring>

#include "odl_common.h"

namespace
{
thread_local char g_error[512] = "";
}

namespace odl
{
void set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int require_device()
{
    // one check per device; the kernels are compiled for gfx950 only and there is no other code path
    static int checked[64] = {0};  // 0 unknown, 1 ok, -1 wrong architecture
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0)
        return fail(ODL_ERR_RUNTIME, "no HIP device available: %s", hipGetErrorString(e));
    if (dev < 64 && checked[dev] == 1)
        return ODL_OK;
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess)
        return fail(ODL_ERR_RUNTIME, "hipGetDeviceProperties failed: %s", hipGetErrorString(e));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    {
        if (dev < 64)
            checked[dev] = -1;
        return fail(ODL_ERR_RUNTIME, "device %d is %s; this library contains gfx950 code only", dev, prop.gcnArchName);
    }
    if (dev < 64)
        checked[dev] = 1;
    return ODL_OK;
}

Chip chip()
{
    static Chip known[64] = {};
    const Chip whole{256, 8};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
    {
        (void)hipGetLastError();
        return whole;
    }
    if (known[dev].cus > 0)
        return known[dev];
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess || prop.multiProcessorCount <= 0)
    {
        (void)hipGetLastError();
        return whole;
    }
    // gfx950 exposes 32 compute units per XCD
    Chip c{prop.multiProcessorCount, prop.multiProcessorCount >= 64 ? prop.multiProcessorCount / 32 : 1};
    known[dev] = c;
    return c;
}
}  // namespace odl

extern "C" {

const char *odl_hip_last_error(void)
{
    return g_error;
}

int odl_hip_device_count(int *count)
{
    ODL_REQUIRE(count != nullptr, "device_count: null output");
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess)
    {
        (void)hipGetLastError();
        n = 0;
    }
    *count = n;
    return ODL_OK;
}

int odl_hip_set_device(int device)
{
    ODL_HIP_CHECK(hipSetDevice(device));
    return ODL_OK;
}

int odl_hip_get_device(int *device)
{
    ODL_REQUIRE(device != nullptr, "get_device: null output");
    ODL_HIP_CHECK(hipGetDevice(device));
    return ODL_OK;
}

int odl_hip_synchronize(void)
{
    ODL_HIP_CHECK(hipDeviceSynchronize());
    return ODL_OK;
}

int odl_hip_device_info(int device, char *buf, size_t len)
{
    ODL_REQUIRE(buf != nullptr && len > 0, "device_info: null buffer");
    hipDeviceProp_t prop;
    ODL_HIP_CHECK(hipGetDeviceProperties(&prop, device));
    snprintf(buf, len, "%s | %s | %d CUs | %d MHz | %zu MiB", prop.name, prop.gcnArchName, prop.multiProcessorCount,
             prop.clockRate / 1000, (size_t)(prop.totalGlobalMem >> 20));
    return ODL_OK;
}

int odl_hip_malloc(void **ptr, size_t bytes)
{
    ODL_REQUIRE(ptr != nullptr, "malloc: null output");
    *ptr = nullptr;
    if (bytes == 0)
        return ODL_OK;
    hipError_t e = hipMalloc(ptr, bytes);
    if (e != hipSuccess)
    {
        size_t fr = 0, tot = 0;
        (void)hipMemGetInfo(&fr, &tot);  // the reference reports free/total on OOM (allocator.cpp:69-80)
        return odl::fail(ODL_ERR_RUNTIME, "hipMalloc(%zu) failed: %s (free %zu MiB of %zu MiB)", bytes,
                         hipGetErrorString(e), fr >> 20, tot >> 20);
    }
    return ODL_OK;
}

int odl_hip_free(void *ptr)
{
    if (ptr)
        ODL_HIP_CHECK(hipFree(ptr));
    return ODL_OK;
}

int odl_hip_mem_info(size_t *free_bytes, size_t *total_bytes)
{
    size_t fr = 0, tot = 0;
    ODL_HIP_CHECK(hipMemGetInfo(&fr, &tot));
    if (free_bytes)
        *free_bytes = fr;
    if (total_bytes)
        *total_bytes = tot;
    return ODL_OK;
}

int odl_hip_memcpy_h2d(void *dst, const void *host_src, size_t bytes, void *stream)
{
    if (!bytes)
        return ODL_OK;
    if (stream == nullptr)
    {
        ODL_HIP_CHECK(hipMemcpy(dst, host_src, bytes, hipMemcpyHostToDevice));
        return ODL_OK;
    }
    // A created stream does not wait for the null stream nor the null stream for it: the copy goes onto the stream
    // itself, behind every kernel queued there (one of them may still be using the block `dst` was recycled from),
    // and the call returns when it has landed, so the host buffer can be reused at once.
    ODL_HIP_CHECK(hipMemcpyAsync(dst, host_src, bytes, hipMemcpyHostToDevice, odl::as_stream(stream)));
    ODL_HIP_CHECK(hipStreamSynchronize(odl::as_stream(stream)));
    return ODL_OK;
}

int odl_hip_memcpy_d2h(void *host_dst, const void *src, size_t bytes)
{
    if (bytes)
    {
        ODL_HIP_CHECK(hipDeviceSynchronize());  // storage.cpp:100-101
        ODL_HIP_CHECK(hipMemcpy(host_dst, src, bytes, hipMemcpyDeviceToHost));
    }
    return ODL_OK;
}

int odl_hip_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream)
{
    if (bytes)
        ODL_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, odl::as_stream(stream)));
    return ODL_OK;
}

int odl_hip_memset(void *dst, int value, size_t bytes, void *stream)
{
    return odl::fill_bytes_launch(dst, value, bytes, odl::as_stream(stream));
}

// ---- streams and captured graphs. A step whose shapes and pointers do not change from one iteration to the next
// (a training step on a fixed batch shape, an inference forward) is dozens of launches of microsecond kernels; recorded
// once into a graph and replayed, it costs one submission.
int odl_hip_stream_create(void **stream)
{
    ODL_REQUIRE(stream != nullptr, "stream_create: null output");
    hipStream_t s = nullptr;
    ODL_HIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));  // default priority
    *stream = s;
    return ODL_OK;
}

int odl_hip_stream_destroy(void *stream)
{
    if (stream)
        ODL_HIP_CHECK(hipStreamDestroy(odl::as_stream(stream)));
    return ODL_OK;
}

int odl_hip_device_synchronize(void)
{
    ODL_HIP_CHECK(hipDeviceSynchronize());
    return ODL_OK;
}

int odl_hip_host_alloc(void **ptr, size_t bytes)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(ptr != nullptr && bytes > 0, "host_alloc: null result pointer or zero size");
    ODL_HIP_CHECK(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
    return ODL_OK;
}

int odl_hip_host_free(void *ptr)
{
    if (ptr)
        ODL_HIP_CHECK(hipHostFree(ptr));
    return ODL_OK;
}

int odl_hip_stream_synchronize(void *stream)
{
    ODL_HIP_CHECK(hipStreamSynchronize(odl::as_stream(stream)));
    return ODL_OK;
}

int odl_hip_graph_capture_begin(void *stream)
{
    ODL_REQUIRE(stream != nullptr, "graph capture needs a created stream: the null stream cannot be captured");
    ODL_HIP_CHECK(hipStreamBeginCapture(odl::as_stream(stream), hipStreamCaptureModeRelaxed));
    return ODL_OK;
}

int odl_hip_event_create(void **event)
{
    ODL_REQUIRE(event != nullptr, "event_create: null argument");
    hipEvent_t e = nullptr;
    ODL_HIP_CHECK(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    *event = e;
    return ODL_OK;
}

int odl_hip_event_destroy(void *event)
{
    if (event)
        ODL_HIP_CHECK(hipEventDestroy(static_cast<hipEvent_t>(event)));
    return ODL_OK;
}

int odl_hip_event_record(void *event, void *stream)
{
    ODL_REQUIRE(event != nullptr, "event_record: null event");
    ODL_HIP_CHECK(hipEventRecord(static_cast<hipEvent_t>(event), odl::as_stream(stream)));
    return ODL_OK;
}

int odl_hip_event_synchronize(void *event)
{
    ODL_REQUIRE(event != nullptr, "event_synchronize: null event");
    ODL_HIP_CHECK(hipEventSynchronize(static_cast<hipEvent_t>(event)));
    return ODL_OK;
}

static thread_local int64_t t_last_graph_nodes = 0;

int odl_hip_graph_last_node_count(int64_t *nodes)
{
    ODL_REQUIRE(nodes != nullptr, "graph_last_node_count: null argument");
    *nodes = t_last_graph_nodes;
    return ODL_OK;
}

int odl_hip_graph_capture_end(void *stream, void **graph_exec)
{
    ODL_REQUIRE(stream != nullptr && graph_exec != nullptr, "graph_capture_end: null argument");
    *graph_exec = nullptr;
    hipGraph_t graph = nullptr;
    ODL_HIP_CHECK(hipStreamEndCapture(odl::as_stream(stream), &graph));
    if (graph == nullptr)
        return odl::fail(ODL_ERR_RUNTIME, "graph capture produced no graph (an operation that cannot be captured ended it)");
    size_t nodes = 0;
    if (hipGraphGetNodes(graph, nullptr, &nodes) != hipSuccess)
        (void)hipGetLastError(), nodes = 0;
    t_last_graph_nodes = (int64_t)nodes;
    hipGraphExec_t exec = nullptr;
    const hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess)
        return odl::fail(ODL_ERR_RUNTIME, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
    *graph_exec = exec;
    return ODL_OK;
}

int odl_hip_graph_capture_abort(void *stream)
{
    ODL_REQUIRE(stream != nullptr, "graph_capture_abort: null stream");
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(odl::as_stream(stream), &status) != hipSuccess)
        (void)hipGetLastError();
    if (status == hipStreamCaptureStatusNone)
        return ODL_OK;
    // ending an invalidated capture reports an error and hands back no graph: both are what is wanted here
    hipGraph_t graph = nullptr;
    if (hipStreamEndCapture(odl::as_stream(stream), &graph) != hipSuccess)
        (void)hipGetLastError();
    if (graph)
        (void)hipGraphDestroy(graph);
    return ODL_OK;
}

int odl_hip_graph_launch(void *graph_exec, void *stream)
{
    ODL_REQUIRE(graph_exec != nullptr, "graph_launch: null graph");
    ODL_HIP_CHECK(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), odl::as_stream(stream)));
    return ODL_OK;
}

int odl_hip_graph_destroy(void *graph_exec)
{
    if (graph_exec)
        ODL_HIP_CHECK(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec)));
    return ODL_OK;
}

}  // extern "C"
