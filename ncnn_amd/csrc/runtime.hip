// Device plumbing behind the C ABI: buffers, streams, events, error text.
#include <stdarg.h>

#include <atomic>
#include <mutex>
#include <string.h>

#include "common.h"
#include "conv_nhwc.h"

namespace ncnnhip {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int map_hip_error(hipError_t e, const char* what)
{
    set_error("%s: %s", what, hipGetErrorString(e));
    (void)hipGetLastError(); // clear the sticky per-thread error
    return e == hipErrorOutOfMemory ? NCNNHIP_OOM : NCNNHIP_ERROR;
}

} // namespace ncnnhip

using namespace ncnnhip;

extern "C" {

int ncnnhip_init(int device)
{
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
    {
        set_error("no HIP device available (%s)", e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
        (void)hipGetLastError();
        return NCNNHIP_ERROR;
    }
    NCNNHIP_REQUIRE(device >= 0 && device < count, "device %d out of range (count %d)", device, count);
    NCNNHIP_CHECK(hipSetDevice(device));
    hipDeviceProp_t prop;
    NCNNHIP_CHECK(hipGetDeviceProperties(&prop, device));
    NCNNHIP_REQUIRE(strncmp(prop.gcnArchName, "gfx950", 6) == 0, "kernels are built for gfx950 only, device is %s",
                    prop.gcnArchName);
    // this device's address of the library-held scratch (ncnnhip_innerproduct_int8_noalloc), looked up once per device
    void* scratch_ptr = 0;
    return static_scratch_for_current_device(&scratch_ptr);
}

const char* ncnnhip_last_error(void)
{
    return g_error;
}

int ncnnhip_device_info(char* name, size_t name_len, int* compute_units, size_t* total_mem)
{
    int dev = 0;
    NCNNHIP_CHECK(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    NCNNHIP_CHECK(hipGetDeviceProperties(&prop, dev));
    if (name && name_len)
    {
        snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
    }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (total_mem) *total_mem = prop.totalGlobalMem;
    return NCNNHIP_OK;
}

int ncnnhip_stream_create(void** stream)
{
    NCNNHIP_REQUIRE(stream, "null stream out pointer");
    hipStream_t s;
    NCNNHIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = s;
    return NCNNHIP_OK;
}

int ncnnhip_stream_destroy(void* stream)
{
    if (stream) NCNNHIP_CHECK(hipStreamDestroy(as_stream(stream)));
    return NCNNHIP_OK;
}

int ncnnhip_stream_synchronize(void* stream)
{
    NCNNHIP_CHECK(hipStreamSynchronize(as_stream(stream)));
    return NCNNHIP_OK;
}

int ncnnhip_copy2d(void* dst_dev, size_t dst_pitch, const void* src_dev, size_t src_pitch, size_t row_bytes, size_t rows, void* stream)
{
    NCNNHIP_REQUIRE(dst_dev && src_dev && dst_pitch >= row_bytes && src_pitch >= row_bytes, "ncnnhip_copy2d: bad argument");
    if (row_bytes == 0 || rows == 0) return NCNNHIP_OK;
    NCNNHIP_CHECK(hipMemcpy2DAsync(dst_dev, dst_pitch, src_dev, src_pitch, row_bytes, rows, hipMemcpyDeviceToDevice, as_stream(stream)));
    return NCNNHIP_OK;
}

int ncnnhip_stream_begin_capture(void* stream)
{
    NCNNHIP_REQUIRE(stream, "ncnnhip_stream_begin_capture: the default stream cannot be captured");
    // thread-local: other threads keep allocating and synchronising; on this thread anything but stream work is an error
    NCNNHIP_CHECK(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal));
    return NCNNHIP_OK;
}

int ncnnhip_stream_end_capture(void* stream, void** graph_exec)
{
    NCNNHIP_REQUIRE(stream && graph_exec, "ncnnhip_stream_end_capture: null pointer");
    *graph_exec = 0;
    hipGraph_t graph = 0;
    NCNNHIP_CHECK(hipStreamEndCapture(as_stream(stream), &graph));
    NCNNHIP_REQUIRE(graph, "ncnnhip_stream_end_capture: the capture was invalidated");
    hipGraphExec_t exec = 0;
    const hipError_t e = hipGraphInstantiate(&exec, graph, 0, 0, 0);
    (void)hipGraphDestroy(graph);
    NCNNHIP_CHECK(e);
    *graph_exec = exec;
    return NCNNHIP_OK;
}

int ncnnhip_graph_launch(void* graph_exec, void* stream)
{
    NCNNHIP_REQUIRE(graph_exec, "ncnnhip_graph_launch: null graph");
    NCNNHIP_CHECK(hipGraphLaunch((hipGraphExec_t)graph_exec, as_stream(stream)));
    return NCNNHIP_OK;
}

int ncnnhip_graph_destroy(void* graph_exec)
{
    if (graph_exec) NCNNHIP_CHECK(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
    return NCNNHIP_OK;
}

int ncnnhip_device_synchronize(void)
{
    NCNNHIP_CHECK(hipDeviceSynchronize());
    return NCNNHIP_OK;
}

// The device allocator every buffer of the library comes from: hipMalloc / hipFree unless the caller has installed a
// table of its own (a pool it already runs, an arena per request, an allocator that refuses: the out-of-memory tests).
static int default_device_malloc(void** dev, size_t bytes, void*)
{
    hipError_t e = hipMalloc(dev, bytes);
    if (e != hipSuccess) return map_hip_error(e, "hipMalloc");
    return NCNNHIP_OK;
}
static int default_device_free(void* dev, void*)
{
    hipError_t e = hipFree(dev);
    if (e != hipSuccess) return map_hip_error(e, "hipFree");
    return NCNNHIP_OK;
}
struct DeviceAllocator
{
    ncnnhip_device_malloc_fn malloc_fn;
    ncnnhip_device_free_fn free_fn;
    void* user;
};
static std::mutex g_allocator_mutex;
static DeviceAllocator g_allocator = {default_device_malloc, default_device_free, 0};

int ncnnhip_set_device_allocator(ncnnhip_device_malloc_fn malloc_fn, ncnnhip_device_free_fn free_fn, void* user)
{
    NCNNHIP_REQUIRE((malloc_fn != 0) == (free_fn != 0), "ncnnhip_set_device_allocator: give both functions, or neither to restore hipMalloc / hipFree");
    std::lock_guard<std::mutex> lock(g_allocator_mutex);
    if (malloc_fn)
        g_allocator = {malloc_fn, free_fn, user};
    else
        g_allocator = {default_device_malloc, default_device_free, 0};
    return NCNNHIP_OK;
}

int ncnnhip_default_device_malloc(void** dev, size_t bytes)
{
    NCNNHIP_REQUIRE(dev, "null out pointer");
    return default_device_malloc(dev, bytes, 0);
}

int ncnnhip_default_device_free(void* dev)
{
    return dev ? default_device_free(dev, 0) : NCNNHIP_OK;
}

int ncnnhip_malloc(void** dev, size_t bytes)
{
    NCNNHIP_REQUIRE(dev, "null out pointer");
    *dev = 0;
    if (bytes == 0) bytes = 4;
    DeviceAllocator a;
    {
        std::lock_guard<std::mutex> lock(g_allocator_mutex);
        a = g_allocator;
    }
    const int ret = a.malloc_fn(dev, bytes, a.user);
    if (ret != NCNNHIP_OK || !*dev)
    {
        *dev = 0;
        if (ret == NCNNHIP_OK || a.malloc_fn != default_device_malloc) set_error("ncnnhip_malloc: the device allocator refused %zu bytes", bytes);
        return NCNNHIP_OOM;
    }
    return NCNNHIP_OK;
}

int ncnnhip_free(void* dev)
{
    if (!dev) return NCNNHIP_OK;
    DeviceAllocator a;
    {
        std::lock_guard<std::mutex> lock(g_allocator_mutex);
        a = g_allocator;
    }
    return a.free_fn(dev, a.user);
}

int ncnnhip_memcpy_h2d(void* dev, const void* host, size_t bytes, void* stream)
{
    if (bytes == 0) return NCNNHIP_OK;
    NCNNHIP_CHECK(hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    return NCNNHIP_OK;
}

int ncnnhip_memcpy_d2h(void* host, const void* dev, size_t bytes, void* stream)
{
    if (bytes == 0) return NCNNHIP_OK;
    NCNNHIP_CHECK(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    return NCNNHIP_OK;
}

int ncnnhip_memcpy_d2d(void* dst_dev, const void* src_dev, size_t bytes, void* stream)
{
    if (bytes == 0) return NCNNHIP_OK;
    NCNNHIP_CHECK(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return NCNNHIP_OK;
}

int ncnnhip_memset(void* dev, int byte, size_t bytes, void* stream)
{
    if (bytes == 0) return NCNNHIP_OK;
    NCNNHIP_CHECK(hipMemsetAsync(dev, byte, bytes, as_stream(stream)));
    return NCNNHIP_OK;
}

int ncnnhip_event_create(void** event)
{
    NCNNHIP_REQUIRE(event, "null out pointer");
    hipEvent_t e;
    // timing events only: no system-scope cache flush when the event is recorded (it would sit between the kernels being timed)
    NCNNHIP_CHECK(hipEventCreateWithFlags(&e, hipEventDisableSystemFence));
    *event = e;
    return NCNNHIP_OK;
}

int ncnnhip_event_destroy(void* event)
{
    if (event) NCNNHIP_CHECK(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
    return NCNNHIP_OK;
}

int ncnnhip_event_record(void* event, void* stream)
{
    NCNNHIP_CHECK(hipEventRecord(reinterpret_cast<hipEvent_t>(event), as_stream(stream)));
    return NCNNHIP_OK;
}

int ncnnhip_event_synchronize(void* event)
{
    NCNNHIP_CHECK(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)));
    return NCNNHIP_OK;
}

int ncnnhip_event_elapsed_ms(void* start, void* stop, float* ms)
{
    NCNNHIP_CHECK(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start), reinterpret_cast<hipEvent_t>(stop)));
    return NCNNHIP_OK;
}

} // extern "C"
