// Device / memory / stream / event entry points of the C ABI: thin, checked
// wrappers over the HIP runtime (the counterpart of cacti_gpu_cu_ffi/src/lib.rs:98-565).
#include <stdarg.h>
#include <atomic>
#include <string.h>

#include "common.h"

namespace cacti {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

static std::atomic<unsigned> g_module_epoch{1};
unsigned module_epoch() { return g_module_epoch.load(std::memory_order_relaxed); }
void module_epoch_advance() { g_module_epoch.fetch_add(1, std::memory_order_relaxed); }
static std::atomic<int> g_live_contexts[64];
int live_contexts(int dev) { return dev >= 0 && dev < 64 ? g_live_contexts[dev].load() : 0; }
void live_contexts_add(int dev, int n)
{
    if (dev >= 0 && dev < 64) g_live_contexts[dev].fetch_add(n);
}

int hip_status(hipError_t e, const char *what)
{
    if (e == hipSuccess) return 0;
    set_error("%s: %s (%d)", what, hipGetErrorString(e), (int)e);
    // the runtime also remembers the failure per thread; it has been reported here, and left in place it
    // would be taken for the status of the next kernel launch (launch_status reads that record)
    (void)hipGetLastError();
    return (int)e;
}

}  // namespace cacti

using namespace cacti;

CACTI_API const char *cacti_hip_last_error(void) { return g_err; }

CACTI_API int cacti_hip_device_count(int *count)
{
    CACTI_REQUIRE(count, CACTI_E_INVALID, "device_count: null out pointer");
    CACTI_HIP(hipGetDeviceCount(count));
    return 0;
}
CACTI_API int cacti_hip_device_get(int *dev)
{
    CACTI_REQUIRE(dev, CACTI_E_INVALID, "device_get: null out pointer");
    CACTI_HIP(hipGetDevice(dev));
    return 0;
}
CACTI_API int cacti_hip_device_set(int dev)
{
    CACTI_HIP(hipSetDevice(dev));
    return 0;
}
CACTI_API int cacti_hip_device_attribute(int dev, int attr, int *value)
{
    CACTI_REQUIRE(value, CACTI_E_INVALID, "device_attribute: null out pointer");
    CACTI_HIP(hipDeviceGetAttribute(value, (hipDeviceAttribute_t)attr, dev));
    return 0;
}
CACTI_API int cacti_hip_device_sync(void)
{
    CACTI_HIP(hipDeviceSynchronize());
    return 0;
}
CACTI_API int cacti_hip_mem_get_info(size_t *free_bytes, size_t *total_bytes)
{
    CACTI_REQUIRE(free_bytes && total_bytes, CACTI_E_INVALID, "mem_get_info: null out pointer");
    CACTI_HIP(hipMemGetInfo(free_bytes, total_bytes));
    return 0;
}
CACTI_API int cacti_hip_mem_alloc(void **dptr, size_t bytes)
{
    CACTI_REQUIRE(dptr, CACTI_E_INVALID, "mem_alloc: null out pointer");
    CACTI_HIP(hipMalloc(dptr, bytes));
    return 0;
}
CACTI_API int cacti_hip_mem_free(void *dptr)
{
    CACTI_HIP(hipFree(dptr));
    return 0;
}
CACTI_API int cacti_hip_mem_alloc_host(void **ptr, size_t bytes)
{
    CACTI_REQUIRE(ptr, CACTI_E_INVALID, "mem_alloc_host: null out pointer");
    CACTI_HIP(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
    return 0;
}
CACTI_API int cacti_hip_mem_free_host(void *ptr)
{
    CACTI_HIP(hipHostFree(ptr));
    return 0;
}
CACTI_API int cacti_hip_memcpy_d2h(void *dst, const void *src, size_t bytes)
{
    CACTI_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return 0;
}
CACTI_API int cacti_hip_memcpy_async(void *dst, const void *src, size_t bytes, void *stream)
{
    CACTI_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
    return 0;
}
CACTI_API int cacti_hip_memcpy_h2d_async(void *dst, const void *src, size_t bytes, void *stream)
{
    CACTI_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
    return 0;
}
CACTI_API int cacti_hip_memcpy_d2h_async(void *dst, const void *src, size_t bytes, void *stream)
{
    CACTI_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
    return 0;
}
CACTI_API int cacti_hip_memset_async(void *dst, int byte, size_t bytes, void *stream)
{
    CACTI_HIP(hipMemsetAsync(dst, byte, bytes, (hipStream_t)stream));
    return 0;
}
CACTI_API int cacti_hip_stream_create(void **stream)
{
    CACTI_REQUIRE(stream, CACTI_E_INVALID, "stream_create: null out pointer");
    CACTI_HIP(hipStreamCreate((hipStream_t *)stream));
    return 0;
}
CACTI_API int cacti_hip_stream_create_nonblocking(void **stream)
{
    CACTI_REQUIRE(stream, CACTI_E_INVALID, "stream_create_nonblocking: null out pointer");
    CACTI_HIP(hipStreamCreateWithFlags((hipStream_t *)stream, hipStreamNonBlocking));
    return 0;
}
CACTI_API int cacti_hip_stream_destroy(void *stream)
{
    CACTI_HIP(hipStreamDestroy((hipStream_t)stream));
    return 0;
}
CACTI_API int cacti_hip_stream_sync(void *stream)
{
    CACTI_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}
CACTI_API int cacti_hip_stream_wait_event(void *stream, void *event)
{
    CACTI_HIP(hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)event, 0));
    return 0;
}
CACTI_API int cacti_hip_event_create(void **event, int enable_timing)
{
    CACTI_REQUIRE(event, CACTI_E_INVALID, "event_create: null out pointer");
    CACTI_HIP(hipEventCreateWithFlags((hipEvent_t *)event,
                                      enable_timing ? hipEventDefault : hipEventDisableTiming));
    return 0;
}
CACTI_API int cacti_hip_event_destroy(void *event)
{
    CACTI_HIP(hipEventDestroy((hipEvent_t)event));
    return 0;
}
CACTI_API int cacti_hip_event_record(void *event, void *stream)
{
    CACTI_HIP(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
    return 0;
}
CACTI_API int cacti_hip_event_query(void *event)
{
    hipError_t e = hipEventQuery((hipEvent_t)event);
    if (e == hipErrorNotReady) return (int)e;   // not an error: still pending
    return hip_status(e, "hipEventQuery");
}
CACTI_API int cacti_hip_event_sync(void *event)
{
    CACTI_HIP(hipEventSynchronize((hipEvent_t)event));
    return 0;
}
CACTI_API int cacti_hip_event_elapsed_ms(void *start, void *stop, float *ms)
{
    CACTI_REQUIRE(ms, CACTI_E_INVALID, "event_elapsed_ms: null out pointer");
    CACTI_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return 0;
}
