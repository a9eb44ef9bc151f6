// Runtime plumbing behind the C ABI: device selection, memory, streams, events, graph capture.
#include "common.hpp"
#include <mutex>

namespace msnh {

static thread_local char g_err[1024] = "";
static hipStream_t       g_defaultStream = nullptr;
static int               g_device = -1;
static std::mutex        g_mutex;

void setError(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

hipStream_t resolveStream(msnh_stream_t s)
{
    return s ? static_cast<hipStream_t>(s) : g_defaultStream;
}

__global__ void fillZeroKernel(uint32_t *dst, size_t words)
{
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (; i < words; i += stride) dst[i] = 0u;
}

} // namespace msnh

using namespace msnh;

extern "C" {

const char *msnh_hip_last_error(void) { return g_err; }

int msnh_hip_init(int device)
{
    std::lock_guard<std::mutex> lock(g_mutex);
    int count = 0;
    MSNH_HIP_CHECK(hipGetDeviceCount(&count));
    MSNH_REQUIRE(count > 0, "no HIP device visible");
    MSNH_REQUIRE(device >= 0 && device < count, "device %d out of range (have %d)", device, count);
    MSNH_HIP_CHECK(hipSetDevice(device));
    if (g_defaultStream == nullptr || g_device != device)
    {
        MSNH_HIP_CHECK(hipStreamCreateWithFlags(&g_defaultStream, hipStreamNonBlocking));
        g_device = device;
    }
    yoloNmsSetupDevice();
    return 0;
}

int msnh_hip_device_count(int *count)
{
    MSNH_REQUIRE(count != nullptr, "count is NULL");
    hipError_t e = hipGetDeviceCount(count);
    if (e != hipSuccess) { *count = 0; (void)hipGetLastError(); }
    return 0;
}

int msnh_hip_device_name(char *dst, int cap, int *cu_count, size_t *total_mem)
{
    hipDeviceProp_t p;
    int dev = 0;
    MSNH_HIP_CHECK(hipGetDevice(&dev));
    MSNH_HIP_CHECK(hipGetDeviceProperties(&p, dev));
    if (dst && cap > 0) snprintf(dst, static_cast<size_t>(cap), "%s (%s)", p.name, p.gcnArchName);
    if (cu_count) *cu_count = p.multiProcessorCount;
    if (total_mem) *total_mem = p.totalGlobalMem;
    return 0;
}

int msnh_hip_malloc(void **dptr, size_t bytes)
{
    MSNH_REQUIRE(dptr != nullptr, "dptr is NULL");
    *dptr = nullptr;
    if (bytes == 0) bytes = 256;
    MSNH_HIP_CHECK(hipMalloc(dptr, bytes));
    return 0;
}

int msnh_hip_free(void *dptr)
{
    if (dptr) MSNH_HIP_CHECK(hipFree(dptr));
    return 0;
}

int msnh_hip_host_alloc(void **hptr, size_t bytes)
{
    MSNH_REQUIRE(hptr != nullptr, "hptr is NULL");
    *hptr = nullptr;
    if (bytes == 0) bytes = 256;
    MSNH_HIP_CHECK(hipHostMalloc(hptr, bytes, hipHostMallocDefault));
    return 0;
}

int msnh_hip_host_free(void *hptr)
{
    if (hptr) MSNH_HIP_CHECK(hipHostFree(hptr));
    return 0;
}

int msnh_hip_memcpy_h2d(void *dst, const void *src, size_t bytes, msnh_stream_t s)
{
    if (bytes == 0) return 0;
    MSNH_REQUIRE(dst && src, "memcpy_h2d: NULL pointer");
    MSNH_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, resolveStream(s)));
    return 0;
}

int msnh_hip_memcpy_d2h(void *dst, const void *src, size_t bytes, msnh_stream_t s)
{
    if (bytes == 0) return 0;
    MSNH_REQUIRE(dst && src, "memcpy_d2h: NULL pointer");
    MSNH_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, resolveStream(s)));
    return 0;
}

int msnh_hip_memcpy_d2d(void *dst, const void *src, size_t bytes, msnh_stream_t s)
{
    if (bytes == 0) return 0;
    MSNH_REQUIRE(dst && src, "memcpy_d2d: NULL pointer");
    MSNH_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, resolveStream(s)));
    return 0;
}

int msnh_hip_fill_zero(void *dst, size_t bytes, msnh_stream_t s)
{
    if (bytes == 0) return 0;
    MSNH_REQUIRE(dst != nullptr, "fill_zero: NULL pointer");
    MSNH_REQUIRE(bytes % 4 == 0 && (reinterpret_cast<uintptr_t>(dst) % 4) == 0, "fill_zero: need 4-byte alignment");
    size_t words = bytes / 4;
    unsigned grid = gridFor(static_cast<long long>(words > (1u << 22) ? (1u << 22) : words), 256);
    hipLaunchKernelGGL(fillZeroKernel, dim3(grid), dim3(256), 0, resolveStream(s), static_cast<uint32_t *>(dst), words);
    MSNH_LAUNCH_CHECK();
    return 0;
}

int msnh_hip_stream_create(msnh_stream_t *s)
{
    MSNH_REQUIRE(s != nullptr, "stream pointer is NULL");
    hipStream_t st;
    MSNH_HIP_CHECK(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));   // default priority only
    *s = st;
    return 0;
}

int msnh_hip_stream_destroy(msnh_stream_t s)
{
    if (s) MSNH_HIP_CHECK(hipStreamDestroy(static_cast<hipStream_t>(s)));
    return 0;
}

int msnh_hip_stream_sync(msnh_stream_t s)
{
    MSNH_HIP_CHECK(hipStreamSynchronize(resolveStream(s)));
    return 0;
}

int msnh_hip_event_create(msnh_event_t *e)
{
    MSNH_REQUIRE(e != nullptr, "event pointer is NULL");
    hipEvent_t ev;
    MSNH_HIP_CHECK(hipEventCreate(&ev));
    *e = ev;
    return 0;
}

int msnh_hip_event_destroy(msnh_event_t e)
{
    if (e) MSNH_HIP_CHECK(hipEventDestroy(static_cast<hipEvent_t>(e)));
    return 0;
}

int msnh_hip_event_record(msnh_event_t e, msnh_stream_t s)
{
    MSNH_REQUIRE(e != nullptr, "event is NULL");
    MSNH_HIP_CHECK(hipEventRecord(static_cast<hipEvent_t>(e), resolveStream(s)));
    return 0;
}

int msnh_hip_stream_wait_event(msnh_stream_t s, msnh_event_t e)
{
    MSNH_REQUIRE(e != nullptr, "event is NULL");
    MSNH_HIP_CHECK(hipStreamWaitEvent(resolveStream(s), static_cast<hipEvent_t>(e), 0));
    return 0;
}

int msnh_hip_event_sync(msnh_event_t e)
{
    MSNH_REQUIRE(e != nullptr, "event is NULL");
    MSNH_HIP_CHECK(hipEventSynchronize(static_cast<hipEvent_t>(e)));
    return 0;
}

int msnh_hip_event_elapsed_ms(msnh_event_t start, msnh_event_t stop, float *ms)
{
    MSNH_REQUIRE(start && stop && ms, "event_elapsed: NULL argument");
    MSNH_HIP_CHECK(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
    return 0;
}

int msnh_hip_graph_begin(msnh_stream_t s)
{
    MSNH_HIP_CHECK(hipStreamBeginCapture(resolveStream(s), hipStreamCaptureModeThreadLocal));
    return 0;
}

int msnh_hip_graph_end(msnh_stream_t s, msnh_graph_t *g)
{
    MSNH_REQUIRE(g != nullptr, "graph pointer is NULL");
    hipGraph_t graph = nullptr;
    MSNH_HIP_CHECK(hipStreamEndCapture(resolveStream(s), &graph));
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess)
    {
        setError("hipGraphInstantiate failed: %s", hipGetErrorString(e));
        return 1;
    }
    *g = exec;
    return 0;
}

int msnh_hip_graph_launch(msnh_graph_t g, msnh_stream_t s)
{
    MSNH_REQUIRE(g != nullptr, "graph is NULL");
    MSNH_HIP_CHECK(hipGraphLaunch(static_cast<hipGraphExec_t>(g), resolveStream(s)));
    return 0;
}

int msnh_hip_graph_destroy(msnh_graph_t g)
{
    if (g) MSNH_HIP_CHECK(hipGraphExecDestroy(static_cast<hipGraphExec_t>(g)));
    return 0;
}

}
