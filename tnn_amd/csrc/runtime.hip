// Device, memory, stream and event entry points of the C ABI.
#include <stdarg.h>
#include <string.h>

#include "common.h"

namespace tnn_rocm {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

}  // namespace tnn_rocm

using namespace tnn_rocm;

extern "C" {

const char *tnn_rocm_last_error(void) { return g_err; }

int tnn_rocm_device_count(int *count) {
    TR_REQUIRE(count, TNN_ROCM_EINVAL, "device_count: null output");
    int n        = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        n = 0;
    }
    *count = n;
    return 0;
}

int tnn_rocm_set_device(int device_id) {
    TR_CHECK_HIP(hipSetDevice(device_id));
    return 0;
}

int tnn_rocm_device_name(int device_id, char *buf, size_t buf_len) {
    TR_REQUIRE(buf && buf_len > 0, TNN_ROCM_EINVAL, "device_name: null buffer");
    hipDeviceProp_t prop;
    TR_CHECK_HIP(hipGetDeviceProperties(&prop, device_id));
    snprintf(buf, buf_len, "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
    return 0;
}

int tnn_rocm_malloc(void **ptr, size_t bytes) {
    TR_REQUIRE(ptr, TNN_ROCM_EINVAL, "malloc: null output");
    *ptr = nullptr;
    if (bytes == 0)
        return 0;
    TR_CHECK_HIP(hipMalloc(ptr, bytes));
    return 0;
}

int tnn_rocm_free(void *ptr) {
    if (ptr)
        TR_CHECK_HIP(hipFree(ptr));
    return 0;
}

int tnn_rocm_malloc_host(void **host_ptr, size_t bytes) {
    TR_REQUIRE(host_ptr, TNN_ROCM_EINVAL, "malloc_host: null output");
    *host_ptr = nullptr;
    if (bytes == 0)
        return 0;
    TR_CHECK_HIP(hipHostMalloc(host_ptr, bytes, hipHostMallocMapped));
    memset(*host_ptr, 0, bytes);
    return 0;
}

int tnn_rocm_free_host(void *host_ptr) {
    if (host_ptr)
        TR_CHECK_HIP(hipHostFree(host_ptr));
    return 0;
}

int tnn_rocm_memset(void *ptr, int value, size_t bytes, void *stream) {
    if (bytes == 0)
        return 0;
    TR_REQUIRE(ptr, TNN_ROCM_EINVAL, "memset: null pointer");
    TR_CHECK_HIP(hipMemsetAsync(ptr, value, bytes, (hipStream_t)stream));
    return 0;
}

// Host buffers handed over by the engine are pageable, so both host copies block until the
// data has moved (the contract of CopyToDevice / CopyFromDevice).
int tnn_rocm_memcpy_h2d(void *dst, const void *host_src, size_t bytes, void *stream) {
    if (bytes == 0)
        return 0;
    TR_REQUIRE(dst && host_src, TNN_ROCM_EINVAL, "memcpy_h2d: null pointer");
    TR_CHECK_HIP(hipMemcpyAsync(dst, host_src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
    TR_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int tnn_rocm_memcpy_d2h(void *host_dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0)
        return 0;
    TR_REQUIRE(host_dst && src, TNN_ROCM_EINVAL, "memcpy_d2h: null pointer");
    TR_CHECK_HIP(hipMemcpyAsync(host_dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
    TR_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int tnn_rocm_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0)
        return 0;
    TR_REQUIRE(dst && src, TNN_ROCM_EINVAL, "memcpy_d2d: null pointer");
    TR_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
    return 0;
}

int tnn_rocm_stream_create(void **stream) {
    TR_REQUIRE(stream, TNN_ROCM_EINVAL, "stream_create: null output");
    hipStream_t s;
    TR_CHECK_HIP(hipStreamCreate(&s));  // default priority only
    *stream = (void *)s;
    return 0;
}

int tnn_rocm_stream_destroy(void *stream) {
    if (stream)
        TR_CHECK_HIP(hipStreamDestroy((hipStream_t)stream));
    return 0;
}

int tnn_rocm_stream_sync(void *stream) {
    TR_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int tnn_rocm_graph_begin_capture(void *stream) {
    TR_REQUIRE(stream, TNN_ROCM_EINVAL, "graph capture needs a non-default stream");
    TR_CHECK_HIP(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
    return 0;
}

int tnn_rocm_graph_end_capture(void *stream, void **graph_exec) {
    TR_REQUIRE(stream && graph_exec, TNN_ROCM_EINVAL, "graph_end_capture: null argument");
    *graph_exec     = nullptr;
    hipGraph_t graph = nullptr;
    TR_CHECK_HIP(hipStreamEndCapture((hipStream_t)stream, &graph));
    hipGraphExec_t exec = nullptr;
    hipError_t e        = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) {
        set_error("hipGraphInstantiate failed: %s", hipGetErrorString(e));
        return (int)e;
    }
    *graph_exec = (void *)exec;
    return 0;
}

int tnn_rocm_graph_launch(void *graph_exec, void *stream) {
    TR_REQUIRE(graph_exec, TNN_ROCM_EINVAL, "graph_launch: null graph");
    TR_CHECK_HIP(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream));
    return 0;
}

int tnn_rocm_graph_destroy(void *graph_exec) {
    if (graph_exec)
        TR_CHECK_HIP(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
    return 0;
}

int tnn_rocm_event_create(void **event) {
    TR_REQUIRE(event, TNN_ROCM_EINVAL, "event_create: null output");
    hipEvent_t e;
    TR_CHECK_HIP(hipEventCreate(&e));
    *event = (void *)e;
    return 0;
}

int tnn_rocm_event_destroy(void *event) {
    if (event)
        TR_CHECK_HIP(hipEventDestroy((hipEvent_t)event));
    return 0;
}

int tnn_rocm_event_record(void *event, void *stream) {
    TR_REQUIRE(event, TNN_ROCM_EINVAL, "event_record: null event");
    TR_CHECK_HIP(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
    return 0;
}

// every translation unit holds its own copy of the switch (common.h); they are set together (weak: a stand-alone
// program may link this file with only some of the kernels)
__attribute__((weak)) int gemm_set_store_through(int on);
__attribute__((weak)) int attention_set_store_through(int on);
__attribute__((weak)) int rowwise_set_store_through(int on);
__attribute__((visibility("default"))) int tnn_rocm_debug_set_store_through(int on) {
    on = on ? 1 : 0;
    TR_CHECK_HIP(hipDeviceSynchronize());
    if (gemm_set_store_through)
        TR_CHECK_HIP((hipError_t)gemm_set_store_through(on));
    if (attention_set_store_through)
        TR_CHECK_HIP((hipError_t)attention_set_store_through(on));
    if (rowwise_set_store_through)
        TR_CHECK_HIP((hipError_t)rowwise_set_store_through(on));
    return 0;
}

int tnn_rocm_event_elapsed_ms(void *start, void *stop, float *ms) {
    TR_REQUIRE(start && stop && ms, TNN_ROCM_EINVAL, "event_elapsed_ms: null argument");
    TR_CHECK_HIP(hipEventSynchronize((hipEvent_t)stop));
    TR_CHECK_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return 0;
}

}  // extern "C"
