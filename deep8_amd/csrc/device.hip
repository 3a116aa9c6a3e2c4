// Device plumbing of the C ABI: what Deep8's GPUDevice / GPUMemoryAllocator obtain from the CUDA
// runtime (deep8/src/model/GPUDevice.cu:10-12, deep8/src/model/GPUMemoryAllocator.cu:17-56),
// expressed on HIP.
#include "common.h"

namespace d8 {

char *error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code ? code : D8_ERR_ARGUMENT;
}

int cu_count() {
    static int cached = 0;
    if (!cached) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
            cached = prop.multiProcessorCount;
        if (cached <= 0) cached = 256;
    }
    return cached;
}

template <typename T>
__global__ void fill_kernel(T *p, T v, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}

}  // namespace d8

using namespace d8;

extern "C" {

const char *d8_last_error(void) { return error_buffer(); }

int d8_device_count(int *count) {
    D8_REQUIRE(count, "count is null");
    D8_HIP(hipGetDeviceCount(count));
    return 0;
}

int d8_device_init(int device_id) {
    int n = 0;
    D8_HIP(hipGetDeviceCount(&n));
    D8_REQUIRE(device_id >= 0 && device_id < n, "device %d out of range (%d visible)", device_id, n);
    D8_HIP(hipSetDevice(device_id));
    hipDeviceProp_t prop;
    D8_HIP(hipGetDeviceProperties(&prop, device_id));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(D8_ERR_ARCH, "device %d is %s; this library holds gfx950 code only", device_id, prop.gcnArchName);
    return static_scratch_setup();  // this device's address of the static scratch array
}

int d8_device_info(int *cus, int *clock_khz, size_t *hbm_bytes, char *name, int name_len) {
    int dev = 0;
    D8_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    D8_HIP(hipGetDeviceProperties(&prop, dev));
    if (cus) *cus = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    if (hbm_bytes) *hbm_bytes = prop.totalGlobalMem;
    if (name && name_len > 0) snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
    return 0;
}

int d8_mem_info(size_t *free_bytes, size_t *total_bytes) {
    size_t f = 0, t = 0;
    D8_HIP(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return 0;
}

int d8_malloc(void **ptr, size_t bytes) {
    D8_REQUIRE(ptr, "ptr is null");
    D8_HIP(hipMalloc(ptr, bytes));
    return 0;
}

int d8_free(void *ptr) {
    D8_HIP(hipFree(ptr));
    return 0;
}

int d8_host_malloc(void **ptr, size_t bytes) {
    D8_REQUIRE(ptr, "ptr is null");
    D8_HIP(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
    return 0;
}

int d8_host_free(void *ptr) {
    D8_HIP(hipHostFree(ptr));
    return 0;
}

// A fill kernel rather than hipMemsetAsync, so that callers may record it into a HIP graph.
__global__ void fill_bytes_kernel(unsigned char *p, unsigned char v, size_t n, size_t head) {
    size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t nthreads = (size_t)gridDim.x * blockDim.x;
    size_t body = (n - head) / 16;
    unsigned w = v * 0x01010101u;
    uint4 vv = make_uint4(w, w, w, w);
    uint4 *pb = (uint4 *)(p + head);
    for (size_t i = tid; i < body; i += nthreads) pb[i] = vv;
    size_t tail0 = head + body * 16;
    if (tid < head) p[tid] = v;
    if (tid < n - tail0) p[tail0 + tid] = v;
}

int d8_memset(void *ptr, int value, size_t bytes, void *stream) {
    if (!bytes) return 0;
    D8_REQUIRE(ptr, "ptr is null");
    size_t head = (16 - ((size_t)ptr & 15)) & 15;
    if (head > bytes) head = bytes;
    size_t body = (bytes - head) / 16;
    int blocks = (int)((body + 255) / 256);
    if (blocks < 1) blocks = 1;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(fill_bytes_kernel, dim3(blocks), dim3(256), 0, as_stream(stream),
                       (unsigned char *)ptr, (unsigned char)value, bytes, head);
    D8_LAUNCH_CHECK();
    return 0;
}

int d8_fill(int dtype, void *ptr, size_t n, float scalar, void *stream) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32 && dtype != D8_FLOAT64)
        return fail(D8_ERR_DTYPE, "d8_fill: element type %d is not supported", dtype);
    if (!n) return 0;
    D8_REQUIRE(ptr, "d8_fill: ptr is null");
    if (scalar == 0.f) return d8_memset(ptr, 0, n * dtype_bytes(dtype), stream);
    int blocks = (int)((n + 255) / 256);
    if (blocks > 8192) blocks = 8192;
    if (dtype == D8_FLOAT64)
        hipLaunchKernelGGL((fill_kernel<double>), dim3(blocks), dim3(256), 0, as_stream(stream), (double *)ptr, (double)scalar, n);
    else if (dtype == D8_FLOAT32)
        hipLaunchKernelGGL((fill_kernel<float>), dim3(blocks), dim3(256), 0, as_stream(stream), (float *)ptr, scalar, n);
    else
        hipLaunchKernelGGL((fill_kernel<f16>), dim3(blocks), dim3(256), 0, as_stream(stream), (f16 *)ptr, (f16)scalar, n);
    D8_LAUNCH_CHECK();
    return 0;
}

int d8_memcpy_h2d(void *dst, const void *src, size_t bytes) {
    if (!bytes) return 0;
    D8_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return 0;
}

int d8_memcpy_d2h(void *dst, const void *src, size_t bytes) {
    if (!bytes) return 0;
    D8_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return 0;
}

int d8_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream) {
    if (!bytes) return 0;
    D8_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return 0;
}

int d8_stream_create(void **stream) {
    D8_REQUIRE(stream, "stream is null");
    hipStream_t s;
    D8_HIP(hipStreamCreate(&s));
    *stream = (void *)s;
    return 0;
}

int d8_stream_destroy(void *stream) {
    D8_HIP(hipStreamDestroy(as_stream(stream)));
    return 0;
}

int d8_stream_sync(void *stream) {
    D8_HIP(hipStreamSynchronize(as_stream(stream)));
    return 0;
}

int d8_event_create(void **event) {
    D8_REQUIRE(event, "event is null");
    hipEvent_t e;
    D8_HIP(hipEventCreate(&e));
    *event = (void *)e;
    return 0;
}

int d8_event_destroy(void *event) {
    D8_HIP(hipEventDestroy((hipEvent_t)event));
    return 0;
}

int d8_event_record(void *event, void *stream) {
    D8_HIP(hipEventRecord((hipEvent_t)event, as_stream(stream)));
    return 0;
}

int d8_graph_begin(void *stream) {
    D8_REQUIRE(stream, "d8_graph_begin: a graph is captured on a stream of its own, not on the default stream");
    D8_HIP(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal));
    return 0;
}

int d8_graph_end(void *stream, void **graph) {
    D8_REQUIRE(stream && graph, "d8_graph_end: null argument");
    hipGraph_t captured = nullptr;
    D8_HIP(hipStreamEndCapture(as_stream(stream), &captured));
    hipGraphExec_t exec = nullptr;
    const hipError_t e = hipGraphInstantiate(&exec, captured, nullptr, nullptr, 0);
    (void)hipGraphDestroy(captured);
    if (e != hipSuccess) return fail((int)e, "hipGraphInstantiate: %s", hipGetErrorString(e));
    *graph = (void *)exec;
    return 0;
}

int d8_graph_launch(void *graph, void *stream) {
    D8_REQUIRE(graph, "d8_graph_launch: graph is null");
    D8_HIP(hipGraphLaunch((hipGraphExec_t)graph, as_stream(stream)));
    return 0;
}

int d8_graph_destroy(void *graph) {
    if (graph) D8_HIP(hipGraphExecDestroy((hipGraphExec_t)graph));
    return 0;
}

int d8_event_elapsed_ms(void *start, void *stop, float *ms) {
    D8_REQUIRE(ms, "ms is null");
    D8_HIP(hipEventSynchronize((hipEvent_t)stop));
    D8_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return 0;
}

}  // extern "C"
