// Runtime half of the C-ABI: device selection, memory, streams, events and
// graph capture.  The host layer reaches the HIP runtime through these only.
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "common.hpp"

static thread_local char g_err[512] = "";

void llm_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
}

__global__ void fill_zero_kernel(uint32_t *p, size_t n_words) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n_words; i += stride) p[i] = 0u;
}

int gemm_init_workspace(); // gemm.hip: split-K partial-sum buffer of the default stream
void gemm_release_workspace(hipStream_t s); // gemm.hip: a stream's split-K buffer
extern "C" int attn_decode_static_setup(int device); // attn_decode.hip: address of its built-in scratch

extern "C" {

const char *llm_last_error(void) { return g_err; }

int llm_device_count(int *count) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        n = 0;
    }
    *count = n;
    return LLM_OK;
}

int llm_init(int device) {
    int n = 0;
    llm_device_count(&n);
    if (n <= 0) {
        llm_set_error("no HIP device is visible");
        return LLM_ERR_NO_DEVICE;
    }
    LLM_REQUIRE(device >= 0 && device < n, "device %d out of range (%d visible)", device, n);
    LLM_HIP_CHECK(hipSetDevice(device));
    hipDeviceProp_t prop;
    LLM_HIP_CHECK(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        llm_set_error("device %d is %s; this library holds gfx950 code only", device, prop.gcnArchName);
        return LLM_ERR_NO_DEVICE;
    }
    int rc = attn_decode_static_setup(device);
    if (rc != LLM_OK) return rc;
    return gemm_init_workspace();
}

int llm_device_name(char *buf, size_t n) {
    int dev = 0;
    LLM_HIP_CHECK(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    LLM_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
    snprintf(buf, n, "%s", prop.gcnArchName);
    return LLM_OK;
}

int llm_device_cu_count(int *n) {
    int dev = 0;
    LLM_HIP_CHECK(hipGetDevice(&dev));
    LLM_HIP_CHECK(hipDeviceGetAttribute(n, hipDeviceAttributeMultiprocessorCount, dev));
    return LLM_OK;
}

int llm_malloc(void **ptr, size_t bytes) {
    *ptr = nullptr;
    LLM_HIP_CHECK(hipMalloc(ptr, bytes ? bytes : 1));
    return LLM_OK;
}

int llm_free(void *ptr) {
    if (ptr) LLM_HIP_CHECK(hipFree(ptr));
    return LLM_OK;
}

int llm_malloc_host(void **ptr, size_t bytes) {
    *ptr = nullptr;
    LLM_HIP_CHECK(hipHostMalloc(ptr, bytes ? bytes : 1, hipHostMallocDefault));
    return LLM_OK;
}

int llm_free_host(void *ptr) {
    if (ptr) LLM_HIP_CHECK(hipHostFree(ptr));
    return LLM_OK;
}

static int copy(void *dst, const void *src, size_t bytes, hipMemcpyKind kind, llm_stream_t stream) {
    if (bytes == 0) return LLM_OK;
    if (stream) {
        LLM_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, kind, (hipStream_t)stream));
    } else {
        LLM_HIP_CHECK(hipMemcpy(dst, src, bytes, kind));
    }
    return LLM_OK;
}

int llm_memcpy_h2d(void *dst, const void *src, size_t bytes, llm_stream_t s) {
    return copy(dst, src, bytes, hipMemcpyHostToDevice, s);
}
int llm_memcpy_d2h(void *dst, const void *src, size_t bytes, llm_stream_t s) {
    return copy(dst, src, bytes, hipMemcpyDeviceToHost, s);
}
int llm_memcpy_d2d(void *dst, const void *src, size_t bytes, llm_stream_t s) {
    return copy(dst, src, bytes, hipMemcpyDeviceToDevice, s);
}

int llm_mem_info(size_t *free_bytes, size_t *total_bytes) {
    size_t f = 0, t = 0;
    LLM_HIP_CHECK(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return LLM_OK;
}

int llm_fill_zero(void *dst, size_t bytes, llm_stream_t stream) {
    LLM_REQUIRE((reinterpret_cast<uintptr_t>(dst) & 3u) == 0 && bytes % 4 == 0,
                "llm_fill_zero needs 4-byte alignment and size");
    if (bytes == 0) return LLM_OK;
    size_t words = bytes / 4;
    size_t blocks = (words + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    fill_zero_kernel<<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>((uint32_t *)dst, words);
    LLM_LAUNCH_CHECK("fill_zero_kernel");
    return LLM_OK;
}

int llm_stream_create(llm_stream_t *stream) {
    hipStream_t s;
    LLM_HIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = (llm_stream_t)s;
    return LLM_OK;
}

int llm_stream_destroy(llm_stream_t stream) {
    if (stream) {
        LLM_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
        gemm_release_workspace((hipStream_t)stream);
        LLM_HIP_CHECK(hipStreamDestroy((hipStream_t)stream));
    }
    return LLM_OK;
}

int llm_stream_sync(llm_stream_t stream) {
    LLM_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return LLM_OK;
}

int llm_device_sync(void) {
    LLM_HIP_CHECK(hipDeviceSynchronize());
    return LLM_OK;
}

int llm_event_create(llm_event_t *ev) {
    hipEvent_t e;
    LLM_HIP_CHECK(hipEventCreate(&e));
    *ev = (llm_event_t)e;
    return LLM_OK;
}

int llm_event_destroy(llm_event_t ev) {
    if (ev) LLM_HIP_CHECK(hipEventDestroy((hipEvent_t)ev));
    return LLM_OK;
}

int llm_event_record(llm_event_t ev, llm_stream_t stream) {
    LLM_HIP_CHECK(hipEventRecord((hipEvent_t)ev, (hipStream_t)stream));
    return LLM_OK;
}

int llm_event_sync(llm_event_t ev) {
    LLM_HIP_CHECK(hipEventSynchronize((hipEvent_t)ev));
    return LLM_OK;
}

int llm_event_elapsed_ms(llm_event_t start, llm_event_t stop, float *ms) {
    LLM_HIP_CHECK(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return LLM_OK;
}

int llm_graph_capture_begin(llm_stream_t stream) {
    LLM_REQUIRE(stream != nullptr, "graph capture needs an explicit stream");
    LLM_HIP_CHECK(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
    return LLM_OK;
}

int llm_graph_capture_end(llm_stream_t stream, llm_graph_t *graph_exec) {
    hipGraph_t g = nullptr;
    LLM_HIP_CHECK(hipStreamEndCapture((hipStream_t)stream, &g));
    hipGraphExec_t ex = nullptr;
    hipError_t e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess) {
        llm_set_error("hipGraphInstantiate: %s", hipGetErrorString(e));
        return LLM_ERR_HIP;
    }
    *graph_exec = (llm_graph_t)ex;
    return LLM_OK;
}

int llm_graph_launch(llm_graph_t graph_exec, llm_stream_t stream) {
    LLM_HIP_CHECK(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream));
    return LLM_OK;
}

int llm_graph_destroy(llm_graph_t graph_exec) {
    if (graph_exec) LLM_HIP_CHECK(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
    return LLM_OK;
}

} // extern "C"
