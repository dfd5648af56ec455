// Library state, error reporting and the thin device-memory helpers of the C ABI.
#include <cmath>
#include <cstring>

#include "chx_internal.h"

namespace chx {

static thread_local std::string g_last_error;

void set_error(const char* fmt, ...) {
    char buf[2048];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
}

bool host_libm_uses_fma() {
    static const bool v = [] {
        volatile float x = 0.0f;
        const uint32_t bits = 0x4202422fu;
        float xf;
        memcpy(&xf, &bits, 4);
        x = xf;
        const float e = expf(x);
        uint32_t eb;
        memcpy(&eb, &e, 4);
        return eb == 0x56fc9f1cu;  // 0x1.f93e38p+46: the fused-reduction result
    }();
    return v;
}

int check_tensor(const chx_hip_tensor* t, const char* what) {
    CHX_REQUIRE(t != nullptr, "%s: null tensor descriptor", what);
    CHX_REQUIRE(t->ndim >= 0 && t->ndim <= CHX_HIP_MAX_NDIM, "%s: ndim %d out of range", what, t->ndim);
    CHX_REQUIRE(dtype_size(t->dtype) != 0, "%s: unknown dtype code %d", what, t->dtype);
    int64_t n = 1;
    for (int i = 0; i < t->ndim; ++i) {
        CHX_REQUIRE(t->shape[i] >= 0, "%s: negative extent on axis %d", what, i);
        n *= t->shape[i];
    }
    CHX_REQUIRE(n == 0 || t->data != nullptr, "%s: null data pointer for %lld elements", what, (long long)n);
    return CHX_HIP_OK;
}

bool same_dense_layout(const chx_hip_tensor& a, const chx_hip_tensor& b) {
    if (!same_shape(a, b)) return false;
    if (is_contiguous(a) && is_contiguous(b)) return true;
    const int64_t ea = dtype_size(a.dtype), eb = dtype_size(b.dtype);
    // identical stride pattern in elements, and dense: sort axes by stride and check packing
    int order[CHX_HIP_MAX_NDIM];
    int nd = 0;
    for (int i = 0; i < a.ndim; ++i) {
        if (a.shape[i] == 1) continue;
        if (a.strides[i] % ea || b.strides[i] % eb) return false;
        if (a.strides[i] / ea != b.strides[i] / eb) return false;
        order[nd++] = i;
    }
    for (int i = 0; i < nd; ++i)
        for (int j = i + 1; j < nd; ++j)
            if (a.strides[order[j]] < a.strides[order[i]]) {
                int t = order[i];
                order[i] = order[j];
                order[j] = t;
            }
    int64_t expect = ea;
    for (int i = 0; i < nd; ++i) {
        if (a.strides[order[i]] != expect) return false;
        expect *= a.shape[order[i]];
    }
    return true;
}

int launch_check(const char* kernel) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) CHX_FAIL(CHX_HIP_ERUNTIME, "launch of %s failed: %s", kernel, hipGetErrorString(e));
    return CHX_HIP_OK;
}

bool stream_is_capturing(hipStream_t s) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &st) != hipSuccess) {
        (void)hipGetLastError();
        return true;  // when in doubt, behave as if it were
    }
    return st != hipStreamCaptureStatusNone;
}

int scratch_alloc(void** p, size_t bytes, hipStream_t s) {
    *p = nullptr;
    if (bytes == 0) return CHX_HIP_OK;
    // A stream-ordered allocation on a capturing stream would become a memory node of the graph, whose replays then
    // run kernels on addresses that are not mapped (a device fault).  Callers that may be captured keep their scratch
    // between calls (plans) or take a path without scratch.
    if (stream_is_capturing(s)) CHX_FAIL(CHX_HIP_EUNSUPPORTED, "scratch memory cannot be allocated while the stream is being captured into a graph");
    CHX_HIP_CALL(hipMallocAsync(p, bytes, s));
    return CHX_HIP_OK;
}

void scratch_free(void* p, hipStream_t s) {
    if (p) (void)hipFreeAsync(p, s);
}

}  // namespace chx

using namespace chx;

struct chx_hip_graph {
    hipGraphExec_t exec;
};

extern "C" {

const char* chx_hip_last_error(void) {
    return g_last_error.c_str();
}

const char* chx_hip_version(void) {
    return "chx_hip 0.1 (gfx950)";
}

int chx_hip_init(int device) {
    int count = 0;
    CHX_HIP_CALL(hipGetDeviceCount(&count));
    CHX_REQUIRE(device >= 0 && device < count, "device %d out of range (%d visible)", device, count);
    CHX_HIP_CALL(hipSetDevice(device));
    hipDeviceProp_t prop;
    CHX_HIP_CALL(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        CHX_FAIL(CHX_HIP_EUNSUPPORTED, "device %d is %s; this library holds gfx950 code only", device, prop.gcnArchName);
    return prepare_noalloc_scratch();
}

int chx_hip_get_device_props(chx_hip_device_props* out) {
    CHX_REQUIRE(out != nullptr, "null output");
    int dev = 0;
    CHX_HIP_CALL(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    CHX_HIP_CALL(hipGetDeviceProperties(&prop, dev));
    memset(out, 0, sizeof(*out));
    out->compute_units = prop.multiProcessorCount;
    out->clock_khz = prop.clockRate;
    out->memory_clock_khz = prop.memoryClockRate;
    out->memory_bus_bits = prop.memoryBusWidth;
    out->total_memory = (int64_t)prop.totalGlobalMem;
    strncpy(out->arch, prop.gcnArchName, sizeof(out->arch) - 1);
    strncpy(out->name, prop.name, sizeof(out->name) - 1);
    return CHX_HIP_OK;
}

int chx_hip_malloc(void** ptr, size_t bytes) {
    CHX_REQUIRE(ptr != nullptr, "null output pointer");
    *ptr = nullptr;
    if (bytes == 0) return CHX_HIP_OK;
    CHX_HIP_CALL(hipMalloc(ptr, bytes));
    return CHX_HIP_OK;
}

int chx_hip_free(void* ptr) {
    if (ptr) CHX_HIP_CALL(hipFree(ptr));
    return CHX_HIP_OK;
}

int chx_hip_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream) {
    if (bytes == 0) return CHX_HIP_OK;
    CHX_REQUIRE(dst && src, "null pointer");
    CHX_HIP_CALL(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    CHX_HIP_CALL(hipStreamSynchronize(as_stream(stream)));
    return CHX_HIP_OK;
}

int chx_hip_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream) {
    if (bytes == 0) return CHX_HIP_OK;
    CHX_REQUIRE(dst && src, "null pointer");
    CHX_HIP_CALL(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    CHX_HIP_CALL(hipStreamSynchronize(as_stream(stream)));
    return CHX_HIP_OK;
}

int chx_hip_memset(void* dst, int value, size_t bytes, void* stream) {
    if (bytes == 0) return CHX_HIP_OK;
    CHX_REQUIRE(dst != nullptr, "null pointer");
    CHX_HIP_CALL(hipMemsetAsync(dst, value, bytes, as_stream(stream)));
    return CHX_HIP_OK;
}

int chx_hip_stream_synchronize(void* stream) {
    CHX_HIP_CALL(hipStreamSynchronize(as_stream(stream)));
    return CHX_HIP_OK;
}

int chx_hip_stream_create(void** stream) {
    CHX_REQUIRE(stream != nullptr, "null output");
    hipStream_t s = nullptr;
    CHX_HIP_CALL(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = s;
    return CHX_HIP_OK;
}

int chx_hip_stream_destroy(void* stream) {
    if (stream) CHX_HIP_CALL(hipStreamDestroy(as_stream(stream)));
    return CHX_HIP_OK;
}

int chx_hip_capture_begin(void* stream) {
    CHX_REQUIRE(stream != nullptr, "the null stream cannot be captured");
    // thread-local mode: calls of other threads (another program running eagerly) are not affected
    CHX_HIP_CALL(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal));
    return CHX_HIP_OK;
}

int chx_hip_capture_end(void* stream, chx_hip_graph** graph) {
    CHX_REQUIRE(stream != nullptr && graph != nullptr, "null argument");
    *graph = nullptr;
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(as_stream(stream), &g);
    if (e != hipSuccess || g == nullptr) {
        (void)hipGetLastError();
        if (g) (void)hipGraphDestroy(g);
        CHX_FAIL(CHX_HIP_ERUNTIME, "the capture did not give a graph: %s", hipGetErrorString(e));
    }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess) CHX_FAIL(CHX_HIP_ERUNTIME, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
    chx_hip_graph* out = new chx_hip_graph();
    out->exec = exec;
    *graph = out;
    return CHX_HIP_OK;
}

int chx_hip_stream_is_capturing(void* stream) {
    if (!stream) return 0;
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(as_stream(stream), &st) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return st != hipStreamCaptureStatusNone ? 1 : 0;
}

int chx_hip_graph_launch(const chx_hip_graph* graph, void* stream) {
    CHX_REQUIRE(graph != nullptr, "null graph");
    CHX_HIP_CALL(hipGraphLaunch(graph->exec, as_stream(stream)));
    return CHX_HIP_OK;
}

void chx_hip_graph_destroy(chx_hip_graph* graph) {
    if (!graph) return;
    (void)hipGraphExecDestroy(graph->exec);
    delete graph;
}

}  // extern "C"
