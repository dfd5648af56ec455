// Shared host-side helpers of the C ABI implementation: error reporting, tensor
// descriptor checks, launch helpers.  Not part of the public interface.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "chx_hip.h"

namespace chx {

void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

#define CHX_FAIL(code, ...)          \
    do {                             \
        ::chx::set_error(__VA_ARGS__); \
        return (code);               \
    } while (0)

#define CHX_REQUIRE(cond, ...)                          \
    do {                                                \
        if (!(cond)) CHX_FAIL(CHX_HIP_EINVAL, __VA_ARGS__); \
    } while (0)

#define CHX_HIP_CALL(expr)                                                                              \
    do {                                                                                                \
        hipError_t e_ = (expr);                                                                         \
        if (e_ != hipSuccess)                                                                           \
            CHX_FAIL(CHX_HIP_ERUNTIME, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
    } while (0)

#define CHX_PROPAGATE(expr)           \
    do {                              \
        int rc_ = (expr);             \
        if (rc_ != CHX_HIP_OK) return rc_; \
    } while (0)

inline int dtype_size(int32_t dt) {
    switch (dt) {
        case CHX_HIP_BOOL:
        case CHX_HIP_INT8:
        case CHX_HIP_UINT8:
            return 1;
        case CHX_HIP_INT16:
        case CHX_HIP_FLOAT16:
            return 2;
        case CHX_HIP_INT32:
        case CHX_HIP_FLOAT32:
            return 4;
        case CHX_HIP_INT64:
        case CHX_HIP_FLOAT64:
            return 8;
        default:
            return 0;
    }
}

inline const char* dtype_name(int32_t dt) {
    switch (dt) {
        case CHX_HIP_BOOL: return "bool";
        case CHX_HIP_INT8: return "int8";
        case CHX_HIP_INT16: return "int16";
        case CHX_HIP_INT32: return "int32";
        case CHX_HIP_INT64: return "int64";
        case CHX_HIP_UINT8: return "uint8";
        case CHX_HIP_FLOAT16: return "float16";
        case CHX_HIP_FLOAT32: return "float32";
        case CHX_HIP_FLOAT64: return "float64";
        default: return "unknown";
    }
}

inline bool is_q8(int32_t dt) {
    return dt == CHX_HIP_INT8 || dt == CHX_HIP_UINT8;
}

inline int64_t numel(const chx_hip_tensor& t) {
    int64_t n = 1;
    for (int i = 0; i < t.ndim; ++i) n *= t.shape[i];
    return n;
}

inline bool same_shape(const chx_hip_tensor& a, const chx_hip_tensor& b) {
    if (a.ndim != b.ndim) return false;
    for (int i = 0; i < a.ndim; ++i)
        if (a.shape[i] != b.shape[i]) return false;
    return true;
}

// C-contiguous (row-major, no gaps).  Axes of extent 1 may carry any stride.
inline bool is_contiguous(const chx_hip_tensor& t) {
    int64_t expect = dtype_size(t.dtype);
    for (int i = t.ndim - 1; i >= 0; --i) {
        if (t.shape[i] != 1 && t.strides[i] != expect) return false;
        expect *= t.shape[i];
    }
    return true;
}

// NCHW-shaped view of channels-last memory: strides (H*W*C', 1, W*C', C') in
// elements, where C' >= C is the allocated channel pitch.
inline bool is_channels_last(const chx_hip_tensor& t, int64_t* channel_pitch) {
    if (t.ndim != 4) return false;
    const int64_t es = dtype_size(t.dtype);
    const int64_t C = t.shape[1], H = t.shape[2], W = t.shape[3];
    if (C != 1 && t.strides[1] != es) return false;
    const int64_t pitch = (W != 1 || H != 1 || t.shape[0] != 1) ? 0 : C * es;
    int64_t p = pitch;
    if (W != 1) p = t.strides[3];
    else if (H != 1) p = t.strides[2];
    else if (t.shape[0] != 1) p = t.strides[0];
    if (p < C * es || p % es != 0) return false;
    if (W != 1 && t.strides[3] != p) return false;
    if (H != 1 && t.strides[2] != W * p) return false;
    if (t.shape[0] != 1 && t.strides[0] != H * W * p) return false;
    if (channel_pitch) *channel_pitch = p / es;
    return true;
}

// True when both tensors cover their elements densely with the same axis order,
// so an element-wise kernel may walk them as flat memory.
bool same_dense_layout(const chx_hip_tensor& a, const chx_hip_tensor& b);

int check_tensor(const chx_hip_tensor* t, const char* what);

// Which operation grouping of expf the host C library uses (faithful_math.h): the two groupings differ on
// exactly two arguments, so evaluating one of them tells.
bool host_libm_uses_fma();

inline hipStream_t as_stream(void* s) {
    return reinterpret_cast<hipStream_t>(s);
}

inline bool aligned(const void* p, size_t a) {
    return (reinterpret_cast<uintptr_t>(p) % a) == 0;
}

int launch_check(const char* kernel);

// Stream-ordered scratch memory for one call.
// device address of the scratch array of chx_hip_reduce_min_max_noalloc on the current device, looked up once (reduce_cast.hip)
int prepare_noalloc_scratch();
// whether work submitted to s is being recorded into a graph instead of executed
bool stream_is_capturing(hipStream_t s);
int scratch_alloc(void** p, size_t bytes, hipStream_t s);
void scratch_free(void* p, hipStream_t s);

struct StridedDesc {
    int32_t ndim;
    int64_t shape[CHX_HIP_MAX_NDIM];
    int64_t strides[CHX_HIP_MAX_NDIM];  // bytes
};

}  // namespace chx
