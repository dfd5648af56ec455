// QuantizeLinear / DequantizeLinear for gfx950: one pass over HBM, 128-bit loads and
// stores, no temporaries.  Arithmetic follows quantize_array / dequantize_array of the
// reference (runtime/ops/quantize.cc:16-44) operation by operation in fp32; the file is
// compiled with -ffp-contract=off so no multiply-add is fused.
#include "chx_internal.h"
#include "quant_math.h"

namespace chx {
namespace {

constexpr int kThreads = 256;

typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

// One 128-bit load and one 32-bit store per lane and step, kUnroll steps per thread at
// a stride of one block, so that every access instruction of a wavefront covers one
// contiguous span (1 KiB in, 256 B out).
constexpr int kUnroll = 4;
// QuantizeLinear of a tensor of a few million elements (a network's input) is a launch of some 10 us, bound by how
// many wavefronts issue at once rather than by bytes in flight: one step per thread then (10.3 against 11.5 us for
// [64, 3, 224, 224]); four steps are 4 % faster on [64, 1024, 1024].
constexpr int64_t kFewVectors = int64_t(1) << 22;

template <bool kRne, int kSteps = kUnroll>
__global__ __launch_bounds__(kThreads) void quantize_flat_kernel(
        const v4f* __restrict__ x, uint32_t* __restrict__ y, int64_t n_vec, QuantParams qp) {
    const int64_t first = (int64_t)blockIdx.x * (kThreads * kSteps) + threadIdx.x;
    v4f v[kSteps];
#pragma unroll
    for (int u = 0; u < kSteps; ++u) {
        const int64_t i = first + u * kThreads;
        if (i < n_vec) v[u] = __builtin_nontemporal_load(x + i);
    }
#pragma unroll
    for (int u = 0; u < kSteps; ++u) {
        const int64_t i = first + u * kThreads;
        if (i < n_vec) {
            const uint32_t out = pack4(quantize_value<kRne>(v[u].x, qp), quantize_value<kRne>(v[u].y, qp),
                                       quantize_value<kRne>(v[u].z, qp), quantize_value<kRne>(v[u].w, qp));
            __builtin_nontemporal_store(out, y + i);
        }
    }
}

// Remainder elements and unaligned buffers: one element per thread.
template <bool kRne>
__global__ __launch_bounds__(kThreads) void quantize_scalar_kernel(
        const float* __restrict__ x, uint8_t* __restrict__ y, int64_t begin, int64_t n, QuantParams qp) {
    const int64_t i = begin + (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (i >= n) return;
    y[i] = (uint8_t)quantize_value<kRne>(x[i], qp);
}

__device__ __forceinline__ int64_t strided_offset(int64_t flat, const StridedDesc& d) {
    int64_t off = 0;
    for (int a = d.ndim - 1; a >= 0; --a) {
        const int64_t q = flat / d.shape[a];
        const int64_t r = flat - q * d.shape[a];
        off += r * d.strides[a];
        flat = q;
    }
    return off;
}

// Any strides on either side (element [i0,i1,..] of x goes to element [i0,i1,..] of y).
template <bool kRne>
__global__ __launch_bounds__(kThreads) void quantize_strided_kernel(
        const char* __restrict__ x, StridedDesc xd, char* __restrict__ y, StridedDesc yd, int64_t n, QuantParams qp) {
    const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (i >= n) return;
    const float v = *reinterpret_cast<const float*>(x + strided_offset(i, xd));
    *reinterpret_cast<uint8_t*>(y + strided_offset(i, yd)) = (uint8_t)quantize_value<kRne>(v, qp);
}

template <bool kSigned>
__device__ __forceinline__ v4f dequant4(uint32_t w, float zpf, float scale) {
    v4f r;
    r.x = dequantize_value(byte_of<kSigned>(w, 0), zpf, scale);
    r.y = dequantize_value(byte_of<kSigned>(w, 1), zpf, scale);
    r.z = dequantize_value(byte_of<kSigned>(w, 2), zpf, scale);
    r.w = dequantize_value(byte_of<kSigned>(w, 3), zpf, scale);
    return r;
}

template <bool kSigned>
__global__ __launch_bounds__(kThreads) void dequantize_flat_kernel(
        const uint32_t* __restrict__ x, v4f* __restrict__ y, int64_t n_vec, float zpf, float scale) {
    const int64_t first = (int64_t)blockIdx.x * (kThreads * kUnroll) + threadIdx.x;
    uint32_t q[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int64_t i = first + u * kThreads;
        if (i < n_vec) q[u] = __builtin_nontemporal_load(x + i);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int64_t i = first + u * kThreads;
        if (i < n_vec) __builtin_nontemporal_store(dequant4<kSigned>(q[u], zpf, scale), y + i);
    }
}

template <bool kSigned>
__global__ __launch_bounds__(kThreads) void dequantize_scalar_kernel(
        const uint8_t* __restrict__ x, float* __restrict__ y, int64_t begin, int64_t n, float zpf, float scale) {
    const int64_t i = begin + (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (i >= n) return;
    const int32_t q = kSigned ? (int32_t)(int8_t)x[i] : (int32_t)x[i];
    y[i] = dequantize_value(q, zpf, scale);
}

template <bool kSigned>
__global__ __launch_bounds__(kThreads) void dequantize_strided_kernel(
        const char* __restrict__ x, StridedDesc xd, char* __restrict__ y, StridedDesc yd, int64_t n, float zpf,
        float scale) {
    const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (i >= n) return;
    const uint8_t raw = *reinterpret_cast<const uint8_t*>(x + strided_offset(i, xd));
    const int32_t q = kSigned ? (int32_t)(int8_t)raw : (int32_t)raw;
    *reinterpret_cast<float*>(y + strided_offset(i, yd)) = dequantize_value(q, zpf, scale);
}

inline unsigned blocks_for(int64_t n) {
    return (unsigned)((n + kThreads - 1) / kThreads);
}

inline unsigned flat_blocks_for(int64_t n_vec) {
    return (unsigned)((n_vec + kThreads * kUnroll - 1) / (kThreads * kUnroll));
}

StridedDesc make_desc(const chx_hip_tensor& t) {
    StridedDesc d;
    d.ndim = t.ndim;
    for (int i = 0; i < t.ndim; ++i) {
        d.shape[i] = t.shape[i];
        d.strides[i] = t.strides[i];
    }
    return d;
}

}  // namespace
}  // namespace chx

using namespace chx;

extern "C" int chx_hip_quantize_linear(
        const chx_hip_tensor* x, float y_scale, int32_t y_zero_point, uint32_t flags, chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(x, "QuantizeLinear x"));
    CHX_PROPAGATE(check_tensor(y, "QuantizeLinear y"));
    CHX_REQUIRE(x->dtype == CHX_HIP_FLOAT32, "QuantizeLinear: x must be float32, got %s", dtype_name(x->dtype));
    CHX_REQUIRE(is_q8(y->dtype), "QuantizeLinear: y must be uint8 or int8, got %s", dtype_name(y->dtype));
    CHX_REQUIRE(same_shape(*x, *y), "QuantizeLinear: x and y shapes differ");
    const bool i8 = y->dtype == CHX_HIP_INT8;
    // CHECK_LE(min, zp) / CHECK_LE(zp, max), runtime/ops/quantize.cc:26-27
    CHX_REQUIRE(y_zero_point >= (i8 ? -128 : 0) && y_zero_point <= (i8 ? 127 : 255),
                "QuantizeLinear: zero point %d outside the range of %s", y_zero_point, dtype_name(y->dtype));
    const int64_t n = numel(*x);
    if (n == 0) return CHX_HIP_OK;
    CHX_REQUIRE(n < (int64_t(1) << 40), "QuantizeLinear: %lld elements is beyond what one launch covers", (long long)n);
    const bool rne = (flags & CHX_HIP_ROUND_ONNX_RNE) != 0;
    QuantParams qp = make_quant_params(y_scale, y_zero_point, i8);
    hipStream_t s = as_stream(stream);

    if (same_dense_layout(*x, *y)) {
        const float* xp = static_cast<const float*>(x->data);
        uint8_t* yp = static_cast<uint8_t*>(y->data);
        int64_t n_vec = 0;
        if (aligned(xp, 16) && aligned(yp, 16)) n_vec = n / 4;
        if (n_vec > 0) {
            const v4f* xv = reinterpret_cast<const v4f*>(xp);
            uint32_t* yv = reinterpret_cast<uint32_t*>(yp);
            if (n_vec <= kFewVectors) {
                if (rne) quantize_flat_kernel<true, 1><<<blocks_for(n_vec), kThreads, 0, s>>>(xv, yv, n_vec, qp);
                else quantize_flat_kernel<false, 1><<<blocks_for(n_vec), kThreads, 0, s>>>(xv, yv, n_vec, qp);
            } else {
                if (rne) quantize_flat_kernel<true><<<flat_blocks_for(n_vec), kThreads, 0, s>>>(xv, yv, n_vec, qp);
                else quantize_flat_kernel<false><<<flat_blocks_for(n_vec), kThreads, 0, s>>>(xv, yv, n_vec, qp);
            }
            CHX_PROPAGATE(launch_check("quantize_flat_kernel"));
        }
        const int64_t done = n_vec * 4;
        if (done < n) {
            if (rne)
                quantize_scalar_kernel<true><<<blocks_for(n - done), kThreads, 0, s>>>(xp, yp, done, n, qp);
            else
                quantize_scalar_kernel<false><<<blocks_for(n - done), kThreads, 0, s>>>(xp, yp, done, n, qp);
            CHX_PROPAGATE(launch_check("quantize_scalar_kernel"));
        }
        return CHX_HIP_OK;
    }
    const StridedDesc xd = make_desc(*x), yd = make_desc(*y);
    if (rne)
        quantize_strided_kernel<true><<<blocks_for(n), kThreads, 0, s>>>(
                static_cast<const char*>(x->data), xd, static_cast<char*>(y->data), yd, n, qp);
    else
        quantize_strided_kernel<false><<<blocks_for(n), kThreads, 0, s>>>(
                static_cast<const char*>(x->data), xd, static_cast<char*>(y->data), yd, n, qp);
    return launch_check("quantize_strided_kernel");
}

extern "C" int chx_hip_dequantize_linear(
        const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(x, "DequantizeLinear x"));
    CHX_PROPAGATE(check_tensor(y, "DequantizeLinear y"));
    CHX_REQUIRE(is_q8(x->dtype), "DequantizeLinear: x must be uint8 or int8, got %s", dtype_name(x->dtype));
    CHX_REQUIRE(y->dtype == CHX_HIP_FLOAT32, "DequantizeLinear: y must be float32, got %s", dtype_name(y->dtype));
    CHX_REQUIRE(same_shape(*x, *y), "DequantizeLinear: x and y shapes differ");
    const int64_t n = numel(*x);
    if (n == 0) return CHX_HIP_OK;
    CHX_REQUIRE(n < (int64_t(1) << 40), "DequantizeLinear: %lld elements is beyond what one launch covers", (long long)n);
    const bool i8 = x->dtype == CHX_HIP_INT8;
    const float zpf = (float)x_zero_point;
    hipStream_t s = as_stream(stream);

    if (same_dense_layout(*x, *y)) {
        const uint8_t* xp = static_cast<const uint8_t*>(x->data);
        float* yp = static_cast<float*>(y->data);
        int64_t n_vec = 0;
        if (aligned(xp, 16) && aligned(yp, 16)) n_vec = n / 4;
        if (n_vec > 0) {
            if (i8)
                dequantize_flat_kernel<true><<<flat_blocks_for(n_vec), kThreads, 0, s>>>(
                        reinterpret_cast<const uint32_t*>(xp), reinterpret_cast<v4f*>(yp), n_vec, zpf, x_scale);
            else
                dequantize_flat_kernel<false><<<flat_blocks_for(n_vec), kThreads, 0, s>>>(
                        reinterpret_cast<const uint32_t*>(xp), reinterpret_cast<v4f*>(yp), n_vec, zpf, x_scale);
            CHX_PROPAGATE(launch_check("dequantize_flat_kernel"));
        }
        const int64_t done = n_vec * 4;
        if (done < n) {
            if (i8)
                dequantize_scalar_kernel<true><<<blocks_for(n - done), kThreads, 0, s>>>(xp, yp, done, n, zpf, x_scale);
            else
                dequantize_scalar_kernel<false><<<blocks_for(n - done), kThreads, 0, s>>>(xp, yp, done, n, zpf, x_scale);
            CHX_PROPAGATE(launch_check("dequantize_scalar_kernel"));
        }
        return CHX_HIP_OK;
    }
    const StridedDesc xd = make_desc(*x), yd = make_desc(*y);
    if (i8)
        dequantize_strided_kernel<true><<<blocks_for(n), kThreads, 0, s>>>(
                static_cast<const char*>(x->data), xd, static_cast<char*>(y->data), yd, n, zpf, x_scale);
    else
        dequantize_strided_kernel<false><<<blocks_for(n), kThreads, 0, s>>>(
                static_cast<const char*>(x->data), xd, static_cast<char*>(y->data), yd, n, zpf, x_scale);
    return launch_check("dequantize_strided_kernel");
}
