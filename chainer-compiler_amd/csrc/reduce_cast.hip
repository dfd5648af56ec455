// The small float ops that the dynamic quantization rewrite puts around the quantized ones
// (compiler/quantize.cc:165-196,230-243 of the chainer-compiler tree): the minimum / maximum of a
// whole float32 tensor (ReduceMin / ReduceMax without axes, keepdims = 0) and element type
// conversions (Cast: int32 -> float32 for the scale-back, float32 -> uint8 / int8 for a computed
// zero point).  Both take any strides; neither is on the timed path of a statically quantized
// network.
#include <mutex>
#include <vector>

#include <type_traits>

#include "chx_internal.h"

namespace chx {
namespace {

constexpr int kThreads = 256;

// Partial results of chx_hip_reduce_min_max_noalloc: one per work-group.  Every GPU the library runs on
// holds its own copy of this array, at its own address, until the process ends.
constexpr int kNoAllocBlocks = 1024;
constexpr int64_t kNoAllocMaxElements = int64_t(1) << 30;
static __device__ __align__(256) float scratch[kNoAllocBlocks];

// Device address of `scratch` on the current device.  The name of the array is a host-side stand-in, not
// an address a kernel could use: the address is asked for once per device, with that device current.
int noalloc_scratch(float** out) {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static float* ptrs[kMaxDevices] = {};
    int dev = 0;
    CHX_HIP_CALL(hipGetDevice(&dev));
    CHX_REQUIRE(dev >= 0 && dev < kMaxDevices, "device %d: more devices than this entry point keeps scratch addresses for", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void* p = nullptr;
        CHX_HIP_CALL(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        CHX_REQUIRE(p != nullptr, "hipGetSymbolAddress gave a null address for the scratch array");
        ptrs[dev] = static_cast<float*>(p);
    }
    *out = ptrs[dev];
    return CHX_HIP_OK;
}

}  // namespace

// chx_hip_init asks for the address on its device, so that the first call of the entry point on a capturing
// stream finds it known (the lookup is no stream operation, but it need not happen inside a recording).
int prepare_noalloc_scratch() {
    float* p = nullptr;
    return noalloc_scratch(&p);
}

namespace {

__device__ __forceinline__ int64_t strided_offset(int64_t flat, const StridedDesc& d) {
    int64_t off = 0;
    for (int a = d.ndim - 1; a >= 0; --a) {
        const int64_t q = flat / d.shape[a];
        off += (flat - q * d.shape[a]) * d.strides[a];
        flat = q;
    }
    return off;
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

// min and max are exact and order-independent (a NaN anywhere gives NaN, as the comparison-based
// reduction of the CPU path does not guarantee either way; NaN inputs are outside the tested domain)
template <bool kMax>
__device__ __forceinline__ float pick(float a, float b) {
    return kMax ? (a > b ? a : b) : (a < b ? a : b);
}

template <bool kMax>
__device__ float block_reduce(float v) {
    __shared__ float red[kThreads];
    red[threadIdx.x] = v;
    __syncthreads();
    for (int s = kThreads / 2; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) red[threadIdx.x] = pick<kMax>(red[threadIdx.x], red[threadIdx.x + s]);
        __syncthreads();
    }
    return red[0];
}

template <bool kMax>
__global__ __launch_bounds__(kThreads) void reduce_partial_kernel(const char* __restrict__ x, StridedDesc xd, int64_t n, float* __restrict__ partial) {
    float v = *reinterpret_cast<const float*>(x);  // element 0 exists: n > 0
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads)
        v = pick<kMax>(v, *reinterpret_cast<const float*>(x + strided_offset(i, xd)));
    v = block_reduce<kMax>(v);
    if (threadIdx.x == 0) partial[blockIdx.x] = v;
}

template <bool kMax>
__global__ __launch_bounds__(kThreads) void reduce_final_kernel(const float* __restrict__ partial, int count, float* __restrict__ y) {
    float v = partial[0];
    for (int i = threadIdx.x; i < count; i += kThreads) v = pick<kMax>(v, partial[i]);
    v = block_reduce<kMax>(v);
    if (threadIdx.x == 0) *y = v;
}

// AsType: float -> integer truncates toward zero; integer -> float rounds to nearest
template <class From, class To>
__global__ __launch_bounds__(kThreads) void cast_kernel(const char* __restrict__ x, StridedDesc xd, char* __restrict__ y, StridedDesc yd, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (i >= n) return;
    *reinterpret_cast<To*>(y + strided_offset(i, yd)) = static_cast<To>(*reinterpret_cast<const From*>(x + strided_offset(i, xd)));
}

// NaN: the only value that differs from itself; Inf: |x| equal to the largest exponent with a zero
// mantissa (chainerx::IsNan / IsInf of the reference's scans)
template <bool kInf>
__global__ __launch_bounds__(kThreads) void count_nonfinite_kernel(const char* __restrict__ x, StridedDesc xd, int64_t n, uint32_t* __restrict__ partial) {
    __shared__ uint32_t red[kThreads];
    uint32_t found = 0;  // a block looks at fewer than 2^32 elements
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads) {
        const uint32_t bits = *reinterpret_cast<const uint32_t*>(x + strided_offset(i, xd)) & 0x7fffffffu;
        found += kInf ? (bits == 0x7f800000u) : (bits > 0x7f800000u);
    }
    red[threadIdx.x] = found;
    __syncthreads();
    for (int s = kThreads / 2; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) partial[blockIdx.x] = red[0];
}

template <class From>
int cast_from(const chx_hip_tensor& x, chx_hip_tensor& y, int64_t n, hipStream_t s) {
    const unsigned blocks = (unsigned)((n + kThreads - 1) / kThreads);
    const StridedDesc xd = make_desc(x), yd = make_desc(y);
    const char* xp = static_cast<const char*>(x.data);
    char* yp = static_cast<char*>(y.data);
    switch (y.dtype) {
        case CHX_HIP_FLOAT32: cast_kernel<From, float><<<blocks, kThreads, 0, s>>>(xp, xd, yp, yd, n); break;
        case CHX_HIP_INT32: cast_kernel<From, int32_t><<<blocks, kThreads, 0, s>>>(xp, xd, yp, yd, n); break;
        case CHX_HIP_UINT8: cast_kernel<From, uint8_t><<<blocks, kThreads, 0, s>>>(xp, xd, yp, yd, n); break;
        case CHX_HIP_INT8: cast_kernel<From, int8_t><<<blocks, kThreads, 0, s>>>(xp, xd, yp, yd, n); break;
        default: CHX_FAIL(CHX_HIP_EUNSUPPORTED, "Cast: no conversion to %s on the device", dtype_name(y.dtype));
    }
    return launch_check("cast_kernel");
}

}  // namespace
}  // namespace chx

using namespace chx;

extern "C" int chx_hip_reduce_min_max(const chx_hip_tensor* x, int32_t is_max, chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(x, "ReduceMin/ReduceMax x"));
    CHX_PROPAGATE(check_tensor(y, "ReduceMin/ReduceMax y"));
    CHX_REQUIRE(x->dtype == CHX_HIP_FLOAT32 && y->dtype == CHX_HIP_FLOAT32, "ReduceMin/ReduceMax: float32 only");
    CHX_REQUIRE(numel(*y) == 1, "ReduceMin/ReduceMax: y must hold one element (all axes reduced)");
    const int64_t n = numel(*x);
    CHX_REQUIRE(n > 0, "ReduceMin/ReduceMax of an empty tensor");
    hipStream_t s = as_stream(stream);
    int blocks = (int)((n + kThreads * 8 - 1) / (kThreads * 8));
    blocks = blocks < 1 ? 1 : blocks > 1024 ? 1024 : blocks;
    void* partial = nullptr;
    CHX_PROPAGATE(scratch_alloc(&partial, sizeof(float) * blocks, s));
    const StridedDesc xd = make_desc(*x);
    if (is_max) {
        reduce_partial_kernel<true><<<blocks, kThreads, 0, s>>>(static_cast<const char*>(x->data), xd, n, static_cast<float*>(partial));
        reduce_final_kernel<true><<<1, kThreads, 0, s>>>(static_cast<const float*>(partial), blocks, static_cast<float*>(y->data));
    } else {
        reduce_partial_kernel<false><<<blocks, kThreads, 0, s>>>(static_cast<const char*>(x->data), xd, n, static_cast<float*>(partial));
        reduce_final_kernel<false><<<1, kThreads, 0, s>>>(static_cast<const float*>(partial), blocks, static_cast<float*>(y->data));
    }
    const int rc = launch_check("reduce_min_max");
    scratch_free(partial, s);
    return rc;
}

extern "C" int chx_hip_reduce_min_max_noalloc(const chx_hip_tensor* x, int32_t is_max, chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(x, "ReduceMin/ReduceMax x"));
    CHX_PROPAGATE(check_tensor(y, "ReduceMin/ReduceMax y"));
    CHX_REQUIRE(x->dtype == CHX_HIP_FLOAT32 && y->dtype == CHX_HIP_FLOAT32, "ReduceMin/ReduceMax: float32 only");
    CHX_REQUIRE(numel(*y) == 1, "ReduceMin/ReduceMax: y must hold one element (all axes reduced)");
    const int64_t n = numel(*x);
    CHX_REQUIRE(n > 0, "ReduceMin/ReduceMax of an empty tensor");
    CHX_REQUIRE(n <= kNoAllocMaxElements,
                "ReduceMin/ReduceMax without allocation: %lld elements, at most %lld (use chx_hip_reduce_min_max for more)", (long long)n,
                (long long)kNoAllocMaxElements);
    float* partial = nullptr;
    CHX_PROPAGATE(noalloc_scratch(&partial));
    hipStream_t s = as_stream(stream);
    int blocks = (int)((n + kThreads * 8 - 1) / (kThreads * 8));
    blocks = blocks < 1 ? 1 : blocks > kNoAllocBlocks ? kNoAllocBlocks : blocks;
    const StridedDesc xd = make_desc(*x);
    // every work-group writes its own partial result and the second kernel reads exactly those: nothing of
    // what an earlier call left in the array is looked at, so nothing has to be cleared
    if (is_max) {
        reduce_partial_kernel<true><<<blocks, kThreads, 0, s>>>(static_cast<const char*>(x->data), xd, n, partial);
        reduce_final_kernel<true><<<1, kThreads, 0, s>>>(partial, blocks, static_cast<float*>(y->data));
    } else {
        reduce_partial_kernel<false><<<blocks, kThreads, 0, s>>>(static_cast<const char*>(x->data), xd, n, partial);
        reduce_final_kernel<false><<<1, kThreads, 0, s>>>(partial, blocks, static_cast<float*>(y->data));
    }
    return launch_check("reduce_min_max (no allocation)");
}

extern "C" int chx_hip_cast(const chx_hip_tensor* x, chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(x, "Cast x"));
    CHX_PROPAGATE(check_tensor(y, "Cast y"));
    CHX_REQUIRE(x->ndim == y->ndim, "Cast: x and y differ in rank");
    for (int i = 0; i < x->ndim; ++i) CHX_REQUIRE(x->shape[i] == y->shape[i], "Cast: x and y differ in shape");
    const int64_t n = numel(*x);
    if (n == 0) return CHX_HIP_OK;
    hipStream_t s = as_stream(stream);
    switch (x->dtype) {
        case CHX_HIP_FLOAT32: return cast_from<float>(*x, *y, n, s);
        case CHX_HIP_INT32: return cast_from<int32_t>(*x, *y, n, s);
        case CHX_HIP_UINT8: return cast_from<uint8_t>(*x, *y, n, s);
        case CHX_HIP_INT8: return cast_from<int8_t>(*x, *y, n, s);
        default: CHX_FAIL(CHX_HIP_EUNSUPPORTED, "Cast: no conversion from %s on the device", dtype_name(x->dtype));
    }
}

namespace chx {
namespace {

// y = x with bit 7 of every byte inverted, one lane per element, any strides on both sides
__global__ __launch_bounds__(kThreads) void flip_sign_bits_kernel(const char* __restrict__ x, StridedDesc xd, char* __restrict__ y, StridedDesc yd, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (i >= n) return;
    y[strided_offset(i, yd)] = (char)(x[strided_offset(i, xd)] ^ 0x80);
}

}  // namespace
}  // namespace chx

extern "C" int chx_hip_codes_minus_128(const chx_hip_tensor* x, chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(x, "codes minus 128: x"));
    CHX_PROPAGATE(check_tensor(y, "codes minus 128: y"));
    CHX_REQUIRE((x->dtype == CHX_HIP_UINT8 && y->dtype == CHX_HIP_INT8) || (x->dtype == CHX_HIP_INT8 && y->dtype == CHX_HIP_UINT8),
                "codes minus 128: uint8 -> int8 (code - 128) or int8 -> uint8 (code + 128), got %s -> %s", dtype_name(x->dtype), dtype_name(y->dtype));
    CHX_REQUIRE(x->ndim == y->ndim, "codes minus 128: x and y differ in rank");
    for (int i = 0; i < x->ndim; ++i) CHX_REQUIRE(x->shape[i] == y->shape[i], "codes minus 128: x and y differ in shape");
    const int64_t n = numel(*x);
    if (n == 0) return CHX_HIP_OK;
    const unsigned blocks = (unsigned)((n + kThreads - 1) / kThreads);
    flip_sign_bits_kernel<<<blocks, kThreads, 0, as_stream(stream)>>>(static_cast<const char*>(x->data), make_desc(*x), static_cast<char*>(y->data),
                                                                      make_desc(*y), n);
    return launch_check("flip_sign_bits_kernel");
}

namespace chx {
namespace {

// z = x << y or x >> y over the broadcast of x and y (strides of 0 on broadcast axes), one lane per element.
// A count of the element width or more shifts every bit out: 0, or for a negative x shifted right the sign (-1), as
// numpy defines it (C leaves it undefined); a right shift of a signed type is arithmetic.
template <typename T, bool kLeft>
__global__ __launch_bounds__(kThreads) void bit_shift_kernel(
        const char* __restrict__ x, StridedDesc xd, const char* __restrict__ y, StridedDesc yd, char* __restrict__ z, StridedDesc zd, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (i >= n) return;
    typedef typename std::make_unsigned<T>::type U;
    const T a = *reinterpret_cast<const T*>(x + strided_offset(i, xd));
    const T c = *reinterpret_cast<const T*>(y + strided_offset(i, yd));
    const int bits = (int)sizeof(T) * 8;
    T r;
    if (c < 0 || (uint64_t)c >= (uint64_t)bits) r = (!kLeft && a < 0) ? (T)-1 : (T)0;
    else if (kLeft) r = (T)((U)a << (int)c);
    else r = (T)(a >> (int)c);
    *reinterpret_cast<T*>(z + strided_offset(i, zd)) = r;
}

template <typename T>
int launch_bit_shift(const chx_hip_tensor& x, const StridedDesc& xd, const chx_hip_tensor& y, const StridedDesc& yd, chx_hip_tensor& z, bool left,
                     int64_t n, hipStream_t s) {
    const unsigned blocks = (unsigned)((n + kThreads - 1) / kThreads);
    const StridedDesc zd = make_desc(z);
    if (left)
        bit_shift_kernel<T, true><<<blocks, kThreads, 0, s>>>(static_cast<const char*>(x.data), xd, static_cast<const char*>(y.data), yd,
                                                               static_cast<char*>(z.data), zd, n);
    else
        bit_shift_kernel<T, false><<<blocks, kThreads, 0, s>>>(static_cast<const char*>(x.data), xd, static_cast<const char*>(y.data), yd,
                                                                static_cast<char*>(z.data), zd, n);
    return launch_check("bit_shift_kernel");
}

// the descriptor of t seen through the shape of z: strides 0 where t broadcasts
int broadcast_desc(const chx_hip_tensor& t, const chx_hip_tensor& z, const char* what, StridedDesc* d) {
    CHX_REQUIRE(t.ndim <= z.ndim, "BitShift: %s has more axes than the result", what);
    d->ndim = z.ndim;
    for (int a = 0; a < z.ndim; ++a) {
        const int ta = a - (z.ndim - t.ndim);
        d->shape[a] = z.shape[a];
        if (ta < 0 || t.shape[ta] == 1) {
            d->strides[a] = 0;
        } else {
            CHX_REQUIRE(t.shape[ta] == z.shape[a], "BitShift: %s does not broadcast to the result (axis %d: %lld vs %lld)", what, a,
                        (long long)t.shape[ta], (long long)z.shape[a]);
            d->strides[a] = t.strides[ta];
        }
    }
    return CHX_HIP_OK;
}

}  // namespace
}  // namespace chx

extern "C" int chx_hip_bit_shift(const chx_hip_tensor* x, const chx_hip_tensor* y, int32_t left, chx_hip_tensor* z, void* stream) {
    CHX_PROPAGATE(check_tensor(x, "BitShift x"));
    CHX_PROPAGATE(check_tensor(y, "BitShift y"));
    CHX_PROPAGATE(check_tensor(z, "BitShift z"));
    CHX_REQUIRE(x->dtype == y->dtype && x->dtype == z->dtype, "BitShift: x, y and z must have one integer type, got %s, %s and %s",
                dtype_name(x->dtype), dtype_name(y->dtype), dtype_name(z->dtype));
    StridedDesc xd, yd;
    CHX_PROPAGATE(broadcast_desc(*x, *z, "x", &xd));
    CHX_PROPAGATE(broadcast_desc(*y, *z, "y", &yd));
    const int64_t n = numel(*z);
    if (n == 0) return CHX_HIP_OK;
    hipStream_t s = as_stream(stream);
    switch (x->dtype) {
        case CHX_HIP_UINT8: return launch_bit_shift<uint8_t>(*x, xd, *y, yd, *z, left != 0, n, s);
        case CHX_HIP_INT8: return launch_bit_shift<int8_t>(*x, xd, *y, yd, *z, left != 0, n, s);
        case CHX_HIP_INT16: return launch_bit_shift<int16_t>(*x, xd, *y, yd, *z, left != 0, n, s);
        case CHX_HIP_INT32: return launch_bit_shift<int32_t>(*x, xd, *y, yd, *z, left != 0, n, s);
        case CHX_HIP_INT64: return launch_bit_shift<int64_t>(*x, xd, *y, yd, *z, left != 0, n, s);
        default: CHX_FAIL(CHX_HIP_EINVAL, "BitShift: %s is not an integer type", dtype_name(x->dtype));  // CHECK(!IsFloat(...)), quantize.cc:154-155
    }
}

extern "C" int chx_hip_count_nonfinite(const chx_hip_tensor* x, int32_t infinities, int64_t* count, void* stream) {
    CHX_PROPAGATE(check_tensor(x, "non-finite scan x"));
    CHX_REQUIRE(count != nullptr, "non-finite scan: count is null");
    *count = 0;
    if (x->dtype != CHX_HIP_FLOAT32) return CHX_HIP_OK;  // integers hold neither
    const int64_t n = numel(*x);
    if (n == 0) return CHX_HIP_OK;
    hipStream_t s = as_stream(stream);
    int blocks = (int)((n + kThreads * 8 - 1) / (kThreads * 8));
    blocks = blocks < 1 ? 1 : blocks > 2048 ? 2048 : blocks;
    CHX_REQUIRE(n / blocks < (int64_t(1) << 32) - kThreads, "non-finite scan: array too large");
    void* dev = nullptr;
    CHX_PROPAGATE(scratch_alloc(&dev, sizeof(uint32_t) * blocks, s));
    const StridedDesc xd = make_desc(*x);
    // every block writes its own count: nothing to clear beforehand, no atomics
    if (infinities) count_nonfinite_kernel<true><<<blocks, kThreads, 0, s>>>(static_cast<const char*>(x->data), xd, n, static_cast<uint32_t*>(dev));
    else count_nonfinite_kernel<false><<<blocks, kThreads, 0, s>>>(static_cast<const char*>(x->data), xd, n, static_cast<uint32_t*>(dev));
    int rc = launch_check("count_nonfinite_kernel");
    std::vector<uint32_t> partial((size_t)blocks);
    if (rc == CHX_HIP_OK && (hipMemcpyAsync(partial.data(), dev, sizeof(uint32_t) * blocks, hipMemcpyDeviceToHost, s) != hipSuccess ||
                             hipStreamSynchronize(s) != hipSuccess)) {
        (void)hipGetLastError();
        rc = CHX_HIP_ERUNTIME;
    }
    scratch_free(dev, s);
    if (rc != CHX_HIP_OK) CHX_FAIL(rc, "non-finite scan: reading the counts back failed");
    int64_t host = 0;
    for (uint32_t c : partial) host += c;
    *count = host;
    return CHX_HIP_OK;
}
