// Pooling on 8-bit quantized tensors, for running whole quantized networks without
// leaving the 8-bit domain.  In a ChxVM program these appear as
//   DequantizeLinear -> MaxPool / AveragePool (runtime/ops/pooling.cc:47-75) -> QuantizeLinear;
// the hip backend lowers each such triple to one of these kernels.
//   max:     with the same scale and zero point on both sides the triple is a function of the
//            maximum of the codes (dequantization is increasing): uint8 Q(DQ(q)) == q; int8
//            Q(DQ(q)) == q + (q < 0), because QuantizeLinear adds 0.5 and the cast truncates toward zero.
//   average: y = Q( (sum of DQ(x) over the window, fp32, in (kh, kw) order) / count ).
// Both are bandwidth-bound; channels-last tensors move 16 channels per lane.
#include <cstring>

#include "chx_internal.h"
#include "quant_math.h"

namespace chx {
namespace {

constexpr int kThreads = 256;
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

struct PoolArgs {
    const char* x;
    char* y;
    int64_t xs[4], ys[4];  // byte strides of N, C, H, W
    int32_t N, C, H, W, OH, OW, kh, kw, sh, sw, ph, pw;
    int32_t is_signed;
    int64_t total;
};

__device__ __forceinline__ uint32_t max4_u8(uint32_t a, uint32_t b) {
    uint32_t r = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t x = (a >> (8 * i)) & 0xffu, y = (b >> (8 * i)) & 0xffu;
        r |= (x > y ? x : y) << (8 * i);
    }
    return r;
}

// The packed 16-bit maximum of two dwords (two 16-bit lanes per instruction).
typedef unsigned short v2us __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(v2us, a), __builtin_bit_cast(v2us, b)));
}

// channels-last, C % 16 == 0: one lane = 16 channels of one output pixel.  int8 codes are
// compared as unsigned after flipping the sign bit.  The taps go out in groups of nine
// unconditional loads: a tap outside the image reads the nearest pixel inside instead, which
// belongs to the same window whenever the window touches the image at all, so it does not change
// the maximum (a branch around the load would make every load wait for the one before).
// The maximum of the bytes of two dwords in three instructions: as 16-bit lanes the dwords compare by
// their high (odd) bytes first, so the packed maximum of the raw dwords carries the maximum of the odd
// bytes in its high bytes whatever the low bytes are; the even bytes are masked out and compared on
// their own.
// The device deals work-groups out to its 8 XCDs in turn, each with its own L2: work-group b takes block
// (b % 8) * xcd_chunk + b / 8, so that an XCD works through a contiguous run of output rows and finds the input rows
// that neighbouring output rows share in its own L2 (the launch is xcd_chunk * 8 work-groups).
template <bool kSigned>
__global__ __launch_bounds__(kThreads) void max_pool_cl16_kernel(PoolArgs a, uint32_t xcd_chunk) {
    const int64_t idx = (int64_t)((blockIdx.x & 7u) * xcd_chunk + (blockIdx.x >> 3)) * kThreads + threadIdx.x;
    if (idx >= a.total) return;
    const int cgroups = a.C / 16;
    const int cg = (int)(idx % cgroups);
    int64_t r = idx / cgroups;
    const int ow = (int)(r % a.OW);
    r /= a.OW;
    const int oh = (int)(r % a.OH);
    const int n = (int)(r / a.OH);
    const uint32_t flip = kSigned ? 0x80808080u : 0u;
    const int ih0 = oh * a.sh - a.ph, iw0 = ow * a.sw - a.pw;
    const bool touches = ih0 < a.H && ih0 + a.kh > 0 && iw0 < a.W && iw0 + a.kw > 0;
    const char* xn = a.x + n * a.xs[0] + cg * 16;
    uint32_t m_odd[4] = {0, 0, 0, 0}, m_even[4] = {0, 0, 0, 0};
    const int taps = a.kh * a.kw;
    int i = 0, j = 0;
    for (int t0 = 0; t0 < taps; t0 += 9) {
        v4u v[9];
#pragma unroll
        for (int t = 0; t < 9; ++t) {
            const int ih = min(max(ih0 + i, 0), a.H - 1), iw = min(max(iw0 + j, 0), a.W - 1);
            v[t] = *reinterpret_cast<const v4u*>(xn + ih * a.xs[2] + iw * a.xs[3]);
            // past the last tap: stay on it
            if (t0 + t + 1 < taps && ++j == a.kw) {
                j = 0;
                ++i;
            }
        }
#pragma unroll
        for (int t = 0; t < 9; ++t)
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const uint32_t x = kSigned ? v[t][d] ^ flip : v[t][d];
                m_odd[d] = pk_max_u16(m_odd[d], x);
                m_even[d] = pk_max_u16(m_even[d], x & 0x00ff00ffu);
            }
    }
    // int8: the QuantizeLinear behind the pool adds 0.5 and truncates toward zero, so a negative code
    // comes back one higher (q + 0.5 truncates to q + 1 for q < 0, to q for q >= 0).  In the flipped
    // domain a negative code is a byte below 128: add one to exactly those (no carry can leave the byte).
    v4u out;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        uint32_t u = touches ? m_even[d] | (m_odd[d] & 0xff00ff00u) : 0u;
        if (kSigned) u += (~u >> 7) & 0x01010101u;
        out[d] = u ^ flip;
    }
    *reinterpret_cast<v4u*>(a.y + n * a.ys[0] + oh * a.ys[2] + ow * a.ys[3] + cg * 16) = out;
}

// any strides: one lane = one output element, channel index fastest
__global__ __launch_bounds__(kThreads) void max_pool_generic_kernel(PoolArgs a) {
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= a.total) return;
    const int c = (int)(idx % a.C);
    int64_t r = idx / a.C;
    const int ow = (int)(r % a.OW);
    r /= a.OW;
    const int oh = (int)(r % a.OH);
    const int n = (int)(r / a.OH);
    int32_t m = a.is_signed ? -128 : 0;  // a window in the padding altogether: the lowest code, as Q(lowest float) is
    for (int i = 0; i < a.kh; ++i) {
        const int ih = oh * a.sh - a.ph + i;
        if ((unsigned)ih >= (unsigned)a.H) continue;
        for (int j = 0; j < a.kw; ++j) {
            const int iw = ow * a.sw - a.pw + j;
            if ((unsigned)iw >= (unsigned)a.W) continue;
            const uint8_t raw = *reinterpret_cast<const uint8_t*>(a.x + n * a.xs[0] + c * a.xs[1] + ih * a.xs[2] + iw * a.xs[3]);
            const int32_t v = a.is_signed ? (int32_t)(int8_t)raw : (int32_t)raw;
            m = v > m ? v : m;
        }
    }
    if (m < 0) ++m;  // int8 only: Q adds 0.5 and truncates toward zero
    *reinterpret_cast<uint8_t*>(a.y + n * a.ys[0] + c * a.ys[1] + oh * a.ys[2] + ow * a.ys[3]) = (uint8_t)m;
}

struct AvgArgs {
    PoolArgs p;
    float x_scale, x_zpf;
    int32_t count_include_pad;
    QuantParams q;
};

template <bool kRne>
__global__ __launch_bounds__(kThreads) void average_pool_kernel(AvgArgs a) {
    const PoolArgs& p = a.p;
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= p.total) return;
    const int c = (int)(idx % p.C);
    int64_t r = idx / p.C;
    const int ow = (int)(r % p.OW);
    r /= p.OW;
    const int oh = (int)(r % p.OH);
    const int n = (int)(r / p.OH);
    float sum = 0.f;
    int32_t cnt = 0;
    for (int i = 0; i < p.kh; ++i) {
        const int ih = oh * p.sh - p.ph + i;
        if ((unsigned)ih >= (unsigned)p.H) continue;
        for (int j = 0; j < p.kw; ++j) {
            const int iw = ow * p.sw - p.pw + j;
            if ((unsigned)iw >= (unsigned)p.W) continue;
            const uint8_t raw = *reinterpret_cast<const uint8_t*>(p.x + n * p.xs[0] + c * p.xs[1] + ih * p.xs[2] + iw * p.xs[3]);
            const int32_t v = p.is_signed ? (int32_t)(int8_t)raw : (int32_t)raw;
            sum = sum + dequantize_value(v, a.x_zpf, a.x_scale);
            ++cnt;
        }
    }
    if (a.count_include_pad) cnt = p.kh * p.kw;
    const float mean = sum / (float)cnt;
    *reinterpret_cast<uint8_t*>(p.y + n * p.ys[0] + c * p.ys[1] + oh * p.ys[2] + ow * p.ys[3]) =
            (uint8_t)quantize_value<kRne>(mean, a.q);
}

// Channels-last operands, four channels per lane: one dword load per tap instead of four byte
// loads, taps of a window row fetched together.  The sum runs over (kh, kw) in the same order as
// above, per channel, so the result is the same bytes.
template <bool kRne>
__global__ __launch_bounds__(kThreads) void average_pool_cl4_kernel(AvgArgs a) {
    constexpr int kBatch = 16;  // loads in flight at a time
    const PoolArgs& p = a.p;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int C4 = p.C >> 2;
    if (idx >= (p.total >> 2)) return;
    const int c = (int)(idx % C4) * 4;
    int64_t r = idx / C4;
    const int ow = (int)(r % p.OW);
    r /= p.OW;
    const int oh = (int)(r % p.OH);
    const int n = (int)(r / p.OH);
    const uint32_t flip = p.is_signed ? 0x80808080u : 0u;   // int8 code = (byte ^ 0x80) - 128
    const float zpf = a.x_zpf + (p.is_signed ? 128.f : 0.f);
    float sum[4] = {0.f, 0.f, 0.f, 0.f};
    int32_t cnt = 0;
    const char* xn = p.x + n * p.xs[0] + c;
    const int ih0 = oh * p.sh - p.ph, iw0 = ow * p.sw - p.pw;
    // taps in (kh, kw) order
    const int taps = p.kh * p.kw;
    int i = 0, j = 0;
    for (int t0 = 0; t0 < taps; t0 += kBatch) {
        uint32_t v[kBatch];
        uint64_t valid = 0;
        int ii = i, jj = j;
#pragma unroll
        for (int t = 0; t < kBatch; ++t) {
            const int ih = ih0 + ii, iw = iw0 + jj;
            // every load goes out, from a clamped address when the tap does not count: a branch around
            // it would make the compiler wait for each load before the next
            const int ihc = min(max(ih, 0), p.H - 1), iwc = min(max(iw, 0), p.W - 1);
            v[t] = *reinterpret_cast<const uint32_t*>(xn + ihc * p.xs[2] + iwc * p.xs[3]) ^ flip;
            valid |= (t0 + t < taps && ih == ihc && iw == iwc) ? uint64_t(1) << t : uint64_t(0);
            if (++jj == p.kw) {
                jj = 0;
                ++ii;
            }
        }
        i = ii;
        j = jj;
#pragma unroll
        for (int t = 0; t < kBatch; ++t) {
            const bool on = (valid >> t) & 1u;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float term = ((float)((v[t] >> (8 * e)) & 0xffu) - zpf) * a.x_scale;
                sum[e] = on ? sum[e] + term : sum[e];
            }
            cnt += on ? 1 : 0;
        }
    }
    if (a.count_include_pad) cnt = p.kh * p.kw;
    int32_t code[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) code[e] = quantize_value<kRne>(sum[e] / (float)cnt, a.q);
    *reinterpret_cast<uint32_t*>(p.y + n * p.ys[0] + oh * p.ys[2] + ow * p.ys[3] + c) = pack4(code[0], code[1], code[2], code[3]);
}

// The window is the whole image (global pooling) and the pixels of an image are one dense run:
// tap t of channel group c is at x + n*xs[0] + t*xs[3] + c, every tap counts, and all loads go out
// before the first sum.  The sum runs over the pixels in storage order = (kh, kw) order, so the
// result is the bytes of the kernels above.
constexpr int kGlobalPoolTaps = 64;
template <bool kRne>
__global__ __launch_bounds__(kThreads) void global_average_pool_cl4_kernel(AvgArgs a) {
    const PoolArgs& p = a.p;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int C4 = p.C >> 2;
    if (idx >= (p.total >> 2)) return;
    const int c = (int)(idx % C4) * 4;
    const int64_t n = idx / C4;
    const uint32_t flip = p.is_signed ? 0x80808080u : 0u;
    const float zpf = a.x_zpf + (p.is_signed ? 128.f : 0.f);
    const int taps = p.H * p.W;
    const char* xn = p.x + n * p.xs[0] + c;
    const uint32_t pitch = (uint32_t)p.xs[3];
    uint32_t v[kGlobalPoolTaps];
#pragma unroll
    for (int t = 0; t < kGlobalPoolTaps; ++t) v[t] = *reinterpret_cast<const uint32_t*>(xn + (uint32_t)min(t, taps - 1) * pitch) ^ flip;
    float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < kGlobalPoolTaps; ++t) {
        if (t < taps) {  // uniform
#pragma unroll
            for (int e = 0; e < 4; ++e) sum[e] = sum[e] + ((float)((v[t] >> (8 * e)) & 0xffu) - zpf) * a.x_scale;
        }
    }
    int32_t code[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) code[e] = quantize_value<kRne>(sum[e] / (float)taps, a.q);
    *reinterpret_cast<uint32_t*>(p.y + n * p.ys[0] + c) = pack4(code[0], code[1], code[2], code[3]);
}

// The float32 pools of MaxPoolOp / AveragePoolOp::RunImpl (runtime/ops/pooling.cc:47-75), for the float layers
// that stay around a quantized network: one lane = one output element, any strides, the taps in (kh, kw)
// order.  max: padding never wins, a window in the padding altogether gives the lowest finite float.  average:
// one float32 addition per tap that lies in the image, starting from 0, divided by the taps that count.
template <bool kMax>
__global__ __launch_bounds__(kThreads) void pool_f32_kernel(PoolArgs a, int count_include_pad) {
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= a.total) return;
    // the unit-stride axis of y fastest, so that neighbouring lanes write neighbouring floats
    const bool channels_fastest = a.ys[1] == 4;
    int c, ow, oh, n;
    int64_t r = idx;
    if (channels_fastest) {
        c = (int)(r % a.C); r /= a.C;
        ow = (int)(r % a.OW); r /= a.OW;
        oh = (int)(r % a.OH);
        n = (int)(r / a.OH);
    } else {
        ow = (int)(r % a.OW); r /= a.OW;
        oh = (int)(r % a.OH); r /= a.OH;
        c = (int)(r % a.C);
        n = (int)(r / a.C);
    }
    float acc = kMax ? -3.402823466e+38f : 0.f;
    int cnt = 0;
    for (int i = 0; i < a.kh; ++i) {
        const int ih = oh * a.sh - a.ph + i;
        if ((unsigned)ih >= (unsigned)a.H) continue;
        for (int j = 0; j < a.kw; ++j) {
            const int iw = ow * a.sw - a.pw + j;
            if ((unsigned)iw >= (unsigned)a.W) continue;
            const float v = *reinterpret_cast<const float*>(a.x + n * a.xs[0] + c * a.xs[1] + ih * a.xs[2] + iw * a.xs[3]);
            if (kMax) acc = v > acc ? v : acc;
            else acc = acc + v;
            ++cnt;
        }
    }
    if (!kMax) {
        if (count_include_pad) cnt = a.kh * a.kw;
        acc = acc / (float)cnt;
    }
    *reinterpret_cast<float*>(a.y + n * a.ys[0] + c * a.ys[1] + oh * a.ys[2] + ow * a.ys[3]) = acc;
}

int fill_pool_args(
        const chx_hip_tensor* x, chx_hip_tensor* y, int kh, int kw, int sh, int sw, int ph0, int pw0, int ph1, int pw1,
        int cover_all, const char* op, PoolArgs* a, bool float32 = false) {
    CHX_PROPAGATE(check_tensor(x, op));
    CHX_PROPAGATE(check_tensor(y, op));
    CHX_REQUIRE(x->ndim == 4 && y->ndim == 4, "%s: x and y must be 4-D", op);
    if (float32) CHX_REQUIRE(x->dtype == CHX_HIP_FLOAT32 && y->dtype == CHX_HIP_FLOAT32, "%s: x and y must be float32", op);
    else CHX_REQUIRE(is_q8(x->dtype) && is_q8(y->dtype), "%s: x and y must be uint8 or int8", op);
    CHX_REQUIRE(kh >= 1 && kw >= 1 && sh >= 1 && sw >= 1 && ph0 >= 0 && pw0 >= 0 && ph1 >= 0 && pw1 >= 0,
                "%s: bad kernel, stride or padding", op);
    const int64_t H = x->shape[2], W = x->shape[3];
    CHX_REQUIRE(H + ph0 + ph1 >= kh && W + pw0 + pw1 >= kw, "%s: kernel larger than the padded input", op);
    const int64_t OH = cover_all ? (H + ph0 + ph1 - kh + sh - 1) / sh + 1 : (H + ph0 + ph1 - kh) / sh + 1;
    const int64_t OW = cover_all ? (W + pw0 + pw1 - kw + sw - 1) / sw + 1 : (W + pw0 + pw1 - kw) / sw + 1;
    CHX_REQUIRE(y->shape[0] == x->shape[0] && y->shape[1] == x->shape[1] && y->shape[2] == OH && y->shape[3] == OW,
                "%s: y is [%lld,%lld,%lld,%lld], expected [%lld,%lld,%lld,%lld]", op, (long long)y->shape[0],
                (long long)y->shape[1], (long long)y->shape[2], (long long)y->shape[3], (long long)x->shape[0],
                (long long)x->shape[1], (long long)OH, (long long)OW);
    memset(a, 0, sizeof(*a));
    a->x = static_cast<const char*>(x->data);
    a->y = static_cast<char*>(y->data);
    for (int i = 0; i < 4; ++i) {
        a->xs[i] = x->strides[i];
        a->ys[i] = y->strides[i];
    }
    a->N = (int32_t)x->shape[0]; a->C = (int32_t)x->shape[1]; a->H = (int32_t)H; a->W = (int32_t)W;
    a->OH = (int32_t)OH; a->OW = (int32_t)OW;
    a->kh = kh; a->kw = kw; a->sh = sh; a->sw = sw; a->ph = ph0; a->pw = pw0;
    a->is_signed = x->dtype == CHX_HIP_INT8;
    a->total = (int64_t)a->N * a->C * OH * OW;
    return CHX_HIP_OK;
}

}  // namespace
}  // namespace chx

using namespace chx;

extern "C" int chx_hip_max_pool_q8(
        const chx_hip_tensor* x, int32_t kernel_h, int32_t kernel_w, int32_t stride_h, int32_t stride_w,
        int32_t pad_h_begin, int32_t pad_w_begin, int32_t pad_h_end, int32_t pad_w_end, int32_t cover_all,
        chx_hip_tensor* y, void* stream) {
    PoolArgs a;
    CHX_PROPAGATE(fill_pool_args(x, y, kernel_h, kernel_w, stride_h, stride_w, pad_h_begin, pad_w_begin, pad_h_end,
                                 pad_w_end, cover_all, "MaxPool", &a));
    CHX_REQUIRE(x->dtype == y->dtype, "MaxPool: x and y must have the same dtype");
    if (a.total == 0) return CHX_HIP_OK;
    hipStream_t s = as_stream(stream);
    int64_t px, py;
    const bool cl16 = a.C % 16 == 0 && is_channels_last(*x, &px) && is_channels_last(*y, &py) && aligned(x->data, 16) &&
                      aligned(y->data, 16) && px % 16 == 0 && py % 16 == 0;
    if (cl16) {
        a.total = (int64_t)a.N * a.OH * a.OW * (a.C / 16);
        const int64_t blocks = (a.total + kThreads - 1) / kThreads;
        CHX_REQUIRE(blocks < (int64_t(1) << 31) - 8, "MaxPool: 2^31 work-groups or more");
        const uint32_t xcd_chunk = (uint32_t)((blocks + 7) / 8);
        if (a.is_signed) max_pool_cl16_kernel<true><<<xcd_chunk * 8, kThreads, 0, s>>>(a, xcd_chunk);
        else max_pool_cl16_kernel<false><<<xcd_chunk * 8, kThreads, 0, s>>>(a, xcd_chunk);
        return launch_check("max_pool_cl16_kernel");
    }
    max_pool_generic_kernel<<<(unsigned)((a.total + kThreads - 1) / kThreads), kThreads, 0, s>>>(a);
    return launch_check("max_pool_generic_kernel");
}

extern "C" int chx_hip_average_pool_q8(
        const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, int32_t kernel_h, int32_t kernel_w,
        int32_t stride_h, int32_t stride_w, int32_t pad_h, int32_t pad_w, int32_t count_include_pad, float y_scale,
        int32_t y_zero_point, uint32_t flags, chx_hip_tensor* y, void* stream) {
    AvgArgs a;
    CHX_PROPAGATE(fill_pool_args(x, y, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, pad_h, pad_w, 0,
                                 "AveragePool", &a.p));
    const bool i8 = y->dtype == CHX_HIP_INT8;
    CHX_REQUIRE(y_zero_point >= (i8 ? -128 : 0) && y_zero_point <= (i8 ? 127 : 255),
                "AveragePool: zero point %d outside the range of %s", y_zero_point, dtype_name(y->dtype));
    if (a.p.total == 0) return CHX_HIP_OK;
    a.x_scale = x_scale;
    a.x_zpf = (float)x_zero_point;
    a.count_include_pad = count_include_pad;
    a.q = make_quant_params(y_scale, y_zero_point, i8);
    hipStream_t s = as_stream(stream);
    const bool cl4 = x->strides[1] == 1 && y->strides[1] == 1 && a.p.C % 4 == 0 && aligned(x->data, 4) && aligned(y->data, 4) &&
                     x->strides[0] % 4 == 0 && x->strides[2] % 4 == 0 && x->strides[3] % 4 == 0 && y->strides[0] % 4 == 0 &&
                     y->strides[2] % 4 == 0 && y->strides[3] % 4 == 0;
    if (cl4) {
        // small work-groups: a global pool has few outputs, and they should reach every compute unit
        const unsigned blocks4 = (unsigned)((a.p.total / 4 + 63) / 64);
        const bool rne = (flags & CHX_HIP_ROUND_ONNX_RNE) != 0;
        const PoolArgs& p = a.p;
        // the window is the whole image, stored as one dense run of pixels
        const bool whole_image = p.OH == 1 && p.OW == 1 && p.ph == 0 && p.pw == 0 && p.kh == p.H && p.kw == p.W &&
                                 (p.H == 1 || p.xs[2] == p.W * p.xs[3]) && p.H * p.W <= kGlobalPoolTaps;
        if (whole_image) {
            if (rne) global_average_pool_cl4_kernel<true><<<blocks4, 64, 0, s>>>(a);
            else global_average_pool_cl4_kernel<false><<<blocks4, 64, 0, s>>>(a);
            return launch_check("global_average_pool_cl4_kernel");
        }
        if (rne) average_pool_cl4_kernel<true><<<blocks4, 64, 0, s>>>(a);
        else average_pool_cl4_kernel<false><<<blocks4, 64, 0, s>>>(a);
        return launch_check("average_pool_cl4_kernel");
    }
    const unsigned blocks = (unsigned)((a.p.total + kThreads - 1) / kThreads);
    if (flags & CHX_HIP_ROUND_ONNX_RNE)
        average_pool_kernel<true><<<blocks, kThreads, 0, s>>>(a);
    else
        average_pool_kernel<false><<<blocks, kThreads, 0, s>>>(a);
    return launch_check("average_pool_kernel");
}

extern "C" int chx_hip_max_pool_f32(
        const chx_hip_tensor* x, int32_t kernel_h, int32_t kernel_w, int32_t stride_h, int32_t stride_w,
        int32_t pad_h_begin, int32_t pad_w_begin, int32_t pad_h_end, int32_t pad_w_end, int32_t cover_all,
        chx_hip_tensor* y, void* stream) {
    PoolArgs a;
    CHX_PROPAGATE(fill_pool_args(x, y, kernel_h, kernel_w, stride_h, stride_w, pad_h_begin, pad_w_begin, pad_h_end,
                                 pad_w_end, cover_all, "MaxPool", &a, true));
    if (a.total == 0) return CHX_HIP_OK;
    pool_f32_kernel<true><<<(unsigned)((a.total + kThreads - 1) / kThreads), kThreads, 0, as_stream(stream)>>>(a, 0);
    return launch_check("pool_f32_kernel");
}

extern "C" int chx_hip_average_pool_f32(
        const chx_hip_tensor* x, int32_t kernel_h, int32_t kernel_w, int32_t stride_h, int32_t stride_w, int32_t pad_h,
        int32_t pad_w, int32_t count_include_pad, chx_hip_tensor* y, void* stream) {
    PoolArgs a;
    CHX_PROPAGATE(fill_pool_args(x, y, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, pad_h, pad_w, 0, "AveragePool", &a, true));
    if (a.total == 0) return CHX_HIP_OK;
    pool_f32_kernel<false><<<(unsigned)((a.total + kThreads - 1) / kThreads), kThreads, 0, as_stream(stream)>>>(a, count_include_pad ? 1 : 0);
    return launch_check("pool_f32_kernel");
}
