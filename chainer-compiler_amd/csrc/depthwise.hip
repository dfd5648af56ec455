// Depthwise 3x3 QLinearConv (group == C == OC, one filter per channel) on channels-last 8-bit
// tensors.  Nine multiply-accumulates per output byte make this a memory-bound op; the work per
// element is kept low by pairing filter taps: for each channel, the codes of taps (2p, 2p+1) are
// gathered into one dword of two 16-bit lanes with a byte permute and multiplied against the
// pre-paired weights with one v_dot2_i32_i16, so a 3x3 window costs five permutes and five dot
// products instead of nine unpack-unpack-multiply-add sequences.
//
// A thread owns 16 consecutive channels (one 16-byte vector per pixel) and walks over
// kDwPixels output pixels of one output row; consecutive lanes own consecutive channel groups,
// so every load and store of a wavefront covers whole pixels.  Weights (80 dwords), scales and
// accumulator seeds stay in registers across the pixels.
//
// Arithmetic: int8 activations are shifted to the unsigned range by flipping the top bit
// (code + 128, zero point + 128); padding taps read the zero point, which makes them contribute
// (zp - zp) * w = 0; the accumulator starts at  -zp * sum_t w[c][t] (+ bias in ONNX mode), so the
// int32 sum is exactly  sum_t (x - zp) * w  and the epilogue is the shared requantization.
#include <type_traits>

#include "contract.h"
#include "depthwise.h"

namespace chx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef short v2s __attribute__((ext_vector_type(2)));

constexpr int kDwPixels = 4;
constexpr int kTaps = 9;
constexpr int kPairs = 5;

// w [C][1][3][3] (any strides) -> pairs [C/16][kPairs][16] dwords (lo16 = tap 2p, hi16 = tap 2p+1 or 0)
// and wsum[c].  One thread per channel.
__global__ __launch_bounds__(256) void pack_depthwise_kernel(
        const char* __restrict__ w, int64_t s_oc, int64_t s_kh, int64_t s_kw, int C, int32_t* __restrict__ pairs,
        int32_t* __restrict__ wsum) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    int32_t t[kTaps + 1];
    int32_t sum = 0;
    for (int i = 0; i < kTaps; ++i) {
        t[i] = *reinterpret_cast<const int8_t*>(w + c * s_oc + (i / 3) * s_kh + (i % 3) * s_kw);
        sum += t[i];
    }
    t[kTaps] = 0;
    for (int p = 0; p < kPairs; ++p)
        pairs[((c / 16) * kPairs + p) * 16 + (c % 16)] = (t[2 * p] & 0xffff) | (t[2 * p + 1] << 16);
    wsum[c] = sum;
}

template <bool kRne>
__global__ __launch_bounds__(256) void depthwise3x3_kernel(DepthwiseArgs a) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int cgs = a.C / 16;
    if (idx >= a.total) return;
    const int cg = (int)(idx % cgs);
    int64_t rest = idx / cgs;
    const int owb = (int)(rest % a.ow_blocks);
    rest /= a.ow_blocks;
    const int oh = (int)(rest % a.OH);
    const int n = (int)(rest / a.OH);
    const int c0 = cg * 16;

    int32_t wp[kPairs][16];
#pragma unroll
    for (int p = 0; p < kPairs; ++p)
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const v4i v = *reinterpret_cast<const v4i*>(a.pairs + ((int64_t)cg * kPairs + p) * 16 + d * 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) wp[p][d * 4 + e] = v[e];
        }
    float sc[16];
    int32_t seed[16];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const v4f s4 = *reinterpret_cast<const v4f*>(a.scale + c0 + d * 4);
        const v4i a4 = *reinterpret_cast<const v4i*>(a.seed + c0 + d * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            sc[d * 4 + e] = s4[e];
            seed[d * 4 + e] = a4[e];
        }
    }
    const int flip = a.x_signed ? (int)0x80808080 : 0;
    const int fill = (int)(((uint32_t)(a.x_zp_u & 0xff)) * 0x01010101u);
    const char* xn = a.x + (int64_t)n * a.x_n_stride + c0;
    char* yrow = a.y + (int64_t)n * a.y_n_stride + (int64_t)oh * a.y_h_stride + c0;
    const int ih0 = oh * a.sh - a.ph;
    const bool float_bias = a.fbias != nullptr;

    for (int p = 0; p < kDwPixels; ++p) {
        const int ow = owb * kDwPixels + p;
        if (ow >= a.OW) break;
        const int iw0 = ow * a.sw - a.pw;
        v4i x[kTaps + 1];
#pragma unroll
        for (int t = 0; t < kTaps; ++t) {
            const int ih = ih0 + t / 3, iw = iw0 + t % 3;
            v4i v = {fill, fill, fill, fill};
            if ((unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W) {
                v = *reinterpret_cast<const v4i*>(xn + (int64_t)ih * a.x_h_stride + (int64_t)iw * a.x_w_stride);
                v ^= flip;
            }
            x[t] = v;
        }
        x[kTaps] = v4i{0, 0, 0, 0};
        uint32_t out[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            int32_t code[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int ch = d * 4 + e;
                int32_t acc = seed[ch];
#pragma unroll
                for (int q = 0; q < kPairs; ++q) {
                    // bytes: [x(2q).b_e, 0, x(2q+1).b_e, 0]
                    const uint32_t sel = 0x0c000c00u | (uint32_t)e | ((uint32_t)(4 + e) << 16);
                    const uint32_t xp = __builtin_amdgcn_perm((uint32_t)x[2 * q + 1][d], (uint32_t)x[2 * q][d], sel);
                    acc = __builtin_amdgcn_sdot2(__builtin_bit_cast(v2s, xp), __builtin_bit_cast(v2s, wp[q][ch]), acc, false);
                }
                float v = (float)acc * sc[ch];
                if (float_bias) v = v + a.fbias[c0 + ch];
                code[e] = quantize_value_folded<kRne>(v, a.q, a.inv_y_scale, a.lo_folded);
            }
            out[d] = pack4(code[0], code[1], code[2], code[3]);
        }
        const v4i o = {(int)out[0], (int)out[1], (int)out[2], (int)out[3]};
        *reinterpret_cast<v4i*>(yrow + (int64_t)ow * a.y_w_stride) = o;
    }
}

// seed[c] = -zp_u * wsum[c] (+ bias, ONNX mode); scale[c] = x_scale * w_scale[c]; fbias[c] = float(bias[c])
__global__ __launch_bounds__(256) void depthwise_params_kernel(
        int C, const int32_t* __restrict__ wsum, int32_t zp_u, const float* __restrict__ w_scale, int w_scale_len,
        float x_scale, const int32_t* __restrict__ bias, int bias_mode, int32_t* __restrict__ seed,
        float* __restrict__ scale, float* __restrict__ fbias) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    int32_t sd = -zp_u * wsum[c];
    if (bias && bias_mode == kBiasOnnxInt32) sd += bias[c];
    seed[c] = sd;
    scale[c] = x_scale * (w_scale_len > 1 ? w_scale[c] : w_scale[0]);
    fbias[c] = (bias && bias_mode == kBiasReferenceFloat) ? (float)bias[c] : 0.f;
}

}  // namespace

int pack_depthwise(const chx_hip_tensor& w, int32_t* pairs, int32_t* wsum, hipStream_t s) {
    const int C = (int)w.shape[0];
    pack_depthwise_kernel<<<(C + 255) / 256, 256, 0, s>>>(
            static_cast<const char*>(w.data), w.strides[0], w.strides[2], w.strides[3], C, pairs, wsum);
    return launch_check("pack_depthwise_kernel");
}

int launch_depthwise_params(
        int C, const int32_t* wsum, int32_t zp_u, const float* w_scale, int w_scale_len, float x_scale, const int32_t* bias,
        int bias_mode, int32_t* seed, float* scale, float* fbias, hipStream_t s) {
    depthwise_params_kernel<<<(C + 255) / 256, 256, 0, s>>>(C, wsum, zp_u, w_scale, w_scale_len, x_scale, bias, bias_mode, seed,
                                                            scale, fbias);
    return launch_check("depthwise_params_kernel");
}

int launch_depthwise3x3(DepthwiseArgs a, bool rne, hipStream_t s) {
    a.ow_blocks = (a.OW + kDwPixels - 1) / kDwPixels;
    a.total = (int64_t)a.N * a.OH * a.ow_blocks * (a.C / 16);
    if (a.total == 0) return CHX_HIP_OK;
    const unsigned blocks = (unsigned)((a.total + 255) / 256);
    if (rne)
        depthwise3x3_kernel<true><<<blocks, 256, 0, s>>>(a);
    else
        depthwise3x3_kernel<false><<<blocks, 256, 0, s>>>(a);
    return launch_check("depthwise3x3_kernel");
}

}  // namespace chx
