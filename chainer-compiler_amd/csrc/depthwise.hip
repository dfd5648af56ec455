// Depthwise 3x3 QLinearConv (group == C == OC, one filter per channel) on channels-last 8-bit
// tensors.  Nine multiply-accumulates per output byte make this a memory-bound op; the work per
// element is kept low by pairing filter taps: for each channel, the codes of taps (2p, 2p+1) are
// gathered into one dword of two 16-bit lanes with a byte permute and multiplied against the
// pre-paired weights with one v_dot2_i32_i16, so a 3x3 window costs five permutes and five dot
// products instead of nine unpack-unpack-multiply-add sequences.
//
// A thread owns kCh consecutive channels (one 8-byte vector per pixel) and walks over
// kDwPixels output pixels of one output row; consecutive lanes own consecutive channel groups,
// so every load and store of a wavefront covers whole pixels.  Weights, scales and accumulator
// seeds stay in registers across the pixels; the register footprint is kept small enough for
// five or more waves per SIMD, which is what hides the load latency.
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

constexpr int kCh = 8;           // channels per thread
constexpr int kDw = kCh / 4;     // dwords per pixel vector
typedef int vxi __attribute__((ext_vector_type(kDw)));

template <bool kRne, bool kFloatBias, bool kXSigned>
__global__ __launch_bounds__(256) void depthwise3x3_kernel(DepthwiseArgs a) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int cgs = a.C / kCh;
    if (idx >= a.total) return;
    const int cg = (int)(idx % cgs);
    int64_t rest = idx / cgs;
    const int owb = (int)(rest % a.ow_blocks);
    rest /= a.ow_blocks;
    const int oh = (int)(rest % a.OH);
    const int n = (int)(rest / a.OH);
    const int c0 = cg * kCh;

    // pairs are stored per group of 16 channels: [c0 / 16][pair][c0 % 16 ...]
    int32_t wp[kPairs][kCh];
    const int32_t* pbase = a.pairs + (int64_t)(c0 / 16) * kPairs * 16 + (c0 % 16);
#pragma unroll
    for (int p = 0; p < kPairs; ++p)
#pragma unroll
        for (int d = 0; d < kDw; ++d) {
            const v4i v = *reinterpret_cast<const v4i*>(pbase + p * 16 + d * 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) wp[p][d * 4 + e] = v[e];
        }
    // per channel: accumulator seed -zp * sum_t w (+ int32 bias, ONNX mode), scale x_scale * w_scale,
    // float bias (reference mode)
    float sc[kCh], fb[kCh];
    int32_t seed[kCh];
#pragma unroll
    for (int d = 0; d < kDw; ++d) {
        const v4i ws4 = *reinterpret_cast<const v4i*>(a.wsum + c0 + d * 4);
        v4i b4 = {0, 0, 0, 0};
        if (a.bias) b4 = *reinterpret_cast<const v4i*>(a.bias + c0 + d * 4);
        v4f s4;
        if (a.w_scale_len > 1) s4 = *reinterpret_cast<const v4f*>(a.w_scale + c0 + d * 4);
        else s4 = v4f{a.w_scale[0], a.w_scale[0], a.w_scale[0], a.w_scale[0]};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            seed[d * 4 + e] = -a.x_zp_u * ws4[e] + (kFloatBias ? 0 : b4[e]);
            sc[d * 4 + e] = a.x_scale * s4[e];
            fb[d * 4 + e] = kFloatBias ? (float)b4[e] : 0.f;
        }
    }
    const bool u8_reference = !kRne && a.q.lo == 0.f && a.q.hi == 255.f, lower_bound = a.lo_folded > 0.f;  // uniform
    const int fill = (int)(((uint32_t)(a.x_zp_u & 0xff)) * 0x01010101u);  // the zero point, already in the unsigned range
    const char* xn = a.x + (int64_t)n * a.x_n_stride + c0;
    char* yrow = a.y + (int64_t)n * a.y_n_stride + (int64_t)oh * a.y_h_stride + c0;
    const int ih0 = oh * a.sh - a.ph;
    // the three input rows of this output row, clamped into the image so that every load is
    // valid; what a tap outside the image contributes is replaced by the zero point afterwards
    const char* rowp[3];
    bool row_ok[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        const int ih = ih0 + i;
        row_ok[i] = (unsigned)ih < (unsigned)a.H;
        rowp[i] = xn + (int64_t)min(max(ih, 0), a.H - 1) * a.x_h_stride;
    }
    const uint32_t wstride = (uint32_t)a.x_w_stride;  // the host checked that a row spans less than 2^31 bytes

    for (int p = 0; p < kDwPixels; ++p) {
        const int ow = owb * kDwPixels + p;
        if (ow >= a.OW) break;
        const int iw0 = ow * a.sw - a.pw;
        vxi x[kTaps + 1];
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            const int iw = iw0 + j;
            const bool col_ok = (unsigned)iw < (unsigned)a.W;
            const uint32_t off = (uint32_t)min(max(iw, 0), a.W - 1) * wstride;
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                vxi v = *reinterpret_cast<const vxi*>(rowp[i] + off);
                if (kXSigned) v ^= (int)0x80808080;
                const bool ok = col_ok && row_ok[i];
#pragma unroll
                for (int d = 0; d < kDw; ++d) v[d] = ok ? v[d] : fill;
                x[i * 3 + j] = v;
            }
        }
#pragma unroll
        for (int d = 0; d < kDw; ++d) x[kTaps][d] = 0;
        vxi o;
#pragma unroll
        for (int d = 0; d < kDw; ++d) {
            int32_t code[4];
            float pre[4];
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
                if (kFloatBias) v = v + fb[ch];
                // uint8 in the reference's rounding: clamp, conversion and packing in floor_sat_u8x4
                if (u8_reference) pre[e] = lower_bound ? quantize_prefloor_u8<true>(v, a.q, a.inv_y_scale, a.lo_folded)
                                                        : quantize_prefloor_u8<false>(v, a.q, a.inv_y_scale, 0.f);
                else code[e] = quantize_value_folded<kRne>(v, a.q, a.inv_y_scale, a.lo_folded);
            }
            o[d] = u8_reference ? (int)floor_sat_u8x4(pre[0], pre[1], pre[2], pre[3]) : (int)pack4(code[0], code[1], code[2], code[3]);
        }
        *reinterpret_cast<vxi*>(yrow + (int64_t)ow * a.y_w_stride) = o;
    }
}

}  // namespace

int pack_depthwise(const chx_hip_tensor& w, int32_t* pairs, int32_t* wsum, hipStream_t s) {
    const int C = (int)w.shape[0];
    pack_depthwise_kernel<<<(C + 255) / 256, 256, 0, s>>>(
            static_cast<const char*>(w.data), w.strides[0], w.strides[2], w.strides[3], C, pairs, wsum);
    return launch_check("pack_depthwise_kernel");
}

int launch_depthwise3x3(DepthwiseArgs a, bool rne, hipStream_t s) {
    a.ow_blocks = (a.OW + kDwPixels - 1) / kDwPixels;
    a.total = (int64_t)a.N * a.OH * a.ow_blocks * (a.C / kCh);
    if (a.total == 0) return CHX_HIP_OK;
    const unsigned blocks = (unsigned)((a.total + 255) / 256);
    const bool fbias = a.bias != nullptr && a.float_bias != 0;
    const bool xs = a.x_signed != 0;
#define CHX_DW(RN, FB, XS) depthwise3x3_kernel<RN, FB, XS><<<blocks, 256, 0, s>>>(a)
    if (rne) {
        if (fbias) { if (xs) CHX_DW(true, true, true); else CHX_DW(true, true, false); }
        else { if (xs) CHX_DW(true, false, true); else CHX_DW(true, false, false); }
    } else {
        if (fbias) { if (xs) CHX_DW(false, true, true); else CHX_DW(false, true, false); }
        else { if (xs) CHX_DW(false, false, true); else CHX_DW(false, false, false); }
    }
#undef CHX_DW
    return launch_check("depthwise3x3_kernel");
}

}  // namespace chx
