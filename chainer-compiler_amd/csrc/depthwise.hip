// Depthwise 3x3 QLinearConv (group == C == OC, one filter per channel) on channels-last 8-bit
// tensors.  Nine multiply-accumulates per output byte make this a memory-bound op, so the work per
// byte has to be small:
//   * a thread owns four consecutive channels (one dword per pixel) of one output column and walks
//     down kRows output rows.  Consecutive lanes own consecutive channel groups, then consecutive
//     pixels of the row: every load and store of a wavefront is one dense run of bytes, whatever
//     the channel count.
//   * per input row the thread loads the three dwords under the filter row and repacks them, per
//     channel, into one dword [x(i,0), x(i,1), x(i,2), 0] with two byte permutes; one
//     v_dot4_i32_i8 against [w(i,0), w(i,1), w(i,2), 0] is then a whole filter row.  The packed
//     rows stay in registers while the window moves down: with stride 1 an output row costs one
//     new input row (3 loads, 8 permutes, 12 dot products for its four bytes) instead of nine
//     loads and nine unpack-multiply-add sequences per byte.
//
// Arithmetic: the codes are brought to the signed range (uint8: flip the top bit = code - 128;
// int8: as stored), the zero point likewise; padding taps read the zero point, which makes them
// contribute (zp - zp) * w = 0; the accumulator starts at  -zp_signed * sum_t w[c][t]  (+ bias in
// ONNX mode), so the int32 sum is exactly  sum_t (x - zp) * w  and the epilogue is the shared
// requantization.
#include <type_traits>

#include "contract.h"
#include "depthwise.h"

namespace chx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));


// w [C][1][3][3] (any strides) -> rows [C/4][3][4] dwords, dword (i, e) of a channel group =
// bytes [w(i,0), w(i,1), w(i,2), 0] of channel 4*group + e, and wsum[c].  One thread per channel.
__global__ __launch_bounds__(256) void pack_depthwise_kernel(
        const char* __restrict__ w, int64_t s_oc, int64_t s_kh, int64_t s_kw, int C, int32_t* __restrict__ rows,
        int32_t* __restrict__ wsum) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    int32_t sum = 0;
    for (int i = 0; i < 3; ++i) {
        uint32_t word = 0;
        for (int j = 0; j < 3; ++j) {
            const int32_t t = *reinterpret_cast<const int8_t*>(w + c * s_oc + i * s_kh + j * s_kw);
            sum += t;
            word |= ((uint32_t)t & 0xffu) << (8 * j);
        }
        rows[(c / 4) * 12 + i * 4 + (c % 4)] = (int32_t)word;
    }
    wsum[c] = sum;
}

// kStep: vertical stride 1 or 2 (the packed input rows shared between neighbouring output rows
// are kept), 0: any stride (every output row loads its three input rows).
// kPath: 0 any 8-bit type and rounding; 1 uint8 in the reference's rounding (floor_sat_u8x4);
// 2 the same with a lower bound above 0 (a folded Relu); 3 as 1 with a zero point of 0.  Chosen by the launcher, so that the
// row loop has no branches and the loads of a whole strip are in flight together.
// Output rows per thread.  More rows spread the per-thread set-up (index arithmetic, masks, filter
// rows and constants) and the two halo rows over more outputs, at the price of registers for the
// loads in flight: stride 1 takes 14 rows when the output height is a multiple of 14 (224 / 2^k
// images) and the image is at least 56 rows high; 7 when it is a multiple of 7 (the 28x28, 14x14 and 7x7 images: with 14
// rows per thread a 14x14 layer at batch 128 is 2.6 wavefronts per SIMD, which is launch and memory latency and nothing
// else; measured on MobileNetV2: the 17 launches 0.306 -> 0.292 ms); otherwise 8.
// kStrip: 0 = 8 rows, 1 = 14, 2 = 7.
constexpr int rows_per_thread(int step, int strip) { return step == 1 ? (strip == 1 ? 14 : strip == 2 ? 7 : 8) : step == 2 ? 4 : 1; }
constexpr int kDwThreads = 64;  // small groups: (output columns x channel groups) of a row is rarely a multiple of 256
template <bool kRne, bool kFloatBias, int kStep, int kPath, int kStrip>
__global__ __launch_bounds__(kDwThreads) void depthwise3x3_kernel(DepthwiseArgs a) {
    constexpr int kRows = rows_per_thread(kStep, kStrip);
    constexpr int kInRows = kStep == 1 ? kRows + 2 : kStep == 2 ? 2 * kRows + 1 : 3;
    // blocks: x over (output column, channel group) of one strip of output rows, then the strips, then the images;
    // which block this work-group takes: see DepthwiseArgs
    const uint32_t block = (blockIdx.x & 7u) * a.xcd_chunk + (blockIdx.x >> 3);
    if (block >= a.blocks) return;
    const uint32_t bz = block / a.grid_xy, bxy = block - bz * a.grid_xy;
    const uint32_t by = bxy / a.grid_x, bx = bxy - by * a.grid_x;
    const uint32_t idx = bx * kDwThreads + threadIdx.x;
    const uint32_t cgs = (uint32_t)a.C >> 2;
    if (idx >= (uint32_t)a.OW * cgs) return;
    const int ow = (int)(idx / cgs);
    const int cg = (int)(idx - (uint32_t)ow * cgs);
    const int ohb = (int)by;
    const int n = (int)bz;
    const int c0 = cg * 4;

    v4i wq[3];
    float sc[4], fb[4];
    int32_t seed[4];
    const uint32_t flip = a.x_signed ? 0u : 0x80808080u;                        // stored code -> signed range
    const uint32_t fill = (uint32_t)((a.x_zp_u ^ 0x80) & 0xff) * 0x01010101u;   // the zero point in the signed range
    // addresses = a base that is the same for the whole work-group (image, row: scalar registers)
    // + a 32-bit offset per lane (column, channel group)
    const char* xn = a.x + (int64_t)n * a.x_n_stride;
    char* yn = a.y + (int64_t)n * a.y_n_stride;
    const uint32_t y_off = (uint32_t)ow * (uint32_t)a.y_w_stride + (uint32_t)c0;  // the host checked that a row spans less than 2^31 bytes
    // the three input columns of this output column, clamped into the image so that every load is
    // valid; what a tap outside the image contributes is replaced by the zero point afterwards
    const int iw0 = ow * a.sw - a.pw;
    uint32_t coff[3], col_mask[3];
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        const int iw = iw0 + j;
        col_mask[j] = (unsigned)iw < (unsigned)a.W ? ~0u : 0u;
        coff[j] = (uint32_t)min(max(iw, 0), a.W - 1) * (uint32_t)a.x_w_stride + (uint32_t)c0;
    }
    // the three dwords of input row ih under the filter, in the signed range, taps outside the image
    // replaced by the zero point
    auto load_row = [&](int ih, uint32_t (&v)[3]) {
        const uint32_t row_mask = (unsigned)ih < (unsigned)a.H ? ~0u : 0u;
        const char* rowp = xn + (int64_t)min(max(ih, 0), a.H - 1) * a.x_h_stride;
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            // bit arithmetic, not a conditional: as a select of the loaded value the compiler
            // turns it into a branch around the load, and every load then waits for the one before
            const uint32_t m = row_mask & col_mask[j];
            v[j] = ((*reinterpret_cast<const uint32_t*>(rowp + coff[j]) ^ flip) & m) | (fill & ~m);
        }
    };
    // ... as four dwords, one per channel: bytes [x(ih, iw0), x(ih, iw0+1), x(ih, iw0+2), 0]
    auto pack_row = [&](const uint32_t (&v)[3], uint32_t (&rp)[4]) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t t = __builtin_amdgcn_perm(v[1], v[0], 0x0c0c0000u | ((4u + e) << 8) | (uint32_t)e);  // [v0.e, v1.e, 0, 0]
            rp[e] = __builtin_amdgcn_perm(v[2], t, 0x0c000100u | ((4u + e) << 16));                               // [v0.e, v1.e, v2.e, 0]
        }
    };
    auto finish = [&](int oh, const uint32_t (&r0)[4], const uint32_t (&r1)[4], const uint32_t (&r2)[4]) {
        int32_t code[4];
        float pre[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            // (all three through the builtin: the compiler then knows they are dot products and keeps the
            // wait states that gfx950 wants between a dot product and a different instruction reading its result)
            int32_t acc = seed[e];
            acc = __builtin_amdgcn_sdot4((int)r0[e], wq[0][e], acc, false);
            acc = __builtin_amdgcn_sdot4((int)r1[e], wq[1][e], acc, false);
            acc = __builtin_amdgcn_sdot4((int)r2[e], wq[2][e], acc, false);
            float v = (float)acc * sc[e];
            if (kFloatBias) v = v + fb[e];
            // uint8 in the reference's rounding: clamp, conversion and packing in floor_sat_u8x4
            if (kPath == 2) pre[e] = quantize_prefloor_u8<true>(v, a.q, a.inv_y_scale, a.lo_folded);
            else if (kPath == 1) pre[e] = quantize_prefloor_u8<false>(v, a.q, a.inv_y_scale, 0.f);
            else if (kPath == 3) pre[e] = quantize_prefloor_u8<false, false>(v, a.q, a.inv_y_scale, 0.f);
            else code[e] = quantize_value_folded<kRne>(v, a.q, a.inv_y_scale, a.lo_folded);
        }
        const uint32_t o = kPath ? floor_sat_u8x4(pre[0], pre[1], pre[2], pre[3]) : pack4(code[0], code[1], code[2], code[3]);
        if (oh < a.OH) *reinterpret_cast<uint32_t*>(yn + (int64_t)oh * a.y_h_stride + y_off) = o ^ a.y_flip;
    };

    // filter rows and per-channel constants; requested after the strip's input rows so that all of it is in flight together
    auto load_constants = [&]() {
#pragma unroll
        for (int i = 0; i < 3; ++i) wq[i] = *reinterpret_cast<const v4i*>(a.rows + (int64_t)cg * 12 + i * 4);
        // per channel: accumulator seed -zp * sum_t w (+ int32 bias, ONNX mode), scale x_scale * w_scale,
        // float bias (reference mode)
        {
            const v4i ws4 = *reinterpret_cast<const v4i*>(a.wsum + c0);
            v4i b4 = {0, 0, 0, 0};
            if (a.bias) b4 = *reinterpret_cast<const v4i*>(a.bias + c0);
            v4f s4;
            if (a.w_scale_len > 1) s4 = *reinterpret_cast<const v4f*>(a.w_scale + c0);
            else s4 = v4f{a.w_scale[0], a.w_scale[0], a.w_scale[0], a.w_scale[0]};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                seed[e] = (128 - a.x_zp_u) * ws4[e] + (kFloatBias ? 0 : b4[e]);
                sc[e] = a.x_scale * s4[e];
                fb[e] = kFloatBias ? (float)b4[e] : 0.f;
            }
        }
    };
    const int oh0 = ohb * kRows;
    uint32_t raw[kInRows][3], rp[3][4];
    if constexpr (kStep == 1) {
        // output row oh0 + p reads input rows ih0 + p .. ih0 + p + 2: two of them are already packed
        const int ih0 = oh0 - a.ph;
#pragma unroll
        for (int r = 0; r < kInRows; ++r) load_row(ih0 + r, raw[r]);
        load_constants();
        pack_row(raw[0], rp[0]);
        pack_row(raw[1], rp[1]);
#pragma unroll
        for (int p = 0; p < kRows; ++p) {
            pack_row(raw[p + 2], rp[(p + 2) % 3]);
            finish(oh0 + p, rp[p % 3], rp[(p + 1) % 3], rp[(p + 2) % 3]);
        }
    } else if constexpr (kStep == 2) {
        // output row oh0 + p reads input rows ih0 + 2p .. ih0 + 2p + 2: the last one is the next row's first
        const int ih0 = oh0 * 2 - a.ph;
#pragma unroll
        for (int r = 0; r < kInRows; ++r) load_row(ih0 + r, raw[r]);
        load_constants();
        pack_row(raw[0], rp[0]);
#pragma unroll
        for (int p = 0; p < kRows; ++p) {
            const int first = (p & 1) ? 2 : 0, last = 2 - first;
            pack_row(raw[2 * p + 1], rp[1]);
            pack_row(raw[2 * p + 2], rp[last]);
            finish(oh0 + p, rp[first], rp[1], rp[last]);
        }
    } else {
        const int ih0 = oh0 * a.sh - a.ph;
#pragma unroll
        for (int r = 0; r < 3; ++r) load_row(ih0 + r, raw[r]);
        load_constants();
#pragma unroll
        for (int r = 0; r < 3; ++r) pack_row(raw[r], rp[r]);
        finish(oh0, rp[0], rp[1], rp[2]);
    }
}

}  // namespace

int pack_depthwise(const chx_hip_tensor& w, int32_t* rows, int32_t* wsum, hipStream_t s) {
    const int C = (int)w.shape[0];
    pack_depthwise_kernel<<<(C + 255) / 256, 256, 0, s>>>(
            static_cast<const char*>(w.data), w.strides[0], w.strides[2], w.strides[3], C, rows, wsum);
    return launch_check("pack_depthwise_kernel");
}

int launch_depthwise3x3(DepthwiseArgs a, bool rne, hipStream_t s) {
    const int step = a.sh == 1 ? 1 : a.sh == 2 ? 2 : 0;
    const int strip = step != 1 ? 0 : (a.OH % 14 == 0 && a.OH >= 56) ? 1 : a.OH % 7 == 0 ? 2 : 0;
    const int rows = rows_per_thread(step, strip);
    a.oh_blocks = (a.OH + rows - 1) / rows;
    a.total = (int64_t)a.N * a.oh_blocks * a.OW * (a.C / 4);
    if (a.total == 0) return CHX_HIP_OK;
    if (a.oh_blocks > 65535 || a.N > 65535 || (int64_t)a.OW * (a.C / 4) >= (int64_t(1) << 31))
        CHX_FAIL(CHX_HIP_EUNSUPPORTED, "depthwise kernel: more than 65535 images or row strips, or a row of 2^31 channel groups");
    const int64_t grid_x = ((int64_t)a.OW * (a.C / 4) + kDwThreads - 1) / kDwThreads;
    const int64_t all_blocks = grid_x * a.oh_blocks * a.N;
    if (all_blocks >= (int64_t(1) << 31) - 8) CHX_FAIL(CHX_HIP_EUNSUPPORTED, "depthwise kernel: 2^31 work-groups or more");
    a.grid_x = (uint32_t)grid_x;
    a.grid_xy = (uint32_t)(grid_x * a.oh_blocks);
    a.blocks = (uint32_t)all_blocks;
    a.xcd_chunk = (uint32_t)((all_blocks + 7) / 8);
    const dim3 blocks(a.xcd_chunk * 8u);
    const bool fbias = a.bias != nullptr && a.float_bias != 0;
    const bool u8_reference = !rne && a.q.lo == 0.f && a.q.hi == 255.f;
    const int path = !u8_reference ? 0 : a.lo_folded > 0.f ? 2 : a.q.zpf == 0.f ? 3 : 1;
#define CHX_DW_P(RN, FB, ST, TL)                                                                    \
    do {                                                                                            \
        if (path == 0) depthwise3x3_kernel<RN, FB, ST, 0, TL><<<blocks, kDwThreads, 0, s>>>(a);     \
        else if (RN) CHX_FAIL(CHX_HIP_ERUNTIME, "depthwise: conversion path");                      \
        else if (path == 1) depthwise3x3_kernel<false, FB, ST, 1, TL><<<blocks, kDwThreads, 0, s>>>(a); \
        else if (path == 3) depthwise3x3_kernel<false, FB, ST, 3, TL><<<blocks, kDwThreads, 0, s>>>(a); \
        else depthwise3x3_kernel<false, FB, ST, 2, TL><<<blocks, kDwThreads, 0, s>>>(a);            \
    } while (0)
#define CHX_DW_S(RN, FB)                               \
    do {                                               \
        if (strip == 1) CHX_DW_P(RN, FB, 1, 1);        \
        else if (strip == 2) CHX_DW_P(RN, FB, 1, 2);   \
        else if (step == 1) CHX_DW_P(RN, FB, 1, 0);    \
        else if (step == 2) CHX_DW_P(RN, FB, 2, 0);    \
        else CHX_DW_P(RN, FB, 0, 0);                   \
    } while (0)
    if (rne) {
        if (fbias) CHX_DW_S(true, true);
        else CHX_DW_S(true, false);
    } else {
        if (fbias) CHX_DW_S(false, true);
        else CHX_DW_S(false, false);
    }
#undef CHX_DW_S
#undef CHX_DW_P
    return launch_check("depthwise3x3_kernel");
}

}  // namespace chx
