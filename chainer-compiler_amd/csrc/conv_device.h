// Device-side pieces shared by the matrix-core convolution kernels (conv_mfma.hip, conv_bs.hip).
// Everything here has internal linkage: each translation unit gets its own copy.
#pragma once

#include "conv_mfma.h"

namespace chx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

// Row b (64 bytes) holds the byte b in every position.  A filter tap outside the image fetches
// the row of the activation zero point, so padding needs no data-dependent fix-up.
#define CHX_B16(v) v, v, v, v, v, v, v, v, v, v, v, v, v, v, v, v
#define CHX_ROW(v) CHX_B16(v), CHX_B16(v), CHX_B16(v), CHX_B16(v)
#define CHX_ROWS16(h)                                                                                     \
    CHX_ROW((h) * 16 + 0), CHX_ROW((h) * 16 + 1), CHX_ROW((h) * 16 + 2), CHX_ROW((h) * 16 + 3),           \
    CHX_ROW((h) * 16 + 4), CHX_ROW((h) * 16 + 5), CHX_ROW((h) * 16 + 6), CHX_ROW((h) * 16 + 7),           \
    CHX_ROW((h) * 16 + 8), CHX_ROW((h) * 16 + 9), CHX_ROW((h) * 16 + 10), CHX_ROW((h) * 16 + 11),         \
    CHX_ROW((h) * 16 + 12), CHX_ROW((h) * 16 + 13), CHX_ROW((h) * 16 + 14), CHX_ROW((h) * 16 + 15)
__device__ __attribute__((aligned(64))) const unsigned char g_fill_rows[256 * 64] = {
        CHX_ROWS16(0), CHX_ROWS16(1), CHX_ROWS16(2),  CHX_ROWS16(3),  CHX_ROWS16(4),  CHX_ROWS16(5),  CHX_ROWS16(6),  CHX_ROWS16(7),
        CHX_ROWS16(8), CHX_ROWS16(9), CHX_ROWS16(10), CHX_ROWS16(11), CHX_ROWS16(12), CHX_ROWS16(13), CHX_ROWS16(14), CHX_ROWS16(15)};
#undef CHX_ROWS16
#undef CHX_ROW
#undef CHX_B16

// n / d for n < 2^31 with the multiplier and shift of magic_divisor() (conv_mfma.h).
__device__ __forceinline__ uint32_t fast_div(uint32_t n, uint32_t mul, uint32_t shift) {
    return (__umulhi(n, mul) + n) >> shift;
}

// Asynchronous copy of 16 bytes per lane from global memory straight into LDS: lane i of the
// wavefront writes LDS bytes [lds_addr + 16*i, lds_addr + 16*i + 16).  lds_addr must be the
// same for all lanes (it travels in M0).  Completion is tracked by the wave's vector-memory
// counter like any load; nothing passes through registers.
__device__ __forceinline__ void async_copy16(const void* src, uint32_t lds_addr) {
    asm volatile(
            "s_mov_b32 m0, %1\n\t"
            "s_nop 0\n\t"
            "global_load_lds_dwordx4 %0, off"
            :
            : "v"(src), "s"(lds_addr)
            : "memory", "m0");
}

// Raw buffer resource over `bytes` bytes at `base` (no stride, no swizzle): an access at byte offset
// voffset + soffset + immediate that does not lie inside [0, bytes) reads zeros, and an asynchronous
// copy writes those zeros into LDS.
__device__ __forceinline__ v4i buffer_resource(const void* base, uint32_t bytes) {
    const uint64_t p = (uint64_t)base;
    v4i r;
    r[0] = (int)(uint32_t)p;
    r[1] = (int)((uint32_t)(p >> 32) & 0xffffu);
    r[2] = (int)bytes;
    r[3] = 0x00020000;
    // The resource is the same in every lane; saying so here makes the compiler keep it in scalar registers, where the
    // "s" operands of the copies below need it (the constraint alone does not: the compiler has handed over vector
    // registers for values it had decided to hold in them, which the assembler refuses).
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = __builtin_amdgcn_readfirstlane(r[i]);
    return r;
}

// The same for a 32-bit value that is the same in every lane.
__device__ __forceinline__ void keep_scalar(uint32_t& v) { v = (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }
__device__ __forceinline__ void keep_scalar(int& v) { v = __builtin_amdgcn_readfirstlane(v); }

// Per-lane byte offsets handed to buffer copies carry this bit when the lane must not fetch anything:
// the offset then lies beyond any resource this library builds (at most 2^31 - 1 bytes).
constexpr uint32_t kOutOfRange = 0x80000000u;

// Copies Q0 .. Q0+N-1 of a wave's group of up to four asynchronous 16-byte-per-lane copies through a buffer
// resource into LDS, as one statement so that nothing can touch M0 between them.  Copy q reads byte offset
// voff[q] + soff + q*1024 of the resource and lane i writes LDS bytes [lds_addr + q*1024 + 16*i, + 16): the
// immediate of the instruction is added on both sides, so the per-lane offsets handed in have q*1024
// subtracted already.
template <int N, int Q0>
__device__ __forceinline__ void buffer_copy16_run(const uint32_t (&voff)[4], v4i srd, uint32_t soff, uint32_t lds_addr) {
    static_assert(N >= 1 && Q0 >= 0 && Q0 + N <= 4, "the 12-bit immediate reaches four copies of 1 KB");
    if constexpr (N == 1)
        asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\t"
                     "buffer_load_dwordx4 %0, %1, %2 offen offset:%4 lds"
                     : : "v"(voff[Q0]), "s"(srd), "s"(soff), "s"(lds_addr), "n"(Q0 * 1024) : "memory", "m0");
    else if constexpr (N == 2)
        asm volatile("s_mov_b32 m0, %4\n\ts_nop 0\n\t"
                     "buffer_load_dwordx4 %0, %2, %3 offen offset:%5 lds\n\t"
                     "buffer_load_dwordx4 %1, %2, %3 offen offset:%6 lds"
                     : : "v"(voff[Q0]), "v"(voff[Q0 + 1]), "s"(srd), "s"(soff), "s"(lds_addr), "n"(Q0 * 1024), "n"(Q0 * 1024 + 1024) : "memory", "m0");
    else if constexpr (N == 3)
        asm volatile("s_mov_b32 m0, %5\n\ts_nop 0\n\t"
                     "buffer_load_dwordx4 %0, %3, %4 offen offset:%6 lds\n\t"
                     "buffer_load_dwordx4 %1, %3, %4 offen offset:%7 lds\n\t"
                     "buffer_load_dwordx4 %2, %3, %4 offen offset:%8 lds"
                     : : "v"(voff[Q0]), "v"(voff[Q0 + 1]), "v"(voff[Q0 + 2]), "s"(srd), "s"(soff), "s"(lds_addr), "n"(Q0 * 1024), "n"(Q0 * 1024 + 1024), "n"(Q0 * 1024 + 2048) : "memory", "m0");
    else
        asm volatile("s_mov_b32 m0, %6\n\ts_nop 0\n\t"
                     "buffer_load_dwordx4 %0, %4, %5 offen lds\n\t"
                     "buffer_load_dwordx4 %1, %4, %5 offen offset:1024 lds\n\t"
                     "buffer_load_dwordx4 %2, %4, %5 offen offset:2048 lds\n\t"
                     "buffer_load_dwordx4 %3, %4, %5 offen offset:3072 lds"
                     : : "v"(voff[0]), "v"(voff[1]), "v"(voff[2]), "v"(voff[3]), "s"(srd), "s"(soff), "s"(lds_addr) : "memory", "m0");
}

// The fields of a residual sum that its per-element arithmetic reads.
__device__ __forceinline__ ResidualAdd in_vector_registers(const ResidualAdd& p) {
    ResidualAdd v = p;
    v.c_flip = in_vector_register(p.c_flip);
    v.r_flip = in_vector_register(p.r_flip);
    v.c_zpf = in_vector_register(p.c_zpf);
    v.c_scale = in_vector_register(p.c_scale);
    v.r_zpf = in_vector_register(p.r_zpf);
    v.r_scale = in_vector_register(p.r_scale);
    v.big = in_vector_register(p.big);
    v.inv_out_scale = in_vector_register(p.inv_out_scale);
    v.out = in_vector_registers(p.out);
    v.out.lo = p.out.lo;  // selects the variant (a uniform branch) and bounds the int8 path only
    v.kc = in_vector_register(p.kc);
    v.kr = in_vector_register(p.kr);
    v.k0 = in_vector_register(p.k0);
    v.floor_pre = in_vector_register(p.floor_pre);
    return v;
}

// Sixteen codes of the convolution and sixteen of the residual -> sixteen codes of the sum
// (see ResidualAdd): the DequantizeLinear, Add, Relu and QuantizeLinear of quant_math.h in the
// reference's order, one IEEE operation each.
// kLean (uint8 result, zero points of r and of the result both 0, as between the Relu outputs of a
// residual network): the two "- 0.0f" / "+ 0.0f" change no value and are left out, and so is the
// Relu, because QuantizeLinear is monotone, Q(max(s, 0)) = max(Q(s), Q(0)) = max(Q(s), 0), and the
// saturating conversion already stops at 0.
template <bool kU8, bool kGuard, bool kLean = false>
__device__ __forceinline__ v4i add_residual16(v4i c, v4i r, const ResidualAdd& p) {
    static_assert(kU8 || !kLean, "the lean variant is for uint8 results");
    v4i out;
    float pre[16];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const uint32_t cw = (uint32_t)c[w] ^ p.c_flip, rw = (uint32_t)r[w] ^ p.r_flip;
        int32_t code[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float fa = ((float)((cw >> (8 * e)) & 0xffu) - p.c_zpf) * p.c_scale;
            const float rb = (float)((rw >> (8 * e)) & 0xffu);
            const float fb = kLean ? rb * p.r_scale : (rb - p.r_zpf) * p.r_scale;
            float sum = fa + fb;
            if (!kLean && p.relu) sum = __builtin_fmaxf(sum, 0.f);
            if (kGuard) sum = __builtin_amdgcn_fmed3f(sum, -p.big, p.big);
            if (kU8) pre[w * 4 + e] = quantize_prefloor_u8<false, !kLean>(sum, p.out, p.inv_out_scale, 0.f);
            else code[e] = quantize_value_folded<false>(sum, p.out, p.inv_out_scale, p.out.lo);
        }
        if (!kU8) out[w] = (int)pack4(code[0], code[1], code[2], code[3]);
    }
    if (kU8) {
        // all sixteen conversions under one switch of the rounding mode
        uint32_t words[4];
        floor_sat_u8x16(pre, words);
#pragma unroll
        for (int w = 0; w < 4; ++w) out[w] = (int)words[w];
    }
    return out;
}

// add_residual16 in the variant the parameters call for (the branches are uniform).
__device__ __forceinline__ v4i add_residual16_any(v4i val, v4i rv, const ResidualAdd& p) {
    if (p.lean) return p.guard ? add_residual16<true, true, true>(val, rv, p) : add_residual16<true, false, true>(val, rv, p);
    if (p.guard) return p.out.lo == 0.f ? add_residual16<true, true>(val, rv, p) : add_residual16<false, true>(val, rv, p);
    return p.out.lo == 0.f ? add_residual16<true, false>(val, rv, p) : add_residual16<false, false>(val, rv, p);
}

// The same sixteen codes from two fused multiply-adds per element (ResidualAdd::affine): with per-tensor scales
// the group Q(act(DQ(c) + DQ(r))) is, in real arithmetic, floor(c*kc + r*kr + k0) saturated; in float32 the two
// forms can differ where a sum falls within rounding distance of a code boundary, so this one is used only with
// constants for which find_affine_residual has compared it with add_residual16 on every pair of codes.  Five
// vector instructions per element instead of twelve.  kFloor: a Relu with a non-zero zero point of the sum (the
// saturation at 0 is the Relu otherwise).
template <bool kFloor>
__device__ __forceinline__ v4i affine_residual16(v4i c, v4i r, const ResidualAdd& p) {
    float pre[16];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const uint32_t cw = (uint32_t)c[w] ^ p.c_flip, rw = (uint32_t)r[w] ^ p.r_flip;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float cf = (float)((cw >> (8 * e)) & 0xffu);
            const float rf = (float)((rw >> (8 * e)) & 0xffu);
            float t = __builtin_fmaf(rf, p.kr, p.k0);
            t = __builtin_fmaf(cf, p.kc, t);
            if (kFloor) t = __builtin_fmaxf(t, p.floor_pre);
            pre[w * 4 + e] = t;
        }
    }
    uint32_t words[4];
    floor_sat_u8x16(pre, words);
    return v4i{(int)words[0], (int)words[1], (int)words[2], (int)words[3]};
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}


}  // namespace
}  // namespace chx
