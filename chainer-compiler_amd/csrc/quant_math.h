// Device-side scalar arithmetic of the quantized ops, shared by every kernel that
// quantizes, dequantizes or requantizes.  Each function is the reference's fp32
// operation sequence; translation units including this header are compiled with
// -ffp-contract=off so that no two operations merge into a fused multiply-add.
#pragma once

#include <hip/hip_runtime.h>

#include <climits>
#include <cstdint>

namespace chx {

struct QuantParams {
    float scale;  // y_scale
    float zpf;    // float(y_zero_point); 0.0f when the reference skips the addition
    float lo;     // 0 or -128
    float hi;     // 255 or 127
};

inline QuantParams make_quant_params(float scale, int32_t zero_point, bool int8_out) {
    QuantParams q;
    q.scale = scale;
    q.zpf = (float)zero_point;
    q.lo = int8_out ? -128.f : 0.f;
    q.hi = int8_out ? 127.f : 255.f;
    return q;
}

// A wave-uniform constant held in a vector register.  Measured on gfx950 with a loop of independent instructions:
// one wavefront issues a vector instruction every 4.5 cycles whatever it is; two wavefronts of a SIMD run float32
// multiply / add / fused multiply-add, v_xor, v_mov and compares side by side (0.94 ns per instruction and SIMD)
// when all operands are vector registers, inline constants or literals, but take turns (1.77 ns) as soon as one
// operand is a scalar register; conversions, v_perm, v_med3, v_cvt_pk_u8, dot products and float64 always take
// turns.  So the constants of per-element float arithmetic that several wavefronts of a SIMD execute at once are
// copied into vector registers, once per tile.  (The convolution epilogue gains 2-3 % on 1x1 layers with few
// multiply-adds per output from it and nothing elsewhere: one wavefront's own issue rate is the usual limit.)
// The copy is opaque to the compiler, which would otherwise fold it back.
__device__ __forceinline__ float in_vector_register(float s) {
    float v;
    asm("v_mov_b32 %0, %1" : "=v"(v) : "v"(s));
    return v;
}
__device__ __forceinline__ uint32_t in_vector_register(uint32_t s) {
    uint32_t v;
    asm("v_mov_b32 %0, %1" : "=v"(v) : "v"(s));
    return v;
}
__device__ __forceinline__ QuantParams in_vector_registers(const QuantParams& q) {
    return QuantParams{in_vector_register(q.scale), in_vector_register(q.zpf), in_vector_register(q.lo), in_vector_register(q.hi)};
}
// quantize_array, runtime/ops/quantize.cc:29-34:
//   scaled = v / y_scale; if (zp != 0) scaled += zp;
//   AsType(Maximum(lo, Minimum(scaled, hi)) + 0.5f)          (AsType truncates)
// Adding zpf == 0.0f is the identity on every finite value except that it turns -0.0
// into +0.0, which the clamp, the +0.5f and the truncation cannot tell apart, so the
// reference's "skip when zero" needs no branch.
// kRne selects the ONNX operator text instead: saturate(rint(v / y_scale) + zp).
template <bool kRne>
__device__ __forceinline__ int32_t quantize_value(float v, const QuantParams& q) {
    float s = v / q.scale;  // IEEE-754 correctly rounded division
    if (kRne) {
        s = rintf(s) + q.zpf;
        s = s < q.hi ? s : q.hi;
        s = q.lo < s ? s : q.lo;
        return (int32_t)s;
    }
    s = s + q.zpf;
    s = s < q.hi ? s : q.hi;
    s = q.lo < s ? s : q.lo;
    s = s + 0.5f;
    return (int32_t)s;  // v_cvt_i32_f32 truncates toward zero
}

// The same code as quantize_value at a fraction of its cost: the IEEE division (about
// ten instructions) is replaced by three.  With inv = the correctly rounded reciprocal of
// the scale (computed on the host),
//     q0 = v * inv;   r = fma(-q0, scale, v);   q = fma(r, inv, q0)
// is the correctly rounded quotient v / scale (Markstein's division: q0 is within an ulp,
// the residual r is exact, and one correction with the rounded reciprocal lands on the
// rounded quotient).  The remaining steps are the reference's; min/max replace the
// compare-selects, which is the same function for every non-NaN value.
template <bool kRne>
__device__ __forceinline__ int32_t quantize_value_fast(float v, const QuantParams& q, float inv_scale) {
    const float q0 = v * inv_scale;
    const float r = __builtin_fmaf(-q0, q.scale, v);
    float s = __builtin_fmaf(r, inv_scale, q0);
    if (kRne) {
        s = rintf(s) + q.zpf;
        s = __builtin_fminf(s, q.hi);
        s = __builtin_fmaxf(s, q.lo);
        return (int32_t)s;
    }
    s = s + q.zpf;
    s = __builtin_fminf(s, q.hi);
    s = __builtin_fmaxf(s, q.lo);
    s = s + 0.5f;
    return (int32_t)s;
}

// The fused Relu (code = max(code, floor), floor = the output zero point) folded into the lower
// clamp bound: for a floor f >= 0 clamping to max(lo, f) gives f + 0.5 -> f for everything
// below, and what the truncation makes of values in [f - 0.5, f) is f either way; for f < 0
// the bound is f - 0.5, which the + 0.5 turns into exactly f, while values in [f - 0.5, f)
// keep the reference's truncation toward zero.  In ONNX rounding mode the clamp acts on
// integers and the bound is simply max(lo, f).
inline float fold_relu_floor(const QuantParams& q, int32_t relu_floor, bool rne) {
    if (relu_floor == INT32_MIN) return q.lo;
    const float f = (float)relu_floor;
    const float bound = (rne || relu_floor >= 0) ? f : f - 0.5f;
    return bound > q.lo ? bound : q.lo;
}

// quantize_value_fast with the lower bound of fold_relu_floor and the clamp as one median
// instruction (the same function as min/max for every non-NaN value).
template <bool kRne>
__device__ __forceinline__ int32_t quantize_value_folded(float v, const QuantParams& q, float inv_scale, float lo_folded) {
    const float q0 = v * inv_scale;
    const float r = __builtin_fmaf(-q0, q.scale, v);
    float s = __builtin_fmaf(r, inv_scale, q0);
    if (kRne) {
        s = rintf(s) + q.zpf;
        return (int32_t)__builtin_amdgcn_fmed3f(s, lo_folded, q.hi);
    }
    s = s + q.zpf;
    s = __builtin_amdgcn_fmed3f(s, lo_folded, q.hi);
    s = s + 0.5f;
    return (int32_t)s;
}

// uint8 results in the reference's rounding without the clamp, the conversion and the byte
// packing as separate instructions.  v_cvt_pk_u8_f32 converts with the current fp32 rounding
// mode, saturates to [0, 255] and drops the byte into place; under round-toward-minus-infinity it
// is clamp(floor(x), 0, 255) for every finite x (checked on gfx950 over all 2^32 inputs).  With
// x = t + 0.5f computed beforehand in the default rounding, that is the reference's
// AsType(Maximum(0, Minimum(t, 255)) + 0.5f): inside the range the two are the same operations,
// below it both give 0 (t + 0.5f <= 0.5 there), above it both give 255.  The rounding mode of the
// wave is switched and restored inside one asm statement, so no other instruction can end up
// between the two switches; the s_nop in front keeps two wait states between the restoring write of
// one statement and the switching write of the next, which the compiler cannot see (two writes of
// the same hardware register want that distance).  A lower bound above 0 (a folded Relu) is applied to t by the caller.
__device__ __forceinline__ uint32_t floor_sat_u8x4(float a, float b, float c, float d) {
    uint32_t r;
    asm volatile(
            "s_nop 1\n\t"
            "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 2\n\t"
            "v_cvt_pk_u8_f32 %0, %1, 0, 0\n\t"
            "v_cvt_pk_u8_f32 %0, %2, 1, %0\n\t"
            "v_cvt_pk_u8_f32 %0, %3, 2, %0\n\t"
            "v_cvt_pk_u8_f32 %0, %4, 3, %0\n\t"
            "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 0"
            : "=&v"(r)
            : "v"(a), "v"(b), "v"(c), "v"(d));
    return r;
}

__device__ __forceinline__ void floor_sat_u8x8(const float (&x)[8], uint32_t* lo, uint32_t* hi) {
    uint32_t r0, r1;
    asm volatile(
            "s_nop 1\n\t"
            "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 2\n\t"
            "v_cvt_pk_u8_f32 %0, %2, 0, 0\n\t"
            "v_cvt_pk_u8_f32 %1, %6, 0, 0\n\t"
            "v_cvt_pk_u8_f32 %0, %3, 1, %0\n\t"
            "v_cvt_pk_u8_f32 %1, %7, 1, %1\n\t"
            "v_cvt_pk_u8_f32 %0, %4, 2, %0\n\t"
            "v_cvt_pk_u8_f32 %1, %8, 2, %1\n\t"
            "v_cvt_pk_u8_f32 %0, %5, 3, %0\n\t"
            "v_cvt_pk_u8_f32 %1, %9, 3, %1\n\t"
            "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 0"
            : "=&v"(r0), "=&v"(r1)
            : "v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]), "v"(x[4]), "v"(x[5]), "v"(x[6]), "v"(x[7]));
    *lo = r0;
    *hi = r1;
}

// Sixteen values under one switch of the rounding mode: word w holds x[4w .. 4w+3].
__device__ __forceinline__ void floor_sat_u8x16(const float (&x)[16], uint32_t (&out)[4]) {
    uint32_t r0, r1, r2, r3;
    asm volatile(
            "s_nop 1\n\t"
            "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 2\n\t"
            "v_cvt_pk_u8_f32 %0, %4, 0, 0\n\t"
            "v_cvt_pk_u8_f32 %1, %8, 0, 0\n\t"
            "v_cvt_pk_u8_f32 %2, %12, 0, 0\n\t"
            "v_cvt_pk_u8_f32 %3, %16, 0, 0\n\t"
            "v_cvt_pk_u8_f32 %0, %5, 1, %0\n\t"
            "v_cvt_pk_u8_f32 %1, %9, 1, %1\n\t"
            "v_cvt_pk_u8_f32 %2, %13, 1, %2\n\t"
            "v_cvt_pk_u8_f32 %3, %17, 1, %3\n\t"
            "v_cvt_pk_u8_f32 %0, %6, 2, %0\n\t"
            "v_cvt_pk_u8_f32 %1, %10, 2, %1\n\t"
            "v_cvt_pk_u8_f32 %2, %14, 2, %2\n\t"
            "v_cvt_pk_u8_f32 %3, %18, 2, %3\n\t"
            "v_cvt_pk_u8_f32 %0, %7, 3, %0\n\t"
            "v_cvt_pk_u8_f32 %1, %11, 3, %1\n\t"
            "v_cvt_pk_u8_f32 %2, %15, 3, %2\n\t"
            "v_cvt_pk_u8_f32 %3, %19, 3, %3\n\t"
            "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 0"
            : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3)
            : "v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]), "v"(x[4]), "v"(x[5]), "v"(x[6]), "v"(x[7]), "v"(x[8]), "v"(x[9]), "v"(x[10]),
              "v"(x[11]), "v"(x[12]), "v"(x[13]), "v"(x[14]), "v"(x[15]));
    out[0] = r0;
    out[1] = r1;
    out[2] = r2;
    out[3] = r3;
}

// The value handed to floor_sat_u8x4/8 for one element: quantize_value_folded up to and including
// the + 0.5f, with only the lower bound applied (and only when it is above 0).
// kZeroPoint = false is for a zero point of 0: adding 0.0f changes no value (-0 becomes +0, which the
// next addition would do as well), so the instruction is left out.
template <bool kLowerBound, bool kZeroPoint = true>
__device__ __forceinline__ float quantize_prefloor_u8(float v, const QuantParams& q, float inv_scale, float lo_folded) {
    const float q0 = v * inv_scale;
    const float r = __builtin_fmaf(-q0, q.scale, v);
    float s = __builtin_fmaf(r, inv_scale, q0);
    if (kZeroPoint) s = s + q.zpf;
    if (kLowerBound) s = __builtin_fmaxf(s, lo_folded);
    return s + 0.5f;
}

// dequantize_array, runtime/ops/quantize.cc:37-44: (float(x) - zp) * scale.
// Subtracting 0.0f is exact, so the "skip when zero" needs no branch either.
__device__ __forceinline__ float dequantize_value(int32_t q, float zpf, float scale) {
    float f = (float)q;
    f = f - zpf;
    return f * scale;
}

template <bool kSigned>
__device__ __forceinline__ int32_t byte_of(uint32_t word, int i) {
    const uint32_t b = (word >> (8 * i)) & 0xffu;
    return kSigned ? (int32_t)(int8_t)b : (int32_t)b;
}

__device__ __forceinline__ uint32_t pack4(int32_t a, int32_t b, int32_t c, int32_t d) {
    return ((uint32_t)a & 0xffu) | (((uint32_t)b & 0xffu) << 8) | (((uint32_t)c & 0xffu) << 16) |
           (((uint32_t)d & 0xffu) << 24);
}

// Requantizing epilogue of the contractions: exact int32 accumulator -> 8-bit code.
//   acc (+ bias, ONNX mode)                         int32
//   v = float(acc) * (x_scale * w_scale[oc])        the scales' fp32 product first
//   v = v + float(bias)                             (reference mode: runtime/ops/quantize.cc:93)
//   code = quantize_value(v);  code = max(code, relu_floor)
struct RequantParams {
    QuantParams q;
    float x_scale;
    int32_t bias_mode;   // 0 none, 1 reference float, 2 ONNX int32
    int32_t relu_floor;  // y_zero_point when Relu is fused, else INT32_MIN
};

enum { kBiasNone = 0, kBiasReferenceFloat = 1, kBiasOnnxInt32 = 2 };

template <bool kRne>
__device__ __forceinline__ int32_t requantize_value(int32_t acc, float w_scale, int32_t bias, const RequantParams& rp) {
    if (rp.bias_mode == kBiasOnnxInt32) acc += bias;
    const float s = rp.x_scale * w_scale;
    float v = (float)acc * s;
    if (rp.bias_mode == kBiasReferenceFloat) v = v + (float)bias;
    const int32_t code = quantize_value<kRne>(v, rp.q);
    return code < rp.relu_floor ? rp.relu_floor : code;
}

}  // namespace chx
