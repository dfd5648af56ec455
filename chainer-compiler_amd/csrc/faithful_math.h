// fp32 exp and tanh that reproduce the host C library bit for bit.
//
// On the CPU a fused group runs as separate ChxVM ops, and ChainerX's native Tanh
// and Exp kernels call std::tanh / std::exp on float, i.e. the C library's tanhf and
// expf.  Inside a chain (tanh(..) * sigmoid(..) + x) a one-ulp difference in a
// transcendental survives cancellation as a large relative error, so the device
// code does not approximate these functions on its own terms: it carries out the
// same sequence of IEEE operations as the C library the oracle runs on
// (GNU libc 2.35, x86-64):
//   expf   the table-driven double-precision algorithm of Szabolcs Nagy's
//          optimized routines (glibc sysdeps/ieee754/flt-32/e_expf.c): N = 32 table
//          entries of 2^(i/N), a cubic in double, one final rounding to float.
//   tanhf  the fdlibm algorithm (Sun Microsystems; glibc
//          sysdeps/ieee754/flt-32/s_tanhf.c) on top of fdlibm's expm1f
//          (s_expm1f.c), all in fp32.
// Every operation below is a single correctly rounded IEEE operation; the file
// must be compiled with floating-point contraction off, except where an explicit
// fma is written.  tests/test_faithful_math.py checks the host build of this very
// header against the C library over all 2^32 inputs, and the device build against
// the host build.
//
// The header has no includes so that it can be handed to the run-time compiler as
// text; FM_FN supplies the function qualifiers.
#pragma once

#ifndef FM_FN
#define FM_FN inline
#endif

// FM_ANY_LANE(c): c for the calling lane; the run-time compiled device code defines it as "c holds for some lane
// of the wavefront", which turns the rare-case tests below into branches that a wavefront takes as a whole.  A
// guarded path therefore has to be right for every lane, not only for those with c (it is the complete routine;
// the path behind it is the routine without the cases that c excludes).  Data-dependent branches cost this code far
// more than their instruction count: expf alone over 2^26 floats takes 124 us with the per-lane test and 93 us without.
#ifndef FM_ANY_LANE
#define FM_ANY_LANE(c) (c)
#endif

namespace chx_fm {

typedef unsigned int fm_u32;
typedef unsigned long long fm_u64;
typedef int fm_i32;
typedef fm_u32 fm_u32x2 __attribute__((vector_size(8)));  // a 64-bit pattern as (low, high) words

FM_FN fm_u32 f2u(float f) {
    return __builtin_bit_cast(fm_u32, f);
}
FM_FN float u2f(fm_u32 u) {
    return __builtin_bit_cast(float, u);
}
FM_FN fm_u64 d2u(double d) {
    return __builtin_bit_cast(fm_u64, d);
}
FM_FN double u2d(fm_u64 u) {
    return __builtin_bit_cast(double, u);
}

// tab[i] = bits(2^(i/32)) - (i << 47)
#ifdef FM_TABLE_QUALIFIER
FM_TABLE_QUALIFIER
#else
static const
#endif
fm_u64 kExp2fTab[32] = {
        0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
        0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
        0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
        0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
        0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
        0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
        0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
        0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull,
};

// n / d for the three divisions of tanhf and the sigmoid below.  On the device (FM_DEVICE_DIV) it is the
// reciprocal instruction, one multiplication and two fused multiply-adds: q = n * rcp(d), then one correction
// by the exact remainder, q + (n - d*q) * rcp(d).  That is 4 instructions where the compiler's IEEE division
// takes 11 (operand scaling, a refined reciprocal, two corrections, special-case fix-up).  It is not a correctly
// rounded quotient for every pair of floats, and it has no range handling (d must be normal and finite, the
// quotient and n * rcp(d) neither overflowing nor denormal); it is used only where the callers' operands stay
// in range, and what makes it valid there is the test that compares tanhf and the sigmoid built on it with the
// C library over every one of the 2^32 arguments on the device (tests/test_gpu_elementwise.py).  The host build
// divides.
FM_FN float div_in_range(float n, float d) {
#ifdef FM_DEVICE_DIV
    const float r = __builtin_amdgcn_rcpf(d);
    const float q = n * r;
    const float rem = __builtin_fmaf(-d, q, n);
    return __builtin_fmaf(rem, r, q);
#else
    return n / d;
#endif
}

// expf.  kUseFma selects the operation grouping of the C library build that is
// dispatched on x86-64 CPUs with FMA3: there the compiler contracted the reduction
// r = InvLn2N*x - kd into one fused multiply-add (and the cubic's multiply-adds,
// which changes no result).  Without it every multiply and add rounds on its own.
// Over all 2^32 inputs the two groupings differ on exactly two, 0x4202422f and
// 0xc27c65d9, which is how a host's variant can be told.
// kNegate evaluates expf(-x) (the sigmoid's use) without spending an instruction on the sign.
// (kd as one fused multiply-add and the cubic in Horner form also give the library's result for
// every argument, but the device compiler spends more on placing their constants than they save.)
//
// The library tests the top 12 bits for |x| >= 88 or NaN (expf_far) and decides those arguments before the
// arithmetic.  Here the arithmetic (expf_arith) runs for every lane (for such arguments on meaningless operands,
// which it tolerates: the table index is masked, nothing traps) and the decided values replace its result
// afterwards (expf_decided).
FM_FN bool expf_far(float x) {
    return !(__builtin_fabsf(x) < 88.0f);
}

template <bool kUseFma, bool kNegate>
FM_FN float expf_arith(float x) {
    const double xd = kNegate ? -(double)x : (double)x;
    const double InvLn2N = 0x1.71547652b82fep+0 * 32.0;
    const double Shift = 0x1.8p+52;
    const double C0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0;
    const double C1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0;
    const double C2 = 0x1.62e42ff0c52d6p-1 / 32.0;
    double z = InvLn2N * xd;
    double kd = z + Shift;
    const fm_u64 ki = d2u(kd);
    kd = kd - Shift;
    const double r = kUseFma ? __builtin_fma(InvLn2N, xd, -kd) : z - kd;
    // t + (ki << 47): the sum only reaches the upper half, as (low word of ki) << 15
    const fm_u64 t = kExp2fTab[ki & 31];
    fm_u32x2 tw = __builtin_bit_cast(fm_u32x2, t);
    tw[1] += (fm_u32)ki << 15;
    const double s = __builtin_bit_cast(double, tw);
    double y;
    if (kUseFma) {
        // not fused, although the library's build fuses it: the result is the same for every argument, and a fused
        // multiply-add with two constant operands makes the device compiler copy one of them into registers first
        z = C0 * r + C1;
        const double r2 = r * r;
        y = __builtin_fma(C2, r, 1.0);
        y = __builtin_fma(z, r2, y);
    } else {
        z = C0 * r + C1;
        const double r2 = r * r;
        y = C2 * r + 1.0;
        y = z * r2 + y;
    }
    y = y * s;
    return (float)y;
}

template <bool kNegate>
FM_FN float expf_decided(float x, float res) {
    const float v = kNegate ? -x : x;
    float sp = v > 0.0f ? u2f(0x7f800000u) : 0.0f;   // overflow beyond 0x1.62e42ep6, underflow below -0x1.9fe368p6, +-inf
    sp = (f2u(v) & 0x7fffffffu) > 0x7f800000u ? v + v : sp;  // NaN
    const bool decided = expf_far(x) && (v > 0x1.62e42ep6f || v < -0x1.9fe368p6f || (f2u(v) & 0x7fffffffu) > 0x7f800000u);
    return decided ? sp : res;
}

template <bool kUseFma, bool kNegate = false>
FM_FN float expf_faithful(float x) {
    float res = expf_arith<kUseFma, kNegate>(x);
    if (__builtin_expect(FM_ANY_LANE(expf_far(x)), 0)) res = expf_decided<kNegate>(x, res);
    return res;
}

// The same for callers that evaluate several elements before they branch: the result is the library's unless `rare`
// comes back set, in which case the caller evaluates the element again with expf_faithful.
template <bool kUseFma, bool kNegate = false>
FM_FN float expf_unless_rare(float x, bool& rare) {
    rare = rare || expf_far(x);
    return expf_arith<kUseFma, kNegate>(x);
}

// expm1f, fdlibm.
FM_FN float expm1f_faithful(float x) {
    const float one = 1.0f, huge = 1.0e+30f, tiny = 1.0e-30f;
    const float o_threshold = u2f(0x42b17180u);
    const float ln2_hi = u2f(0x3f317180u);
    const float ln2_lo = u2f(0x3717f7d1u);
    const float invln2 = u2f(0x3fb8aa3bu);
    const float Q1 = u2f(0xbd088889u);
    const float Q2 = u2f(0x3ad00d01u);
    const float Q3 = u2f(0xb8a670cdu);
    const float Q4 = u2f(0x36867e54u);
    const float Q5 = u2f(0xb457edbbu);

    float y, hi, lo, c = 0.0f, t, e, hxs, hfx, r1;
    fm_i32 k;
    fm_u32 hx = f2u(x);
    const fm_u32 xsb = hx & 0x80000000u;
    hx &= 0x7fffffffu;

    if (hx >= 0x4195b844u) {      // |x| >= 27 ln2
        if (hx >= 0x42b17218u) {  // |x| >= 88.721...
            if (hx > 0x7f800000u) return x + x;
            if (hx == 0x7f800000u) return xsb == 0 ? x : -1.0f;
            if (x > o_threshold) return huge * huge;
        }
        if (xsb != 0) return tiny - one;
    }

    if (hx > 0x3eb17218u) {       // |x| > 0.5 ln2
        if (hx < 0x3F851592u) {   // |x| < 1.5 ln2
            if (xsb == 0) {
                hi = x - ln2_hi;
                lo = ln2_lo;
                k = 1;
            } else {
                hi = x + ln2_hi;
                lo = -ln2_lo;
                k = -1;
            }
        } else {
            k = (fm_i32)(invln2 * x + (xsb == 0 ? 0.5f : -0.5f));
            t = (float)k;
            hi = x - t * ln2_hi;
            lo = t * ln2_lo;
        }
        x = hi - lo;
        c = (hi - x) - lo;
    } else if (hx < 0x33000000u) {  // |x| < 2^-25
        t = huge + x;
        return x - (t - (huge + x));
    } else {
        k = 0;
    }

    hfx = 0.5f * x;
    hxs = x * hfx;
    r1 = one + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
    t = 3.0f - r1 * hfx;
    e = hxs * ((r1 - t) / (6.0f - x * t));
    if (k == 0) return x - (x * e - hxs);
    e = (x * (e - c) - c);
    e -= hxs;
    if (k == -1) return 0.5f * (x - e) - 0.5f;
    if (k == 1) {
        if (x < -0.25f) return -2.0f * (e - (x + 0.5f));
        return one + 2.0f * (x - e);
    }
    if (k <= -2 || k > 56) {
        y = one - (e - x);
        y = u2f(f2u(y) + ((fm_u32)k << 23));
        return y - one;
    }
    if (k < 23) {
        t = u2f(0x3f800000u - (0x1000000u >> k));  // 1 - 2^-k
        y = t - (e - x);
        y = u2f(f2u(y) + ((fm_u32)k << 23));
    } else {
        t = u2f((fm_u32)(0x7f - k) << 23);  // 2^-k
        y = x - (e + t);
        y += one;
        y = u2f(f2u(y) + ((fm_u32)k << 23));
    }
    return y;
}

// tanhf, fdlibm, written without data-dependent branches so that a 64-wide wavefront
// does not serialise the algorithm's many cases: every lane evaluates the one shared
// expm1f core (argument reduction, polynomial, one division) on the argument its case
// calls for, the reconstruction formulas, and selects:
//   |x| >= 1 : t = expm1f( 2|x|), z = 1 - 2/(t+2)      (k = 3..63 in expm1f)
//   |x| <  1 : t = expm1f(-2|x|), z = -t/(t+2)         (k = 0, -1, -2, -3)
// with k*ln2_hi == +-ln2_hi exactly for k == +-1 and hi == x, lo == 0 for k == 0, so the
// reduction needs no case split either.
//
// Where fdlibm's operation sequence can be shortened without changing the result for any of the
// 2^32 arguments, it is: the checks named in the header comment compare this function with the C
// library's tanhf over all of them, on the host and on the device, and each of the following was
// added only after that comparison came out equal (and others were dropped because it did not:
// contracting r1, t3, the divisor or e2 changes between 70 and 118718 results):
//  * k = trunc(invln2*arg +- 0.5) as one fused multiply-add, and without expm1f's special cases
//    for |arg| < 1.5 ln2 (k = +-1) and |arg| <= 0.5 ln2 (k = 0): the formula gives the same k;
//  * hi = arg - k*ln2_hi contracted (k*ln2_hi is exact, so this cannot round differently), the
//    four inner steps of the polynomial contracted, 0.5*(x - e) - 0.5 contracted (the product is
//    exact);
//  * for k == 0 the correction c is 0 and fdlibm's x - (x*e - hxs) is -(e2 - x) of the general
//    path, operation for operation;
//  * one reconstruction 2^k * (tb - (e - x)) with tb = 1 - 2^-k (1 where 2^-k is below half an ulp
//    of 1, i.e. k > 24, and for k < 0), minus 1 for negative k.  That is fdlibm's formula for
//    k <= -2 and for 1 < k < 23.  For k >= 23 fdlibm adds 2^-k last instead of first, or leaves it
//    out (k > 56); there t is above 2^22 and 1 - 2/(t+2) does not resolve the difference;
//  * |x| >= 22 and +-inf through the same arithmetic, the argument limited to 88 (k = 127, t about
//    2^127, z = 1 exactly) instead of a select at the end;
//  * |x| < 2^-55 (fdlibm: x*(1+x)), +-0 and expm1f's |arg| < 2^-25 through the general path, which
//    returns the argument itself there; only NaN is selected separately.
FM_FN float tanhf_faithful(float x) {
    const float one = 1.0f, two = 2.0f;
    const float ln2_hi = u2f(0x3f317180u);
    const float ln2_lo = u2f(0x3717f7d1u);
    const float invln2 = u2f(0x3fb8aa3bu);
    const float Q1 = u2f(0xbd088889u);
    const float Q2 = u2f(0x3ad00d01u);
    const float Q3 = u2f(0xb8a670cdu);
    const float Q4 = u2f(0x36867e54u);
    const float Q5 = u2f(0xb457edbbu);

    const fm_u32 ix = f2u(x) & 0x7fffffffu;
    const float ax = u2f(ix);
    const bool big = ix >= 0x3f800000u;  // |x| >= 1
    const float arg = __builtin_fminf(big ? two * ax : -two * ax, 88.0f);

    // expm1f(arg)
    const fm_i32 k = (fm_i32)__builtin_fmaf(invln2, arg, big ? 0.5f : -0.5f);
    const float tk = (float)k;
    const float hi = __builtin_fmaf(-tk, ln2_hi, arg);
    const float lo = tk * ln2_lo;
    const float xr = hi - lo;
    const float c = (hi - xr) - lo;
    const float hfx = 0.5f * xr;
    const float hxs = xr * hfx;
    float p = __builtin_fmaf(hxs, Q5, Q4);
    p = __builtin_fmaf(hxs, p, Q3);
    p = __builtin_fmaf(hxs, p, Q2);
    p = __builtin_fmaf(hxs, p, Q1);
    const float r1 = one + hxs * p;
    const float t3 = 3.0f - r1 * hfx;
    // 6 - xr*t3 is within a few percent of 6 and r1 - t3 of -2 (xr is the reduced argument, |xr| <= 0.35)
    const float e = hxs * div_in_range(r1 - t3, 6.0f - xr * t3);
    float e2 = (xr * (e - c) - c);
    e2 -= hxs;
    const float emx = e2 - xr;
    const fm_u32 sh = (fm_u32)k < 31u ? (fm_u32)k : 31u;  // negative k: 31, tb = 1
    const float tb = u2f(0x3f800000u - (0x1000000u >> sh));
    float y = tb - emx;
    y = u2f(f2u(y) + ((fm_u32)k << 23));
    float t = big ? y : y - one;
    t = k == -1 ? __builtin_fmaf(-0.5f, emx, -0.5f) : t;
    t = k == 0 ? -emx : t;

    // |x| >= 1: 2 / (t + 2) with t = expm1(2|x|) in [6.3, 2^127]; |x| < 1: t / (t + 2) with t in (-0.87, 0] and
    // t + 2 in (1.13, 2]
    const float q = div_in_range(big ? two : t, t + two);
    const float z = big ? one - q : -q;  // z >= 0
    const float r = __builtin_copysignf(z, x);
    return ix > 0x7f800000u ? x : r;  // NaN
}

// ChainerX's Sigmoid routine as the oracle restates it: Reciprocal(1 + Exp(-x)),
// one rounding per operation.
template <bool kUseFma>
FM_FN float sigmoid_faithful(float x) {
    const float e = expf_faithful<kUseFma, true>(x);
    const float d = 1.0f + e;
    // d >= 1; beyond 2^125 (x < -86.6) the reciprocal approaches the denormal range and the plain division takes over
    if (__builtin_expect(FM_ANY_LANE(d > 0x1p125f), 0)) return 1.0f / d;
    return div_in_range(1.0f, d);
}

// As expf_unless_rare: valid unless `rare` comes back set.
template <bool kUseFma>
FM_FN float sigmoid_unless_rare(float x, bool& rare) {
    const float e = expf_unless_rare<kUseFma, true>(x, rare);
    const float d = 1.0f + e;
    rare = rare || d > 0x1p125f;
    return div_in_range(1.0f, d);
}

}  // namespace chx_fm
