/*
 * CPU oracle for the quantized-inference path of chainer-compiler's ChxVM.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the GPU kernels are
 * compared against and the "restated reference CPU path" that the benchmark
 * times next to them.  Nothing in the shipped library links, loads or calls it.
 *
 * Every function restates, in plain C and in the reference's own operation
 * order, what the reference computes through ChainerX's native (CPU) device.
 * Citations are relative to the chainer-compiler source tree.
 *
 * Parity status of each function (what pins it is in tests/test_oracle_*.py):
 *   orc_quantize_linear      pinned: ONNX node-test vector test_quantizelinear,
 *                            brute force vs an independent numpy restatement,
 *                            monotonicity / range / Q(DQ(q))==q invariants.
 *   orc_dequantize_linear    pinned: test_dequantizelinear vector, exhaustive
 *                            over the 256 codes.
 *   orc_matmul_integer       pinned: test_matmulinteger vector + int64 einsum.
 *   orc_conv_integer         pinned: test_basic_convinteger,
 *                            test_convinteger_with_padding + int64 brute force.
 *   orc_qlinear_conv_int     pinned: test_qlinearconv vector, equality with
 *   orc_qlinear_matmul_int   orc_*_literal on the power-of-two-scale family
 *                            (where both are provably identical), and
 *                            test_qlinearmatmul_2D/3D vectors.
 *   orc_qlinear_conv_literal PARITY UNPINNED for the fp32 summation order: the
 *   orc_qlinear_matmul_literal  order used here (k = (c,kh,kw) sequential, fp32
 *                            accumulate) is ChainerX's BLAS-less native Dot as
 *                            recalled; ChainerX is not vendored in the reference
 *                            tree and a BLAS build changes the order.  Used for
 *                            reporting and for CPU timing only, never as a gate.
 *   orc_sigmoid_f32          PARITY UNPINNED for the formula 1/(1+exp(-x)):
 *                            ChainerX's Sigmoid routine is not in the tree.
 *   orc_tanh_f32/orc_exp_f32 call the host libm, as std::tanh/std::exp do in
 *                            ChainerX's native kernels.
 *   orc_max_pool_f32         pinned: numpy restatement over an explicitly padded array (pads, strides,
 *                            cover_all, whole-image window).
 *   orc_average_pool_f32     pinned like orc_average_pool_q8 (tap-major numpy loop, both pad-count modes,
 *                            integer-valued images where every sum is exact, the whole-image window against
 *                            a sequential running sum); the same PARITY UNPINNED remainder.
 *   orc_softmax_f32          pinned against float64 (relative error of a few roundings), rows sum to 1 within
 *                            len roundings, exact shift invariance, both axis semantics against each other;
 *                            PARITY UNPINNED for the sequence max / exp / ascending sum / multiply by the
 *                            reciprocal: chainerx::Softmax is not in the tree.
 *   orc_conv_f32             pinned against float64 within the bound of a K-term float32 sum, bit for bit on
 *                            integer-valued operands (groups, strides, pads), against orc_gemm_f32 on the
 *                            explicitly expanded matrix; PARITY UNPINNED for the order (c, kh, kw):
 *                            chainerx::Conv is not in the tree.
 *   orc_fixed_batch_norm_f32 pinned against float64 (error bound of its five roundings) and bit for bit on
 *                            operands for which every step is exact (power-of-two deviations and scales);
 *                            PARITY UNPINNED for the order of its operations: chainerx::FixedBatchNorm is not
 *                            in the tree.
 *   orc_gemm_f32             pinned for everything but the order of the fp32 sum:
 *                            float64 numpy within a bound from the row norms,
 *                            bit-equal on integer-valued operands (every sum
 *                            exact), the alpha/beta/c branches one by one, a
 *                            row against a sequential float32 running sum.
 *                            PARITY UNPINNED for the order (ascending k):
 *                            ChainerX's Dot is not in the tree.
 *   orc_max_pool_q8          pinned: numpy restatement over an explicitly padded
 *                            array (both types, cover_all, pads, whole-image
 *                            window), and the three float ops spelled out
 *                            (DequantizeLinear, maximum over a -inf padded
 *                            tensor, QuantizeLinear) for uint8 and int8.
 *   orc_average_pool_q8      pinned: numpy restatement (tap-major loop over a
 *                            zero-padded float tensor, both pad-count modes,
 *                            both roundings, all four type pairs), the exact
 *                            family (power-of-two scales: integer arithmetic
 *                            fixes the mean), constant images, and the
 *                            whole-image window against a sequential float32
 *                            running sum.  What stays PARITY UNPINNED is only
 *                            that ChainerX's kernel sums in (kh, kw) order and
 *                            divides by the count (its source is not in the
 *                            tree); the tests show the order matters.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 1;

/* Number of OpenMP threads used by the heavy loops (1 = the reference's
 * single-threaded native device). */
void orc_set_threads(int n) {
    g_threads = n < 1 ? 1 : n;
}

int orc_get_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

enum { ORC_ROUND_REFERENCE = 0, ORC_ROUND_ONNX_RNE = 1 };
enum { ORC_BIAS_NONE = 0, ORC_BIAS_REFERENCE_FLOAT = 1, ORC_BIAS_ONNX_INT32 = 2 };

/* ------------------------------------------------------------------------- */
/* quantize_array: runtime/ops/quantize.cc:16-35.
 *   scaled = y / y_scale;  if (zp != 0) scaled += zp;
 *   out    = AsType( Maximum(lo, Minimum(scaled, hi)) + 0.5f )
 * AsType is a C cast (truncation toward zero).  Every step is one fp32
 * operation, so a one-pass loop gives the same bits as ChainerX's six passes.
 * ORC_ROUND_ONNX_RNE is the ONNX operator text instead:
 *   saturate(round_half_even(y / y_scale) + zp). */
static inline int32_t quantize_one(float v, float y_scale, int32_t zp, float lo, float hi, int round_mode) {
    volatile float scaled = v / y_scale;
    if (round_mode == ORC_ROUND_ONNX_RNE) {
        float r = rintf(scaled) + (float)zp;
        r = r < hi ? r : hi;
        r = lo < r ? r : lo;
        return (int32_t)r;
    }
    float s = scaled;
    if (zp != 0) s = s + (float)zp;
    /* Minimum(scaled, hi) then Maximum(lo, .) */
    s = s < hi ? s : hi;
    s = lo < s ? s : lo;
    s = s + 0.5f;
    return (int32_t)s; /* in range by construction, so int32 trunc == uint8/int8 trunc */
}

void orc_quantize_linear(
        const float* x, int64_t n, float y_scale, int32_t zp, int out_is_int8, int round_mode, void* y) {
    const float lo = out_is_int8 ? -128.f : 0.f;
    const float hi = out_is_int8 ? 127.f : 255.f;
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < n; ++i) {
        int32_t q = quantize_one(x[i], y_scale, zp, lo, hi, round_mode);
        if (out_is_int8)
            ((int8_t*)y)[i] = (int8_t)q;
        else
            ((uint8_t*)y)[i] = (uint8_t)q;
    }
}

/* The reference really runs this as separate element-wise passes with a
 * temporary after each one; this variant does the same and exists only so the
 * CPU timing has the reference's memory traffic. Results equal the one above. */
void orc_quantize_linear_multipass(
        const float* x, int64_t n, float y_scale, int32_t zp, int out_is_int8, float* tmp, void* y) {
    const float lo = out_is_int8 ? -128.f : 0.f;
    const float hi = out_is_int8 ? 127.f : 255.f;
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < n; ++i) tmp[i] = x[i] / y_scale;
    if (zp != 0) {
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
        for (int64_t i = 0; i < n; ++i) tmp[i] = tmp[i] + (float)zp;
    }
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < n; ++i) tmp[i] = tmp[i] < hi ? tmp[i] : hi;
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < n; ++i) tmp[i] = lo < tmp[i] ? tmp[i] : lo;
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < n; ++i) tmp[i] = tmp[i] + 0.5f;
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < n; ++i) {
        if (out_is_int8)
            ((int8_t*)y)[i] = (int8_t)tmp[i];
        else
            ((uint8_t*)y)[i] = (uint8_t)tmp[i];
    }
}

/* dequantize_array: runtime/ops/quantize.cc:37-44.
 *   f = float(x);  if (zp != 0) f -= zp;  return f * scale */
static inline float dequantize_one(int32_t q, float scale, int32_t zp) {
    float f = (float)q;
    if (zp != 0) f = f - (float)zp;
    return f * scale;
}

static inline int32_t load_q(const void* p, int is_i8, int64_t i) {
    return is_i8 ? (int32_t)((const int8_t*)p)[i] : (int32_t)((const uint8_t*)p)[i];
}

void orc_dequantize_linear(const void* x, int x_is_int8, int64_t n, float scale, int32_t zp, float* y) {
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < n; ++i) y[i] = dequantize_one(load_q(x, x_is_int8, i), scale, zp);
}

void orc_dequantize_linear_multipass(const void* x, int x_is_int8, int64_t n, float scale, int32_t zp, float* y) {
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < n; ++i) y[i] = (float)load_q(x, x_is_int8, i);
    if (zp != 0) {
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
        for (int64_t i = 0; i < n; ++i) y[i] = y[i] - (float)zp;
    }
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < n; ++i) y[i] = y[i] * scale;
}

/* ------------------------------------------------------------------------- */
/* MatMulIntegerOp::RunImpl: runtime/ops/quantize.cc:96-114 with NumpyMatMul
 * (runtime/chainerx_util.cc:210-230).  a [batch,M,K], b [batch,K,N] (batch==1
 * for 2-D).  Zero points are subtracted by plain numpy broadcasting, so a 1-D
 * zero point lines up with the LAST axis: a_zp length 0 (absent), 1 or K;
 * b_zp length 0, 1 or N. */
void orc_matmul_integer(
        const void* a, int a_is_int8, const void* b, int b_is_int8, int64_t batch, int64_t M, int64_t K, int64_t N,
        const int32_t* a_zp, int64_t a_zp_len, const int32_t* b_zp, int64_t b_zp_len, int32_t* y) {
#pragma omp parallel for collapse(2) num_threads(g_threads) if (g_threads > 1)
    for (int64_t bt = 0; bt < batch; ++bt) {
        for (int64_t i = 0; i < M; ++i) {
            int32_t* out = y + (bt * M + i) * N;
            for (int64_t j = 0; j < N; ++j) out[j] = 0;
            for (int64_t k = 0; k < K; ++k) {
                int32_t av = load_q(a, a_is_int8, (bt * M + i) * K + k);
                if (a_zp_len == 1) av -= a_zp[0];
                if (a_zp_len > 1) av -= a_zp[k];
                for (int64_t j = 0; j < N; ++j) {
                    int32_t bv = load_q(b, b_is_int8, (bt * K + k) * N + j);
                    if (b_zp_len == 1) bv -= b_zp[0];
                    if (b_zp_len > 1) bv -= b_zp[j];
                    out[j] += av * bv;
                }
            }
        }
    }
}

/* ------------------------------------------------------------------------- */
/* GemmOp::RunImpl, runtime/ops/math.cc:160-177 (and through it LinearOp::RunImpl,
 * runtime/ops/connection.cc:12-15, which is the case trans_b, alpha = beta = 1 with a
 * vector c).  a is [M,K] (or [K,M] when trans_a), b [K,N] (or [N,K] when trans_b), both
 * dense row-major; c is dense [c_rows, c_cols] with each extent 1 or the full one (numpy
 * broadcasting), c == NULL for none.
 *   r = Dot(op(a), op(b));  if (alpha != 1) r *= alpha;  if (beta == 0 || !c) return r;
 *   xc = beta != 1 ? c * beta : c;  return r + xc
 * Dot is a float32 sum in ascending k from 0, one rounding per operation (this file is
 * compiled with -ffp-contract=off). */
void orc_gemm_f32(
        const float* a, const float* b, const float* c, int64_t M, int64_t N, int64_t K, int trans_a, int trans_b, float alpha,
        float beta, int64_t c_rows, int64_t c_cols, float* y) {
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < M; ++i) {
        for (int64_t j = 0; j < N; ++j) {
            float acc = 0.f;
            for (int64_t k = 0; k < K; ++k) {
                const float av = trans_a ? a[k * M + i] : a[i * K + k];
                const float bv = trans_b ? b[j * K + k] : b[k * N + j];
                const float p = av * bv;
                acc = acc + p;
            }
            float r = acc;
            if (alpha != 1.f) r = r * alpha;
            if (c != NULL && beta != 0.f) {
                float xc = c[(c_rows == 1 ? 0 : i) * c_cols + (c_cols == 1 ? 0 : j)];
                if (beta != 1.f) xc = xc * beta;
                r = r + xc;
            }
            y[i * N + j] = r;
        }
    }
}

/* Geometry shared by the convolutions.  Padding follows GroupedConv
 * (runtime/chainerx_util.cc:313-340): explicit begin pads, with an end pad that
 * may differ only when SAME_UPPER auto-padding produced it
 * (CalculateAutoPad, :276-311); the padded border holds zeros of the
 * already zero-point-subtracted / dequantized tensor (ApplyAsymmetricPad :232-274,
 * chainerx::Conv's own zero padding).  out = floor((in + pb + pe - k)/s) + 1. */
typedef struct {
    int64_t N, C, H, W;      /* input NCHW */
    int64_t OC, KH, KW;      /* weight [OC, C/group, KH, KW] */
    int64_t sh, sw;          /* strides */
    int64_t ph0, pw0, ph1, pw1; /* begin / end pads */
    int64_t group;
} orc_conv_geom;

static inline int64_t out_dim(int64_t in, int64_t p0, int64_t p1, int64_t k, int64_t s) {
    return (in + p0 + p1 - k) / s + 1;
}

int64_t orc_conv_out_h(const orc_conv_geom* g) { return out_dim(g->H, g->ph0, g->ph1, g->KH, g->sh); }
int64_t orc_conv_out_w(const orc_conv_geom* g) { return out_dim(g->W, g->pw0, g->pw1, g->KW, g->sw); }

/* CalculateAutoPad, runtime/chainerx_util.cc:276-311 (SAME_UPPER only). */
void orc_same_upper_pads(int64_t in_dim, int64_t stride, int64_t kernel, int64_t* pad_beg, int64_t* pad_end) {
    int64_t legacy_target_size = (in_dim + stride - 1) / stride;
    int64_t pad_needed = (legacy_target_size - 1) * stride + kernel - in_dim;
    *pad_beg = pad_needed / 2;
    *pad_end = pad_needed - *pad_beg;
}

/* ConvIntegerOp::RunImpl: runtime/ops/quantize.cc:116-146.
 *   x32 = int32(x) - x_zp (scalar);  w32 = int32(w) - w_zp (scalar, or per
 *   output channel when 1-D);  GroupedConv in int32;  no bias.
 * Exact integer arithmetic: any summation order gives the same result. */
void orc_conv_integer(
        const void* x, int x_is_int8, const void* w, int w_is_int8, const orc_conv_geom* g, int32_t x_zp,
        const int32_t* w_zp, int64_t w_zp_len, int32_t* y) {
    const int64_t OH = orc_conv_out_h(g), OW = orc_conv_out_w(g);
    const int64_t Cg = g->C / g->group, OCg = g->OC / g->group;
#pragma omp parallel for collapse(2) num_threads(g_threads) if (g_threads > 1)
    for (int64_t n = 0; n < g->N; ++n) {
        for (int64_t oc = 0; oc < g->OC; ++oc) {
            const int64_t grp = oc / OCg;
            const int32_t wz = w_zp_len == 0 ? 0 : (w_zp_len == 1 ? w_zp[0] : w_zp[oc]);
            for (int64_t oh = 0; oh < OH; ++oh) {
                for (int64_t ow = 0; ow < OW; ++ow) {
                    int64_t acc = 0;
                    for (int64_t c = 0; c < Cg; ++c) {
                        const int64_t ic = grp * Cg + c;
                        for (int64_t kh = 0; kh < g->KH; ++kh) {
                            const int64_t ih = oh * g->sh - g->ph0 + kh;
                            if (ih < 0 || ih >= g->H) continue;
                            for (int64_t kw = 0; kw < g->KW; ++kw) {
                                const int64_t iw = ow * g->sw - g->pw0 + kw;
                                if (iw < 0 || iw >= g->W) continue;
                                int32_t xv = load_q(x, x_is_int8, ((n * g->C + ic) * g->H + ih) * g->W + iw) - x_zp;
                                int32_t wv = load_q(w, w_is_int8, ((oc * Cg + c) * g->KH + kh) * g->KW + kw) - wz;
                                acc += (int64_t)xv * wv;
                            }
                        }
                    }
                    y[((n * g->OC + oc) * OH + oh) * OW + ow] = (int32_t)acc;
                }
            }
        }
    }
}

/* ------------------------------------------------------------------------- */
/* QLinearConv, integer-accumulating oracle ("ref_int").
 * QLinearConvOp::RunImpl (runtime/ops/quantize.cc:62-94) dequantizes x and w,
 * convolves in fp32 and re-quantizes.  Mathematically
 *   conv(DQ(x), DQ(w))[oc] = x_scale * w_scale[oc] * sum (x - x_zp)(w - w_zp[oc]),
 * and the sum is what ConvIntegerOp computes exactly.  ref_int evaluates
 *   v = float(acc) * (x_scale * w_scale[oc])      (fp32 product of the scales first)
 * then the bias in the chosen mode, then quantize_array verbatim.
 *   ORC_BIAS_REFERENCE_FLOAT: v + float(b[oc])   (quantize.cc:93 hands the raw
 *       bias array to the fp32 convolution, which adds it unscaled)
 *   ORC_BIAS_ONNX_INT32:      acc + b[oc] before the conversion (the ONNX
 *       operator's definition: bias is int32 with scale x_scale*w_scale). */
static inline int32_t requantize_one(
        int64_t acc, float x_scale, float w_scale, float y_scale, int32_t y_zp, float lo, float hi, int has_bias,
        int32_t bias, int bias_mode, int round_mode) {
    if (has_bias && bias_mode == ORC_BIAS_ONNX_INT32) acc += bias;
    volatile float s = x_scale * w_scale;
    volatile float v = (float)(int32_t)acc * s;
    if (has_bias && bias_mode == ORC_BIAS_REFERENCE_FLOAT) v = v + (float)bias;
    return quantize_one(v, y_scale, y_zp, lo, hi, round_mode);
}

void orc_qlinear_conv_int(
        const void* x, int x_is_int8, float x_scale, int32_t x_zp, const void* w, int w_is_int8, const float* w_scale,
        int64_t w_scale_len, const int32_t* w_zp, const orc_conv_geom* g, float y_scale, int32_t y_zp, int y_is_int8,
        const int32_t* bias, int bias_mode, int round_mode, void* y) {
    const int64_t OH = orc_conv_out_h(g), OW = orc_conv_out_w(g);
    const int64_t total = g->N * g->OC * OH * OW;
    int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)total);
    orc_conv_integer(x, x_is_int8, w, w_is_int8, g, x_zp, w_zp, w_scale_len, acc);
    const float lo = y_is_int8 ? -128.f : 0.f, hi = y_is_int8 ? 127.f : 255.f;
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < total; ++i) {
        const int64_t oc = (i / (OH * OW)) % g->OC;
        const float ws = w_scale_len <= 1 ? w_scale[0] : w_scale[oc];
        int32_t q = requantize_one(
                acc[i], x_scale, ws, y_scale, y_zp, lo, hi, bias != NULL, bias ? bias[oc] : 0, bias_mode, round_mode);
        if (y_is_int8)
            ((int8_t*)y)[i] = (int8_t)q;
        else
            ((uint8_t*)y)[i] = (uint8_t)q;
    }
    free(acc);
}

/* QLinearConv, literal fp32 oracle ("ref_literal"): the reference's op sequence.
 *   x_f = dequantize(x);  w_f[oc] = dequantize(w[oc], w_scale[oc], w_zp[oc])
 *   (quantize.cc:73-88);  im2col + Dot with k = (c, kh, kw) visited in order and
 *   an fp32 accumulator starting from 0;  bias added afterwards as float(b)
 *   (bias_mode REFERENCE_FLOAT) -- ONNX_INT32 mode adds float(b)*(x_scale*w_scale)
 *   so that the two oracles can be compared on the same graph;  quantize_array.
 * `col` scratch is allocated per call like the reference's im2col. */
void orc_qlinear_conv_literal(
        const void* x, int x_is_int8, float x_scale, int32_t x_zp, const void* w, int w_is_int8, const float* w_scale,
        int64_t w_scale_len, const int32_t* w_zp, const orc_conv_geom* g, float y_scale, int32_t y_zp, int y_is_int8,
        const int32_t* bias, int bias_mode, int round_mode, void* y) {
    const int64_t OH = orc_conv_out_h(g), OW = orc_conv_out_w(g);
    const int64_t Cg = g->C / g->group, OCg = g->OC / g->group;
    const int64_t Kdim = Cg * g->KH * g->KW;
    const int64_t xin = g->N * g->C * g->H * g->W;
    const int64_t win = g->OC * Kdim;
    float* xf = (float*)malloc(sizeof(float) * (size_t)xin);
    float* wf = (float*)malloc(sizeof(float) * (size_t)win);
    orc_dequantize_linear_multipass(x, x_is_int8, xin, x_scale, x_zp, xf);
    for (int64_t oc = 0; oc < g->OC; ++oc) {
        const float ws = w_scale_len <= 1 ? w_scale[0] : w_scale[oc];
        const int32_t wz = w_scale_len <= 1 ? w_zp[0] : w_zp[oc];
        for (int64_t k = 0; k < Kdim; ++k) wf[oc * Kdim + k] = dequantize_one(load_q(w, w_is_int8, oc * Kdim + k), ws, wz);
    }
    const float lo = y_is_int8 ? -128.f : 0.f, hi = y_is_int8 ? 127.f : 255.f;
#pragma omp parallel num_threads(g_threads) if (g_threads > 1)
    {
        float* col = (float*)malloc(sizeof(float) * (size_t)Kdim);
#pragma omp for collapse(2)
        for (int64_t n = 0; n < g->N; ++n) {
            for (int64_t p = 0; p < OH * OW; ++p) {
                const int64_t oh = p / OW, ow = p % OW;
                for (int64_t grp = 0; grp < g->group; ++grp) {
                    /* im2col row for this output position and group */
                    for (int64_t c = 0; c < Cg; ++c) {
                        const int64_t ic = grp * Cg + c;
                        for (int64_t kh = 0; kh < g->KH; ++kh) {
                            const int64_t ih = oh * g->sh - g->ph0 + kh;
                            for (int64_t kw = 0; kw < g->KW; ++kw) {
                                const int64_t iw = ow * g->sw - g->pw0 + kw;
                                float v = 0.f;
                                if (ih >= 0 && ih < g->H && iw >= 0 && iw < g->W)
                                    v = xf[((n * g->C + ic) * g->H + ih) * g->W + iw];
                                col[(c * g->KH + kh) * g->KW + kw] = v;
                            }
                        }
                    }
                    for (int64_t j = 0; j < OCg; ++j) {
                        const int64_t oc = grp * OCg + j;
                        const float* wr = wf + oc * Kdim;
                        float v = 0.f;
                        for (int64_t k = 0; k < Kdim; ++k) {
                            float prod = col[k] * wr[k];
                            v = v + prod;
                        }
                        if (bias) {
                            if (bias_mode == ORC_BIAS_REFERENCE_FLOAT) v = v + (float)bias[oc];
                            if (bias_mode == ORC_BIAS_ONNX_INT32) {
                                const float ws = w_scale_len <= 1 ? w_scale[0] : w_scale[oc];
                                volatile float s = x_scale * ws;
                                volatile float bf = (float)bias[oc] * s;
                                v = v + bf;
                            }
                        }
                        int32_t q = quantize_one(v, y_scale, y_zp, lo, hi, round_mode);
                        const int64_t o = ((n * g->OC + oc) * OH + oh) * OW + ow;
                        if (y_is_int8)
                            ((int8_t*)y)[o] = (int8_t)q;
                        else
                            ((uint8_t*)y)[o] = (uint8_t)q;
                    }
                }
            }
        }
        free(col);
    }
    free(xf);
    free(wf);
}

/* ------------------------------------------------------------------------- */
/* QLinearMatMul.  Not a ChxVM op: ReplaceQLinearMatMul
 * (compiler/simplifier.cc:675-694) rewrites it to
 *   DequantizeLinear(a), DequantizeLinear(b) -> MatMul (fp32) -> QuantizeLinear.
 * Per-tensor scales/zero points only (they are scalars in that rewrite).
 * The integer oracle follows the same reasoning as orc_qlinear_conv_int; an
 * optional int32 bias (ONNX accumulator mode) and a fused Relu
 * (Q(Relu(DQ(q))) == max(q, y_zp)) cover the MLP configuration. */
void orc_qlinear_matmul_int(
        const void* a, int a_is_int8, float a_scale, int32_t a_zp, const void* b, int b_is_int8, float b_scale,
        int32_t b_zp, int64_t batch, int64_t M, int64_t K, int64_t N, float y_scale, int32_t y_zp, int y_is_int8,
        const int32_t* bias, int relu, int round_mode, void* y) {
    int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)(batch * M * N));
    orc_matmul_integer(a, a_is_int8, b, b_is_int8, batch, M, K, N, &a_zp, 1, &b_zp, 1, acc);
    const float lo = y_is_int8 ? -128.f : 0.f, hi = y_is_int8 ? 127.f : 255.f;
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < batch * M * N; ++i) {
        const int64_t j = i % N;
        int32_t q = requantize_one(
                acc[i], a_scale, b_scale, y_scale, y_zp, lo, hi, bias != NULL, bias ? bias[j] : 0, ORC_BIAS_ONNX_INT32,
                round_mode);
        if (relu && q < y_zp) q = y_zp;
        if (y_is_int8)
            ((int8_t*)y)[i] = (int8_t)q;
        else
            ((uint8_t*)y)[i] = (uint8_t)q;
    }
    free(acc);
}

void orc_qlinear_matmul_literal(
        const void* a, int a_is_int8, float a_scale, int32_t a_zp, const void* b, int b_is_int8, float b_scale,
        int32_t b_zp, int64_t batch, int64_t M, int64_t K, int64_t N, float y_scale, int32_t y_zp, int y_is_int8,
        int round_mode, void* y) {
    float* af = (float*)malloc(sizeof(float) * (size_t)(batch * M * K));
    float* bf = (float*)malloc(sizeof(float) * (size_t)(batch * K * N));
    float* yf = (float*)malloc(sizeof(float) * (size_t)(batch * M * N));
    orc_dequantize_linear_multipass(a, a_is_int8, batch * M * K, a_scale, a_zp, af);
    orc_dequantize_linear_multipass(b, b_is_int8, batch * K * N, b_scale, b_zp, bf);
    /* native Dot: for i, for k, for j: out[i,j] += a[i,k] * b[k,j] */
#pragma omp parallel for collapse(2) num_threads(g_threads) if (g_threads > 1)
    for (int64_t bt = 0; bt < batch; ++bt) {
        for (int64_t i = 0; i < M; ++i) {
            float* out = yf + (bt * M + i) * N;
            for (int64_t j = 0; j < N; ++j) out[j] = 0.f;
            for (int64_t k = 0; k < K; ++k) {
                const float av = af[(bt * M + i) * K + k];
                const float* br = bf + (bt * K + k) * N;
                for (int64_t j = 0; j < N; ++j) {
                    float prod = av * br[j];
                    out[j] = out[j] + prod;
                }
            }
        }
    }
    orc_quantize_linear(yf, batch * M * N, y_scale, y_zp, y_is_int8, round_mode, y);
    free(af);
    free(bf);
    free(yf);
}

/* ------------------------------------------------------------------------- */
/* Element-wise ops a CPU FusionGroup expands to (compiler/chxvm/emitter.cc:697-726
 * inlines the group's nodes as ordinary ChxVM ops): one pass and one rounding
 * per op.  Binary ops take operands whose flat length divides n and index them
 * modulo that length, which covers scalars, last-axis vectors and full arrays.
 *   Add/Sub/Mul: runtime/ops/math.cc:31-41;  Div: the nvrtc builder's '/'
 *   Tanh: runtime/ops/activation.cc:55-57 (chainerx::Tanh -> std::tanh)
 *   Sigmoid: activation.cc:59-61 (chainerx::Sigmoid, recalled as
 *            Reciprocal(1 + Exp(-x)))
 *   Exp: runtime/ops/math.cc:105;  Relu: activation.cc:20-22 (Maximum(0, x))
 *   Clip: math.cc:140-154 (Minimum(Maximum(x, lo), hi)) */
enum { ORC_ADD = 0, ORC_SUB = 1, ORC_MUL = 2, ORC_DIV = 3 };

void orc_binary_f32(int op, const float* a, int64_t a_len, const float* b, int64_t b_len, int64_t n, float* y) {
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < n; ++i) {
        const float av = a[a_len == n ? i : i % a_len];
        const float bv = b[b_len == n ? i : i % b_len];
        float r;
        switch (op) {
            case ORC_ADD: r = av + bv; break;
            case ORC_SUB: r = av - bv; break;
            case ORC_MUL: r = av * bv; break;
            default: r = av / bv; break;
        }
        y[i] = r;
    }
}

void orc_tanh_f32(const float* x, int64_t n, float* y) {
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < n; ++i) y[i] = tanhf(x[i]);
}

void orc_exp_f32(const float* x, int64_t n, float* y) {
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < n; ++i) y[i] = expf(x[i]);
}

void orc_sigmoid_f32(const float* x, int64_t n, float* y) {
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < n; ++i) {
        volatile float e = expf(-x[i]);
        volatile float d = 1.0f + e;
        y[i] = 1.0f / d;
    }
}

/* The generated fused kernel of the reference's GPU path spells sigmoid as
 * tanh(x*0.5)*0.5+0.5 (compiler/nvrtc_builder.cc:132-137).  Kept for reporting
 * how far the two spellings are apart; not a parity gate. */
void orc_sigmoid_tanh_form_f32(const float* x, int64_t n, float* y) {
    for (int64_t i = 0; i < n; ++i) {
        volatile float h = x[i] * 0.5f;
        volatile float t = tanhf(h);
        volatile float m = t * 0.5f;
        y[i] = m + 0.5f;
    }
}

void orc_relu_f32(const float* x, int64_t n, float* y) {
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < n; ++i) y[i] = x[i] < 0.f ? 0.f : x[i];
}

void orc_clip_f32(const float* x, int64_t n, float lo, float hi, float* y) {
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < n; ++i) {
        float v = x[i] < lo ? lo : x[i];
        y[i] = v < hi ? v : hi;
    }
}

/* RoundOp (runtime/ops/quantize.cc:148-151) -> SlowRound
 * (runtime/chainerx_util.cc:397-410): rint in double, cast back. */
void orc_round_f32(const float* x, int64_t n, float* y) {
    for (int64_t i = 0; i < n; ++i) y[i] = (float)rint((double)x[i]);
}


/* ------------------------------------------------------------------------- */
/* Pooling between a DequantizeLinear and a QuantizeLinear, as a quantized network
 * runs it (MaxPoolOp / AveragePoolOp::RunImpl, runtime/ops/pooling.cc:47-75).
 *
 * orc_max_pool_q8: DequantizeLinear -> MaxPool -> QuantizeLinear with the same scale
 * and zero point on both sides is a function of the maximum m of the codes, because the
 * dequantization map is increasing: Q(DQ(m)) == m for uint8 and m + (m < 0) for int8
 * (both checked exhaustively in the tests against the three float operations).  Out-of-image taps never win (ChainerX pads max-pooling with the
 * lowest value); cover_all adds a last window for what floor would leave uncovered
 * (out = ceil((in + p0 + p1 - k) / s) + 1 instead of floor), which with pads can lie in the
 * padding altogether.
 *
 * orc_average_pool_q8: y = Q( (sum over the window of DQ(x)) / count ), the sum taken
 * in fp32 in (kh, kw) order starting from 0; padding taps add 0 and count toward
 * `count` when count_include_pad.  (That ChainerX's AveragePool kernel, which is not
 * in the tree, uses this order and divides by the count is recalled, not verified.) */
static int64_t pool_out_dim(int64_t in, int64_t p0, int64_t p1, int64_t k, int64_t s, int cover_all) {
    if (cover_all) return (in + p0 + p1 - k + s - 1) / s + 1;
    return (in + p0 + p1 - k) / s + 1;
}

int64_t orc_pool_out_dim(int64_t in, int64_t p0, int64_t p1, int64_t k, int64_t s, int cover_all) {
    return pool_out_dim(in, p0, p1, k, s, cover_all);
}

void orc_max_pool_q8(
        const void* x, int x_is_int8, int64_t N, int64_t C, int64_t H, int64_t W, int64_t kh, int64_t kw, int64_t sh,
        int64_t sw, int64_t ph0, int64_t pw0, int64_t ph1, int64_t pw1, int cover_all, void* y) {
    const int64_t OH = pool_out_dim(H, ph0, ph1, kh, sh, cover_all), OW = pool_out_dim(W, pw0, pw1, kw, sw, cover_all);
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t nc = 0; nc < N * C; ++nc) {
        for (int64_t oh = 0; oh < OH; ++oh)
            for (int64_t ow = 0; ow < OW; ++ow) {
                /* a window that lies in the padding altogether (possible with cover_all and pads) has the
                 * lowest float as its maximum, which QuantizeLinear clamps to the lowest code */
                int32_t m = x_is_int8 ? -128 : 0;
                for (int64_t i = 0; i < kh; ++i)
                    for (int64_t j = 0; j < kw; ++j) {
                        const int64_t ih = oh * sh - ph0 + i, iw = ow * sw - pw0 + j;
                        if (ih < 0 || ih >= H || iw < 0 || iw >= W) continue;
                        const int32_t v = load_q(x, x_is_int8, (nc * H + ih) * W + iw);
                        if (v > m) m = v;
                    }
                /* int8: QuantizeLinear adds 0.5 and the cast truncates toward zero (quantize.cc:16-35), so a
                 * negative code q comes back as q + 1: q + 0.5 (give or take the rounding of DQ and the
                 * division, far below 0.5) truncates to q + 1 for q < 0 and to q for q >= 0 */
                if (x_is_int8)
                    ((int8_t*)y)[(nc * OH + oh) * OW + ow] = (int8_t)(m < 0 ? m + 1 : m);
                else
                    ((uint8_t*)y)[(nc * OH + oh) * OW + ow] = (uint8_t)m;
            }
    }
}

/* MaxPoolOp / AveragePoolOp::RunImpl on float32 arrays (runtime/ops/pooling.cc:47-75), NCHW dense.
 * max: padding never wins (a window in the padding altogether gives the lowest finite float, ChainerX's
 * padding value as recalled); cover_all as above.  average: the window's taps in (kh, kw) order, one float32
 * addition each starting from 0, divided by the number of taps that count (all kh*kw with count_include_pad,
 * else those inside the image).  PARITY UNPINNED where orc_average_pool_q8 is: ChainerX's kernels are not in
 * the tree. */
void orc_max_pool_f32(
        const float* x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph0,
        int64_t pw0, int64_t ph1, int64_t pw1, int cover_all, float* y) {
    const int64_t OH = pool_out_dim(H, ph0, ph1, kh, sh, cover_all), OW = pool_out_dim(W, pw0, pw1, kw, sw, cover_all);
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t nc = 0; nc < N * C; ++nc)
        for (int64_t oh = 0; oh < OH; ++oh)
            for (int64_t ow = 0; ow < OW; ++ow) {
                float m = -3.402823466e+38f;
                for (int64_t i = 0; i < kh; ++i)
                    for (int64_t j = 0; j < kw; ++j) {
                        const int64_t ih = oh * sh - ph0 + i, iw = ow * sw - pw0 + j;
                        if (ih < 0 || ih >= H || iw < 0 || iw >= W) continue;
                        const float v = x[(nc * H + ih) * W + iw];
                        if (v > m) m = v;
                    }
                y[(nc * OH + oh) * OW + ow] = m;
            }
}

void orc_average_pool_f32(
        const float* x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph,
        int64_t pw, int count_include_pad, float* y) {
    const int64_t OH = pool_out_dim(H, ph, ph, kh, sh, 0), OW = pool_out_dim(W, pw, pw, kw, sw, 0);
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t nc = 0; nc < N * C; ++nc)
        for (int64_t oh = 0; oh < OH; ++oh)
            for (int64_t ow = 0; ow < OW; ++ow) {
                float sum = 0.f;
                int32_t cnt = 0;
                for (int64_t i = 0; i < kh; ++i)
                    for (int64_t j = 0; j < kw; ++j) {
                        const int64_t ih = oh * sh - ph + i, iw = ow * sw - pw + j;
                        if (ih < 0 || ih >= H || iw < 0 || iw >= W) continue;
                        sum = sum + x[(nc * H + ih) * W + iw];
                        ++cnt;
                    }
                if (count_include_pad) cnt = (int32_t)(kh * kw);
                y[(nc * OH + oh) * OW + ow] = sum / (float)cnt;
            }
}

/* SoftmaxOp::RunImpl, runtime/ops/activation.cc:66-95, on a dense [outer][len][inner] float32 array, reduced over len:
 * m = max, e = expf(x - m) (the host libm, as std::exp in ChainerX's native kernel), s = the sum of e in ascending
 * order from 0, result e * (1 / s); a NaN wins the maximum.  PARITY UNPINNED for this sequence (chainerx::Softmax is
 * not in the tree); pinned against float64, by the rows summing to 1 within len roundings, and by shift invariance
 * where the shift is exact. */
void orc_softmax_f32(const float* x, int64_t outer, int64_t len, int64_t inner, float* y) {
#pragma omp parallel for collapse(2) num_threads(g_threads) if (g_threads > 1)
    for (int64_t o = 0; o < outer; ++o)
        for (int64_t i = 0; i < inner; ++i) {
            const float* xp = x + o * len * inner + i;
            float* yp = y + o * len * inner + i;
            float m = xp[0];
            for (int64_t k = 1; k < len; ++k) {
                const float v = xp[k * inner];
                m = v > m ? v : m;
                m = v != v ? v : m;
            }
            float s = 0.f;
            for (int64_t k = 0; k < len; ++k) {
                const float e = expf(xp[k * inner] - m);
                s = s + e;
            }
            const float r = 1.0f / s;
            for (int64_t k = 0; k < len; ++k) {
                const float e = expf(xp[k * inner] - m);
                yp[k * inner] = e * r;
            }
        }
}

/* ConvOp::RunImpl on float32, runtime/ops/connection.cc:24-30 (GroupedConv, runtime/chainerx_util.cc:313-340):
 * the expanded-matrix product of orc_qlinear_conv_literal without the quantization around it: k = (c, kh, kw) in
 * order, an fp32 accumulator from 0, a tap in the padding as the product 0 * w, the bias added last.
 * PARITY UNPINNED for that order (chainerx::Conv is not in the tree); pinned against float64 within the bound of
 * a K-term float32 sum and bit for bit on integer-valued operands. */
void orc_conv_f32(const float* x, const float* w, const float* bias, const orc_conv_geom* g, float* y) {
    const int64_t OH = orc_conv_out_h(g), OW = orc_conv_out_w(g);
    const int64_t Cg = g->C / g->group, OCg = g->OC / g->group;
    const int64_t Kdim = Cg * g->KH * g->KW;
#pragma omp parallel for collapse(2) num_threads(g_threads) if (g_threads > 1)
    for (int64_t n = 0; n < g->N; ++n)
        for (int64_t oc = 0; oc < g->OC; ++oc) {
            const int64_t grp = oc / OCg;
            const float* wr = w + oc * Kdim;
            for (int64_t oh = 0; oh < OH; ++oh)
                for (int64_t ow = 0; ow < OW; ++ow) {
                    float v = 0.f;
                    for (int64_t c = 0; c < Cg; ++c)
                        for (int64_t kh = 0; kh < g->KH; ++kh) {
                            const int64_t ih = oh * g->sh - g->ph0 + kh;
                            for (int64_t kw = 0; kw < g->KW; ++kw) {
                                const int64_t iw = ow * g->sw - g->pw0 + kw;
                                float xv = 0.f;
                                if (ih >= 0 && ih < g->H && iw >= 0 && iw < g->W) xv = x[((n * g->C + grp * Cg + c) * g->H + ih) * g->W + iw];
                                const float prod = xv * wr[(c * g->KH + kh) * g->KW + kw];
                                v = v + prod;
                            }
                        }
                    if (bias) v = v + bias[oc];
                    y[((n * g->OC + oc) * OH + oh) * OW + ow] = v;
                }
        }
}

/* FixedBatchNormalizationOp::RunImpl, runtime/ops/normalization.cc:210-225, on a contiguous [N, C, inner] float32
 * array: ((x - mean) * (1 / sqrt(var + eps))) * s + bias, one rounding per operation, eps adjusted as the op does
 * (lines 217-218).  PARITY UNPINNED for the order of the operations (chainerx::FixedBatchNorm is not in the tree);
 * pinned against float64 within 4 ulp-sized terms and bit for bit where every step is exact. */
void orc_fixed_batch_norm_f32(
        const float* x, const float* s, const float* bias, const float* mean, const float* var, float epsilon, int64_t N, int64_t C,
        int64_t inner, float* y) {
    const float eps = epsilon <= 1e-5f ? (float)(1e-5 + 1e-12) : epsilon;
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t nc = 0; nc < N * C; ++nc) {
        const int64_t c = nc % C;
        const float ve = var[c] + eps;
        const float sd = sqrtf(ve);
        const float inv_std = 1.0f / sd;
        for (int64_t i = 0; i < inner; ++i) {
            float r = x[nc * inner + i] - mean[c];
            r = r * inv_std;
            r = r * s[c];
            r = r + bias[c];
            y[nc * inner + i] = r;
        }
    }
}

void orc_average_pool_q8(
        const void* x, int x_is_int8, float x_scale, int32_t x_zp, int64_t N, int64_t C, int64_t H, int64_t W, int64_t kh,
        int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw, int count_include_pad, float y_scale, int32_t y_zp,
        int y_is_int8, int round_mode, void* y) {
    const int64_t OH = pool_out_dim(H, ph, ph, kh, sh, 0), OW = pool_out_dim(W, pw, pw, kw, sw, 0);
    const float lo = y_is_int8 ? -128.f : 0.f, hi = y_is_int8 ? 127.f : 255.f;
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
    for (int64_t nc = 0; nc < N * C; ++nc) {
        for (int64_t oh = 0; oh < OH; ++oh)
            for (int64_t ow = 0; ow < OW; ++ow) {
                float sum = 0.f;
                int32_t cnt = 0;
                for (int64_t i = 0; i < kh; ++i)
                    for (int64_t j = 0; j < kw; ++j) {
                        const int64_t ih = oh * sh - ph + i, iw = ow * sw - pw + j;
                        if (ih < 0 || ih >= H || iw < 0 || iw >= W) continue;
                        sum = sum + dequantize_one(load_q(x, x_is_int8, (nc * H + ih) * W + iw), x_scale, x_zp);
                        ++cnt;
                    }
                if (count_include_pad) cnt = (int32_t)(kh * kw);
                volatile float mean = sum / (float)cnt;
                const int32_t q = quantize_one(mean, y_scale, y_zp, lo, hi, round_mode);
                if (y_is_int8)
                    ((int8_t*)y)[(nc * OH + oh) * OW + ow] = (int8_t)q;
                else
                    ((uint8_t*)y)[(nc * OH + oh) * OW + ow] = (uint8_t)q;
            }
    }
}
