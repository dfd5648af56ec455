/*
 * chx_hip.h -- C ABI of the MI355X (gfx950) quantized-inference kernels that sit
 * under chainer-compiler's ChxVM op layer.
 *
 * Every entry point is what a ChxVM op's RunImpl body binds for this path; the
 * reference interface each one replaces is cited as file:line of the
 * chainer-compiler tree.  Plain pointers and sizes only; no C++ or torch types.
 *
 * Conventions
 *   - Return value: 0 on success, a CHX_HIP_E* code otherwise; the message for
 *     the calling thread's last failure is chx_hip_last_error().  No exceptions
 *     cross this boundary and nothing aborts the process (the reference's
 *     CHECK macros do, common/log.h:31-44; the RunImpl wrappers keep that
 *     behaviour by CHECKing the return code).
 *   - Tensors are described by chx_hip_tensor: device pointer, ChainerX dtype
 *     code (compiler/dtype.h:14-25), shape and strides IN BYTES (ChainerX
 *     arrays carry byte strides).  The caller allocates outputs; shape
 *     inference stays in the RunImpl wrappers.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *     Calls only enqueue work; they synchronize with the host where the comment
 *     of an entry point says so and nowhere else.
 *   - Scales and zero points that ChxVM hands over as StrictScalar
 *     (runtime/strict_scalar.h:8-34) are host values here.
 *   - Activations may be given either NCHW-contiguous or as NCHW-shaped views of
 *     channels-last (NHWC) memory; both are valid ChainerX arrays.  Channels-last
 *     is the layout the MFMA kernels read and write without a transposition.
 */
#ifndef CHX_HIP_H_
#define CHX_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CHX_HIP_MAX_NDIM 10 /* chainerx::kMaxNdim */

/* ChainerX dtype codes, compiler/dtype.h:14-25 */
enum {
    CHX_HIP_BOOL = 1,
    CHX_HIP_INT8 = 2,
    CHX_HIP_INT16 = 3,
    CHX_HIP_INT32 = 4,
    CHX_HIP_INT64 = 5,
    CHX_HIP_UINT8 = 6,
    CHX_HIP_FLOAT16 = 7,
    CHX_HIP_FLOAT32 = 8,
    CHX_HIP_FLOAT64 = 9
};

enum {
    CHX_HIP_OK = 0,
    CHX_HIP_EINVAL = 1,      /* bad argument: dtype, shape, stride, null pointer */
    CHX_HIP_EUNSUPPORTED = 2,/* valid for the reference op but not implemented on the device */
    CHX_HIP_ERUNTIME = 3,    /* a HIP / hiprtc call failed */
    CHX_HIP_ECOMPILE = 4,    /* run-time compilation of a fused kernel failed */
    CHX_HIP_EPINNED = 5      /* the call would have to move memory that a recorded run (HIP graph) addresses */
};

/* Behaviour switches.  0 is always the reference's behaviour. */
enum {
    /* rounding of QuantizeLinear and of every requantizing epilogue */
    CHX_HIP_ROUND_REFERENCE = 0u,     /* AsType(clip(v/scale + zp) + 0.5f): runtime/ops/quantize.cc:29-34 */
    CHX_HIP_ROUND_ONNX_RNE = 1u,      /* saturate(round_half_even(v/scale) + zp): the ONNX operator text */
    /* how a QLinearConv bias enters */
    CHX_HIP_BIAS_REFERENCE_FLOAT = 0u,/* float(b) added unscaled to the fp32 result: runtime/ops/quantize.cc:93 */
    CHX_HIP_BIAS_ONNX_INT32 = 2u,     /* b added to the int32 accumulator (scale x_scale*w_scale) */
    /* Q(Relu(DQ(q))) folded into the epilogue: output clamped below at y_zero_point */
    CHX_HIP_FUSE_RELU = 4u,
    /* chx_hip_qconv_plan_run / _run_add / _run_pair only: the result is quantized as uint8 (its zero point is given in
     * the uint8 range) but every byte is stored as code - 128, in an array of dtype int8.  An int8 array with zero point
     * zp - 128 denotes the same numbers, so a later QLinearConv reads it as its int8 x (or a fused residual sum as its
     * int8 r) with that zero point and gives the bytes it would give on the uint8 array, without flipping sign bits in
     * its inner loop.  No counterpart in the reference; a storage convention between the convolutions of one host.
     * CHX_HIP_EUNSUPPORTED where neither the matrix-core kernel nor the depthwise 3x3 kernel runs (store uint8 then). */
    CHX_HIP_STORE_MINUS_128 = 8u
};

typedef struct chx_hip_tensor {
    void* data;                        /* device address of element [0,0,...] */
    int32_t dtype;                     /* CHX_HIP_* dtype code */
    int32_t ndim;
    int64_t shape[CHX_HIP_MAX_NDIM];
    int64_t strides[CHX_HIP_MAX_NDIM]; /* bytes */
} chx_hip_tensor;

/* Convolution attributes after the RunImpl wrapper has completed them
 * (ComplementStride/ComplementPad runtime/chainerx_util.cc:180-200 and
 * CalculateAutoPad :276-311): explicit begin and end pads per spatial axis. */
typedef struct chx_hip_conv_params {
    int32_t stride_h, stride_w;
    int32_t pad_h_begin, pad_w_begin;
    int32_t pad_h_end, pad_w_end;
    int32_t group;
} chx_hip_conv_params;

/* The same for convolutions over 1, 2 or 3 spatial axes (ComplementStride, ComplementPad and GroupedConv are
 * rank-generic, runtime/chainerx_util.cc:180-200,313-340): entry i describes spatial axis i of x, outermost first. */
typedef struct chx_hip_conv_nd_params {
    int32_t n_spatial;
    int32_t stride[3];
    int32_t pad_begin[3];
    int32_t pad_end[3];
    int32_t group;
} chx_hip_conv_nd_params;

typedef struct chx_hip_device_props {
    int32_t compute_units;
    int32_t clock_khz;
    int32_t memory_clock_khz;
    int32_t memory_bus_bits;
    int64_t total_memory;
    char arch[64];
    char name[128];
} chx_hip_device_props;

/* ---- library state ----------------------------------------------------------------- */

/* Selects `device` for the calling thread and checks that it is a gfx950 part.
 * Replaces nothing in the reference (ChainerX owns device selection there,
 * tools/run_onnx.cc:343-357). */
int chx_hip_init(int device);
const char* chx_hip_last_error(void);
const char* chx_hip_version(void);
int chx_hip_get_device_props(chx_hip_device_props* out);

/* Thin device-memory helpers for hosts that have no allocator of their own (the
 * C++ ChxVM runtime mirror uses them where the reference uses chainerx::Empty /
 * Device::MakeDataFromForeignPointer, runtime/chainerx_util.cc:60-120). */
int chx_hip_malloc(void** ptr, size_t bytes);
int chx_hip_free(void* ptr);
int chx_hip_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream); /* synchronizes the stream */
int chx_hip_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream); /* synchronizes the stream */
int chx_hip_memset(void* dst, int value, size_t bytes, void* stream);
int chx_hip_stream_synchronize(void* stream);

/* Streams and captured graphs, for hosts that replay a fixed instruction sequence (the ChxVM runtime
 * mirror captures one run of a program and replays it; nothing in the reference corresponds: its
 * interpreter launches every kernel from the host on the default stream, runtime/chxvm.cc:168-236).
 * A stream from chx_hip_stream_create has the default priority and does not synchronize with the
 * null stream.  Between capture_begin and capture_end the calls of this library on that stream are
 * recorded instead of run; calls that must synchronize, allocate with the device runtime or time
 * kernels are refused by the device runtime, capture_end then fails and leaves no graph. */
int chx_hip_stream_create(void** stream);
int chx_hip_stream_destroy(void* stream);
typedef struct chx_hip_graph chx_hip_graph;
int chx_hip_capture_begin(void* stream);
int chx_hip_capture_end(void* stream, chx_hip_graph** graph);
/* 1 while `stream` records (a null stream never does) */
int chx_hip_stream_is_capturing(void* stream);
int chx_hip_graph_launch(const chx_hip_graph* graph, void* stream);
void chx_hip_graph_destroy(chx_hip_graph* graph);

/* ---- QuantizeLinear / DequantizeLinear ------------------------------------------------ */

/* QuantizeLinearOp::RunImpl -> quantize_array, runtime/ops/quantize.cc:16-35,48-53.
 * x float32; y uint8 or int8 (the dtype the zero point has in the reference),
 * same shape.  One pass: y = cast(max(lo, min(x / y_scale + zp, hi)) + 0.5f). */
int chx_hip_quantize_linear(
        const chx_hip_tensor* x, float y_scale, int32_t y_zero_point, uint32_t flags, chx_hip_tensor* y, void* stream);

/* DequantizeLinearOp::RunImpl -> dequantize_array, runtime/ops/quantize.cc:37-44,55-60.
 * x uint8 or int8; y float32: y = (float(x) - zp) * x_scale. */
int chx_hip_dequantize_linear(
        const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, chx_hip_tensor* y, void* stream);

/* ---- QLinearConv ---------------------------------------------------------------------- */

/* QLinearConvOp::RunImpl, runtime/ops/quantize.cc:62-94 (+ GroupedConv,
 * runtime/chainerx_util.cc:313-340).
 *   x uint8/int8 [N,C,H,W]; w int8/uint8 [OC,C/group,KH,KW]; w_scale float32 0-d or
 *   [OC]; w_zero_point same element count as w_scale, dtype of w; bias int32 [OC] or
 *   NULL; y uint8/int8 [N,OC,OH,OW].
 * The contraction accumulates exactly in int32 and the epilogue evaluates
 *   v = float(acc) * (x_scale * w_scale[oc]);  (+ bias per `flags`);  quantize_array(v)
 * in that fp32 operation order.  Reads w_zero_point back to the host once per call
 * (a stream synchronization) to pick the kernel; use a plan to avoid that. */
int chx_hip_qlinear_conv(
        const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, const chx_hip_tensor* w,
        const chx_hip_tensor* w_scale, const chx_hip_tensor* w_zero_point, float y_scale, int32_t y_zero_point,
        const chx_hip_tensor* bias, const chx_hip_conv_params* params, uint32_t flags, chx_hip_tensor* y, void* stream);

/* QLinearConvOp::RunImpl and ConvIntegerOp::RunImpl (runtime/ops/quantize.cc:62-94,116-146) for x [N,C,L],
 * [N,C,H,W] or [N,C,D,H,W] with w and y of the same rank.  One spatial axis runs as a 2-D convolution over images one
 * pixel high (every kernel of the 2-D entry points); three run on the direct kernel (one lane per output element,
 * exact int32 accumulation, the same requantization). */
int chx_hip_qlinear_conv_nd(
        const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, const chx_hip_tensor* w,
        const chx_hip_tensor* w_scale, const chx_hip_tensor* w_zero_point, float y_scale, int32_t y_zero_point,
        const chx_hip_tensor* bias, const chx_hip_conv_nd_params* params, uint32_t flags, chx_hip_tensor* y, void* stream);
int chx_hip_conv_integer_nd(
        const chx_hip_tensor* x, const chx_hip_tensor* w, int32_t x_zero_point, const chx_hip_tensor* w_zero_point,
        const chx_hip_conv_nd_params* params, chx_hip_tensor* y, void* stream);

/* The same op with the weight-side work (repacking for the MFMA kernel, per-channel
 * sums, the zero-point read-back) done once.  The reference redoes its weight
 * dequantization on every call (runtime/ops/quantize.cc:76-88); a ChxVM op object
 * lives as long as the program, so the wrapper keeps one plan per QLinearConv
 * instruction, in the manner of the stateful backend ops (runtime/ops/tvm.cc:90-158).
 * create() synchronizes the stream; run() does not, and allocates nothing once the plan
 * has seen its largest input (it keeps its own transposition / im2col space), so a
 * sequence of runs can be captured into a HIP graph.  One plan must not be run from two
 * threads or streams at once.  The plan keeps pointers to w_scale and bias: they must
 * stay alive and unchanged. */
typedef struct chx_hip_qconv_plan chx_hip_qconv_plan;
int chx_hip_qconv_plan_create(
        const chx_hip_tensor* w, const chx_hip_tensor* w_scale, const chx_hip_tensor* w_zero_point,
        const chx_hip_tensor* bias, const chx_hip_conv_params* params, void* stream, chx_hip_qconv_plan** plan);
int chx_hip_qconv_plan_run(
        const chx_hip_qconv_plan* plan, const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, float y_scale,
        int32_t y_zero_point, uint32_t flags, chx_hip_tensor* y, void* stream);
/* The launch configurations the plan has measured so far, as text into buf (truncated to buf_size - 1
 * characters): one "M=<output pixels> <OH>x<OW> res=<0|1> tile=<oc>x<px> wgs_per_cu=<n, 0 = as many as fit>"
 * per line (followed by "waves=<4|8>", the wavefronts per work-group), and after a chx_hip_qconv_plan_run_add a line
 * "residual=affine" or "residual=exact" (which arithmetic the fused sum uses, see there); empty for a plan that
 * does not run on the matrix-core kernel or has not run eagerly yet.  No counterpart in the reference; benchmarks
 * report it next to their timings. */
int chx_hip_qconv_plan_describe(const chx_hip_qconv_plan* plan, char* buf, size_t buf_size);
/* Two QLinearConv (QLinearConvOp::RunImpl, runtime/ops/quantize.cc:62-94, twice) that read the same x with the same
 * activation quantization, kernel size, strides and pads, as ONE launch: the main-path and the shortcut convolution
 * of a down-sampling residual block.  The plan is created from both filter sets concatenated along the output
 * channels (w [OC1 + OC2, C, KH, KW]; w_scale, w_zero_point and bias likewise); output channels [0, split) are
 * requantized with (y1_scale, y1_zero_point, flags1) into y1 [N, split, OH, OW], the others with the second set into
 * y2 [N, OC - split, OH, OW].  The bytes are those of the two ops run one after the other; x is read once and one
 * kernel boundary disappears.  flags1 and flags2 may differ in CHX_HIP_FUSE_RELU only.  x, y1 and y2 must not
 * overlap (CHX_HIP_EINVAL).  CHX_HIP_EUNSUPPORTED when split is not a multiple of 64, when the weights do not run on
 * the matrix-core kernel or an operand is not channels-last: the caller then runs two plans. */
int chx_hip_qconv_plan_run_pair(
        const chx_hip_qconv_plan* plan, const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, int32_t split,
        float y1_scale, int32_t y1_zero_point, uint32_t flags1, chx_hip_tensor* y1, float y2_scale, int32_t y2_zero_point,
        uint32_t flags2, chx_hip_tensor* y2, void* stream);
/* A QLinearConv (QLinearConvOp::RunImpl, runtime/ops/quantize.cc:62-94) whose only reader is the
 * element-wise group  QuantizeLinear(act(DequantizeLinear(y) + DequantizeLinear(r)))  of a
 * residual block (ElementWiseNvrtcOp::RunImpl, runtime/ops/nvrtc.cc:90-161, act = Relu or
 * nothing), run as one kernel: the convolution's 8-bit result y (type y_dtype, quantization
 * y_scale / y_zero_point) is never written, `out` receives the group's result, the bytes the two ops
 * give.  The sum is computed operation by operation as the ops would; for a uint8 result the first
 * call with new parameters (outside stream capture; it synchronizes the stream) also looks for
 * constants with which floor(y*kc + (r*kr + k0)), two fused multiply-adds, gives the same byte as that
 * arithmetic on every one of the 65536 pairs of codes, checks each candidate on the device against
 * the arithmetic itself, and uses the short form from then on if one passes (CHX_HIP_AFFINE_RESIDUAL=0
 * in the environment when the plan is created keeps the long one).  r and out: same shape as y, channels-last, uint8 or int8.
 * `out` must not overlap x or r in memory (the first call on a new shape may run the kernel several
 * times on the call's operands to pick a launch configuration): CHX_HIP_EINVAL when it does.
 * CHX_HIP_EUNSUPPORTED when the plan's weights or the layouts do not fit the matrix-core kernel;
 * the caller then runs the two ops separately. */
int chx_hip_qconv_plan_run_add(
        const chx_hip_qconv_plan* plan, const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, float y_scale,
        int32_t y_zero_point, int32_t y_dtype, uint32_t flags, const chx_hip_tensor* r, float r_scale, int32_t r_zero_point,
        float out_scale, int32_t out_zero_point, int32_t relu, chx_hip_tensor* out, void* stream);
/* Pins (delta = +1) or releases (-1) the plan's device memory for a recorded run: a HIP graph captured over
 * chx_hip_qconv_plan_run holds the addresses of the packed weights and of the scratch memory.  While a plan is
 * pinned, a run that would have to enlarge (move) the scratch memory fails with CHX_HIP_EPINNED, and
 * chx_hip_qconv_plan_destroy is deferred until the last pin is released.  No counterpart in the reference (it has
 * no recorded runs); the ChxVM runtime pins every plan a recorded program run has used. */
int chx_hip_qconv_plan_pin(chx_hip_qconv_plan* plan, int32_t delta);
void chx_hip_qconv_plan_destroy(chx_hip_qconv_plan* plan);

/* ---- integer contractions ------------------------------------------------------------- */

/* ConvIntegerOp::RunImpl, runtime/ops/quantize.cc:116-146.  y int32 [N,OC,OH,OW].
 * w_zero_point: NULL, 0-d or [OC]. */
int chx_hip_conv_integer(
        const chx_hip_tensor* x, const chx_hip_tensor* w, int32_t x_zero_point, const chx_hip_tensor* w_zero_point,
        const chx_hip_conv_params* params, chx_hip_tensor* y, void* stream);

/* MatMulIntegerOp::RunImpl, runtime/ops/quantize.cc:96-114 with NumpyMatMul,
 * runtime/chainerx_util.cc:210-230.  a [..,M,K], b [..,K,N] with equal leading
 * dims, y int32 [..,M,N].  Zero points: NULL, or arrays of ndim <= 1 subtracted by
 * numpy broadcasting (a 1-D one lines up with the last axis: K for a, N for b). */
int chx_hip_matmul_integer(
        const chx_hip_tensor* a, const chx_hip_tensor* b, const chx_hip_tensor* a_zero_point,
        const chx_hip_tensor* b_zero_point, chx_hip_tensor* y, void* stream);

/* The instruction sequence DequantizeLinear, DequantizeLinear, MatMul, QuantizeLinear
 * that ReplaceQLinearMatMul (compiler/simplifier.cc:675-694) leaves for an ONNX
 * QLinearMatMul node, as one kernel.  Per-tensor scales and zero points.
 * `bias` (int32 [N], added to the accumulator) and CHX_HIP_FUSE_RELU are
 * extensions used by the MLP configuration; pass NULL / 0 for the reference op. */
int chx_hip_qlinear_matmul(
        const chx_hip_tensor* a, float a_scale, int32_t a_zero_point, const chx_hip_tensor* b, float b_scale,
        int32_t b_zero_point, float y_scale, int32_t y_zero_point, const chx_hip_tensor* bias, uint32_t flags,
        chx_hip_tensor* y, void* stream);

/* ---- float32 layers around a quantized network ------------------------------------------ */

/* GemmOp::RunImpl, runtime/ops/math.cc:160-177:  r = op(a) . op(b);  r *= alpha when alpha != 1;
 * y = r when c is NULL or beta == 0, else r + (beta != 1 ? c * beta : c), c broadcast over
 * [M, N] as numpy does (a vector is a row).  All float32, any strides; trans_a / trans_b
 * transpose the matrix operands.  The dot product is summed in float32 in ascending k from 0,
 * one rounding per multiplication and per addition (the order of ChainerX's Dot is not in the
 * reference tree; results are compared with the reference's own tolerance). */
int chx_hip_gemm_f32(
        const chx_hip_tensor* a, const chx_hip_tensor* b, const chx_hip_tensor* c, float alpha, float beta, int32_t trans_a,
        int32_t trans_b, chx_hip_tensor* y, void* stream);

/* LinearOp::RunImpl, runtime/ops/connection.cc:12-15 (chainerx::Linear): x is taken as a matrix
 * [product of its first n_batch_axes extents, product of the rest], y = x . w^T + b with
 * w [out, in] and b [out] or NULL; y has the batch extents of x and one axis of `out`.  The axes
 * of x (and of y) on each side of n_batch_axes must be contiguous with each other.  The same
 * arithmetic as chx_hip_gemm_f32 with trans_b, alpha = beta = 1 (GemmOp takes this route then,
 * math.cc:162-164). */
int chx_hip_linear_f32(
        const chx_hip_tensor* x, const chx_hip_tensor* w, const chx_hip_tensor* b, int32_t n_batch_axes, chx_hip_tensor* y,
        void* stream);

/* MaxPoolOp / AveragePoolOp::RunImpl on float32 arrays, runtime/ops/pooling.cc:47-75: [N,C,H,W] with any
 * strides.  max: out extent with cover_all as in ChainerX (ceil instead of floor, plus one), taps in the
 * padding never win, a window in the padding altogether gives the lowest finite float.  average: symmetric
 * pads, the window's taps added in (kh, kw) order in float32 from 0, divided by kernel_h * kernel_w when
 * count_include_pad and by the number of taps inside the image otherwise.  (The sum order and the padding value
 * of ChainerX's own kernels are not in the reference tree.) */
int chx_hip_max_pool_f32(
        const chx_hip_tensor* x, int32_t kernel_h, int32_t kernel_w, int32_t stride_h, int32_t stride_w,
        int32_t pad_h_begin, int32_t pad_w_begin, int32_t pad_h_end, int32_t pad_w_end, int32_t cover_all,
        chx_hip_tensor* y, void* stream);
int chx_hip_average_pool_f32(
        const chx_hip_tensor* x, int32_t kernel_h, int32_t kernel_w, int32_t stride_h, int32_t stride_w, int32_t pad_h,
        int32_t pad_w, int32_t count_include_pad, chx_hip_tensor* y, void* stream);

/* FixedBatchNormalizationOp::RunImpl, runtime/ops/normalization.cc:210-225 (the inference form a
 * BatchNormalization node with one output is emitted as, compiler/chxvm/emitter.cc:193-206): x float32
 * [N, C, ...] with any batch and channel strides and the remaining axes one evenly strided run (NCHW,
 * channels-last); s, bias, mean, var contiguous float32 with C elements each;
 *   y = ((x - mean) * (1 / sqrt(var + eps))) * s + bias
 * one float32 rounding per operation in this order, eps <= 1e-5 replaced by (float)(1e-5 + 1e-12) as the op
 * does.  (The operation order of ChainerX's FixedBatchNorm is not in the reference tree.) */
int chx_hip_fixed_batch_norm_f32(
        const chx_hip_tensor* x, const chx_hip_tensor* s, const chx_hip_tensor* bias, const chx_hip_tensor* mean,
        const chx_hip_tensor* var, float epsilon, chx_hip_tensor* y, void* stream);

/* ConvOp::RunImpl, runtime/ops/connection.cc:24-30 (GroupedConv, runtime/chainerx_util.cc:313-340) on
 * float32: the convolutions the quantizer does not rewrite (a Conv with a bias, compiler/quantize.cc:376-381).
 * x [N,C,H,W], w [OC,C/group,KH,KW], b [OC] or NULL, y [N,OC,OH,OW], all float32 with any strides; params as
 * for chx_hip_qlinear_conv (auto_pad already resolved into explicit pads).  The sum runs over (c, kh, kw) in
 * this order in float32 from 0, one rounding per multiplication and per addition, b added last.  (The order
 * of ChainerX's own Conv is not in the reference tree; against the reference the result carries its
 * tolerance, rtol 1e-4 / atol 1e-6.)  A coverage kernel, not tuned. */
int chx_hip_conv_f32(
        const chx_hip_tensor* x, const chx_hip_tensor* w, const chx_hip_tensor* b, const chx_hip_conv_params* params,
        chx_hip_tensor* y, void* stream);

/* SoftmaxOp::RunImpl, runtime/ops/activation.cc:66-95 (chainerx::Softmax): x and y contiguous float32 of one
 * shape; with is_onnx_semantics the axes from `axis` on are reduced together (RunSoftmax's reshape), otherwise
 * `axis` alone.  m = max over the reduced elements, e = exp(x - m) as the host C library computes expf,
 * s = the sum of e in ascending order from 0, y = e * (1 / s), one float32 rounding per operation.  (The sequence
 * inside ChainerX's Softmax is not in the reference tree.) */
int chx_hip_softmax_f32(const chx_hip_tensor* x, int32_t axis, int32_t is_onnx_semantics, chx_hip_tensor* y, void* stream);

/* ---- pooling on quantized tensors ------------------------------------------------------ */

/* MaxPoolOp::RunImpl, runtime/ops/pooling.cc:47-61, as it occurs in a quantized
 * network: DequantizeLinear -> MaxPool -> QuantizeLinear with one scale and zero
 * point on both sides.  For uint8 that is the maximum m of the 8-bit codes; for int8
 * it is m + (m < 0), because quantize_array (runtime/ops/quantize.cc:16-35) adds 0.5
 * and casts with truncation toward zero, which moves a negative code up by one (a
 * window in the padding altogether gives -127).  x, y uint8 or int8 (same dtype),
 * [N,C,H,W].  cover_all as in ChainerX: the output extent is
 * ceil((in + pads - k) / s) + 1 and overhanging windows see only the image. */
int chx_hip_max_pool_q8(
        const chx_hip_tensor* x, int32_t kernel_h, int32_t kernel_w, int32_t stride_h, int32_t stride_w,
        int32_t pad_h_begin, int32_t pad_w_begin, int32_t pad_h_end, int32_t pad_w_end, int32_t cover_all,
        chx_hip_tensor* y, void* stream);

/* AveragePoolOp::RunImpl, runtime/ops/pooling.cc:63-75, between a DequantizeLinear
 * (x_scale, x_zero_point) and a QuantizeLinear (y_scale, y_zero_point):
 * y = Q(sum_{window} DQ(x) / count), fp32 sum in (kh, kw) order. */
int chx_hip_average_pool_q8(
        const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, int32_t kernel_h, int32_t kernel_w,
        int32_t stride_h, int32_t stride_w, int32_t pad_h, int32_t pad_w, int32_t count_include_pad, float y_scale,
        int32_t y_zero_point, uint32_t flags, chx_hip_tensor* y, void* stream);

/* ---- fused element-wise chains ---------------------------------------------------------- */

/* ElementWiseNvrtcOp::RunImpl, runtime/ops/nvrtc.cc:90-161.  `code` is the program
 * text the hip fusion builder emits for a FusionGroup (the counterpart of the CUDA
 * source from compiler/nvrtc_builder.cc:91-206): one SSA statement per node in
 * topological order.  All inputs must have one dtype; the result shape is the
 * broadcast of the input shapes; inputs are read through their strides (nothing is
 * materialised).  The kernel is generated and compiled with hiprtc on first use
 * and cached by program text and operand layout, like the reference's two-level
 * cache (runtime/ops/nvrtc.cc:41-84). */
int chx_hip_elementwise(
        const char* code, int32_t fusion_id, const chx_hip_tensor* const* inputs, int32_t n_inputs,
        chx_hip_tensor* const* outputs, int32_t n_outputs, void* stream);

/* The result types of a FusionGroup program, in the order of its outputs: what
 * ElementWiseNvrtcOp::RunImpl needs to allocate its results (the reference allocates
 * them with the type of the inputs, runtime/ops/nvrtc.cc:138-141; a program of this
 * library may also end in a QuantizeLinear).  Writes at most `capacity` codes; *count
 * receives the number of outputs.  Touches no device memory. */
int chx_hip_elementwise_output_dtypes(const char* code, int32_t* dtypes, int32_t capacity, int32_t* count);

/* Diagnostics for the same op: writes the HIP source that chx_hip_elementwise would
 * generate for these operands into `buffer` (truncated to buffer_size, always
 * terminated; *needed receives the full size) and, when `compile` is non-zero, also
 * runs it through hiprtc.  Touches no device memory and needs no GPU, so it is what
 * a build machine uses to validate a program.  Counterpart of the reference's source
 * dumps (runtime/ops/nvrtc.cc:118-123, compiler/chxvm/emitter.cc:625-627). */
int chx_hip_elementwise_source(
        const char* code, int32_t fusion_id, const chx_hip_tensor* const* inputs, int32_t n_inputs,
        chx_hip_tensor* const* outputs, int32_t n_outputs, int32_t compile, char* buffer, size_t buffer_size,
        size_t* needed);

/* ReduceMaxOp / ReduceMinOp::RunImpl (runtime/ops/statistics.cc:13-19, chainerx::AMax / AMin) for the only form
 * the quantizer emits (compiler/quantize.cc:171-174): every axis reduced, keepdims = 0.  x float32,
 * any strides; y float32 with one element. */
int chx_hip_reduce_min_max(const chx_hip_tensor* x, int32_t is_max, chx_hip_tensor* y, void* stream);
/* The same reduction for callers that cannot allocate device memory (code under graph capture, serving
 * loops, harnesses that forbid it); it has no counterpart in the reference.  chx_hip_reduce_min_max takes its
 * per-work-group partial results from the stream-ordered allocator; this one keeps them in a 4 KiB array in
 * the library's device image (every GPU the library runs on holds its own copy until the process ends) and
 * calls no allocation routine.  At most 2^30 elements: CHX_HIP_EINVAL beyond.  Calls that overlap on one GPU
 * (two streams, two threads) share the array and race: keep them in one stream's order.  Results are
 * identical to chx_hip_reduce_min_max's. */
int chx_hip_reduce_min_max_noalloc(const chx_hip_tensor* x, int32_t is_max, chx_hip_tensor* y, void* stream);

/* BitShiftOp::RunImpl, runtime/ops/quantize.cc:153-163 (chainerx::LeftShift / RightShift): z = x << y when `left`
 * is non-zero, x >> y otherwise, over the broadcast of x and y; one integer type (uint8, int8, int16, int32, int64)
 * for x, y and z; z has the broadcast shape.  The right shift of a signed type is arithmetic; a count of the element
 * width or more (which C leaves undefined) gives 0, or -1 for a negative x shifted right. */
int chx_hip_bit_shift(const chx_hip_tensor* x, const chx_hip_tensor* y, int32_t left, chx_hip_tensor* z, void* stream);

/* The scan behind ChxVMState::CheckNans / CheckInfs (runtime/chxvm_state.cc:215-263: chainerx::IsNan / IsInf,
 * Sum, AsScalar): *count receives the number of NaN elements of x (infinities = 0) or of +-Inf elements
 * (infinities != 0).  float32 arrays with any strides are scanned, other element types hold neither and
 * give 0.  Synchronizes the stream (the caller acts on the count), so it is a debugging aid and stays out
 * of captured graphs. */
int chx_hip_count_nonfinite(const chx_hip_tensor* x, int32_t infinities, int64_t* count, void* stream);

/* CastOp::RunImpl (runtime/ops/manipulation.cc:157-159, CastTo): element types float32,
 * int32, uint8, int8 on either side; float -> integer truncates toward zero. */
int chx_hip_cast(const chx_hip_tensor* x, chx_hip_tensor* y, void* stream);

/* Moves 8-bit codes between the two storages that CHX_HIP_STORE_MINUS_128 distinguishes; it has no counterpart
 * in the reference, whose uint8 tensors have one storage.  x uint8, y int8: y = code - 128; x int8, y uint8:
 * y = code + 128 (either way bit 7 of every byte inverted).  Same shape, any strides.  A runtime that keeps
 * some values in the minus-128 storage uses it when such a value reaches a reader that wants plain codes. */
int chx_hip_codes_minus_128(const chx_hip_tensor* x, chx_hip_tensor* y, void* stream);

/* Says whether a fusion program (the `code` of an ElementWiseNvrtc instruction, emitted per
 * FusionGroup by compiler/chxvm/emitter.cc:621-729) is exactly the residual sum of a quantized
 * network,  out = QuantizeLinear(act(DequantizeLinear(in0) + DequantizeLinear(in1)))  with
 * act = Relu or nothing, and if so with which constants: the form chx_hip_qconv_plan_run_add
 * computes inside the convolution that produces one of the operands.  Host-only (no GPU work).
 * A program that does not parse is an error; one that parses but has another form sets
 * *matches = 0. */
typedef struct chx_hip_residual_group {
    float in_scale[2];          /* DequantizeLinear constants of input 0 and input 1 */
    int32_t in_zero_point[2];
    int32_t in_dtype[2];
    int32_t relu;
    float out_scale;
    int32_t out_zero_point;
    int32_t out_dtype;
} chx_hip_residual_group;
int chx_hip_elementwise_match_residual_add(const char* code, int32_t* matches, chx_hip_residual_group* group);

#ifdef __cplusplus
}
#endif

#endif /* CHX_HIP_H_ */
