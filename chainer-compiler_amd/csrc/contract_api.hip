// Entry points of the integer contractions: QLinearConv, ConvInteger, MatMulInteger,
// QLinearMatMul.  Validation and shape rules follow the reference's RunImpl bodies
// (runtime/ops/quantize.cc:62-146) and GroupedConv (runtime/chainerx_util.cc:313-340);
// the arithmetic is in the kernels.
#include <climits>
#include <cstring>
#include <vector>

#include "contract.h"

namespace chx {
namespace {

struct ConvShape {
    int32_t N, C, H, W, OC, Cg, KH, KW, OH, OW;
};

int conv_shape(
        const chx_hip_tensor& x, const chx_hip_tensor& w, const chx_hip_conv_params& p, const chx_hip_tensor& y,
        const char* op, ConvShape* cs) {
    CHX_REQUIRE(x.ndim == 4 && w.ndim == 4 && y.ndim == 4, "%s: x, w and y must be 4-D (2-D convolution only)", op);
    CHX_REQUIRE(is_q8(x.dtype), "%s: x must be uint8 or int8, got %s", op, dtype_name(x.dtype));
    CHX_REQUIRE(is_q8(w.dtype), "%s: w must be uint8 or int8, got %s", op, dtype_name(w.dtype));
    CHX_REQUIRE(p.group >= 1 && p.stride_h >= 1 && p.stride_w >= 1, "%s: group and strides must be positive", op);
    CHX_REQUIRE(p.pad_h_begin >= 0 && p.pad_w_begin >= 0 && p.pad_h_end >= 0 && p.pad_w_end >= 0,
                "%s: negative padding is not supported", op);
    for (int i = 0; i < 4; ++i)
        CHX_REQUIRE(x.shape[i] <= INT32_MAX && w.shape[i] <= INT32_MAX, "%s: extent too large", op);
    cs->N = (int32_t)x.shape[0];
    cs->C = (int32_t)x.shape[1];
    cs->H = (int32_t)x.shape[2];
    cs->W = (int32_t)x.shape[3];
    cs->OC = (int32_t)w.shape[0];
    cs->Cg = (int32_t)w.shape[1];
    cs->KH = (int32_t)w.shape[2];
    cs->KW = (int32_t)w.shape[3];
    CHX_REQUIRE(cs->C == cs->Cg * p.group, "%s: x has %d channels but w expects %d x group %d", op, cs->C, cs->Cg, p.group);
    CHX_REQUIRE(cs->OC % p.group == 0, "%s: %d output channels do not divide into %d groups", op, cs->OC, p.group);
    const int64_t eh = (int64_t)cs->H + p.pad_h_begin + p.pad_h_end - cs->KH;
    const int64_t ew = (int64_t)cs->W + p.pad_w_begin + p.pad_w_end - cs->KW;
    CHX_REQUIRE(eh >= 0 && ew >= 0, "%s: kernel %dx%d larger than the padded input", op, cs->KH, cs->KW);
    cs->OH = (int32_t)(eh / p.stride_h + 1);
    cs->OW = (int32_t)(ew / p.stride_w + 1);
    CHX_REQUIRE(y.shape[0] == cs->N && y.shape[1] == cs->OC && y.shape[2] == cs->OH && y.shape[3] == cs->OW,
                "%s: y is [%lld,%lld,%lld,%lld], expected [%d,%d,%d,%d]", op, (long long)y.shape[0], (long long)y.shape[1],
                (long long)y.shape[2], (long long)y.shape[3], cs->N, cs->OC, cs->OH, cs->OW);
    return CHX_HIP_OK;
}

// A 0-d or 1-d parameter array with `expect_one_or` elements.
int param_vector(const chx_hip_tensor& t, int64_t per_channel, const char* what, int64_t* len, int64_t* stride) {
    CHX_REQUIRE(t.ndim <= 1, "%s must be 0-d or 1-d", what);
    *len = numel(t);
    CHX_REQUIRE(*len == 1 || *len == per_channel, "%s has %lld elements, expected 1 or %lld", what, (long long)*len,
                (long long)per_channel);
    *stride = t.ndim == 1 ? t.strides[0] : 0;
    return CHX_HIP_OK;
}

void fill_conv_args(
        const chx_hip_tensor& x, const chx_hip_tensor& w, const chx_hip_conv_params& p, const chx_hip_tensor& y,
        const ConvShape& cs, ConvDirectArgs* a) {
    memset(a, 0, sizeof(*a));
    a->x = static_cast<const char*>(x.data);
    a->w = static_cast<const char*>(w.data);
    a->y = static_cast<char*>(y.data);
    for (int i = 0; i < 4; ++i) {
        a->xs[i] = x.strides[i];
        a->ws[i] = w.strides[i];
        a->ys[i] = y.strides[i];
    }
    a->N = cs.N; a->C = cs.C; a->H = cs.H; a->W = cs.W;
    a->OC = cs.OC; a->Cg = cs.Cg; a->KH = cs.KH; a->KW = cs.KW; a->OH = cs.OH; a->OW = cs.OW;
    a->sh = p.stride_h; a->sw = p.stride_w; a->ph = p.pad_h_begin; a->pw = p.pad_w_begin; a->group = p.group;
    a->x_signed = x.dtype == CHX_HIP_INT8;
    a->w_signed = w.dtype == CHX_HIP_INT8;
    a->total = (int64_t)cs.N * cs.OC * cs.OH * cs.OW;
}

int fill_requant(
        float x_scale, float y_scale, int32_t y_zp, const chx_hip_tensor& y, const chx_hip_tensor* bias, int64_t bias_len,
        uint32_t flags, const char* op, RequantParams* rq, const int32_t** bias_ptr) {
    CHX_REQUIRE(is_q8(y.dtype), "%s: y must be uint8 or int8, got %s", op, dtype_name(y.dtype));
    const bool i8 = y.dtype == CHX_HIP_INT8;
    CHX_REQUIRE(y_zp >= (i8 ? -128 : 0) && y_zp <= (i8 ? 127 : 255), "%s: zero point %d outside the range of %s", op,
                y_zp, dtype_name(y.dtype));
    rq->q = make_quant_params(y_scale, y_zp, i8);
    rq->x_scale = x_scale;
    rq->relu_floor = (flags & CHX_HIP_FUSE_RELU) ? y_zp : INT32_MIN;
    rq->bias_mode = kBiasNone;
    *bias_ptr = nullptr;
    if (bias) {
        CHX_PROPAGATE(check_tensor(bias, "bias"));
        CHX_REQUIRE(bias->dtype == CHX_HIP_INT32, "%s: bias must be int32, got %s", op, dtype_name(bias->dtype));
        CHX_REQUIRE(bias->ndim == 1 && bias->shape[0] == bias_len && is_contiguous(*bias),
                    "%s: bias must be a contiguous [%lld] vector", op, (long long)bias_len);
        rq->bias_mode = (flags & CHX_HIP_BIAS_ONNX_INT32) ? kBiasOnnxInt32 : kBiasReferenceFloat;
        *bias_ptr = static_cast<const int32_t*>(bias->data);
    }
    return CHX_HIP_OK;
}

struct MatMulShape {
    int64_t batch, M, K, N;
    int64_t a_batch, b_batch, y_batch;
};

// NumpyMatMul, runtime/chainerx_util.cc:210-230: 2-D Dot, or N-D with equal leading dims
// flattened into a batch.  Leading dims must be contiguous among themselves.
int matmul_shape(const chx_hip_tensor& a, const chx_hip_tensor& b, const chx_hip_tensor& y, const char* op, MatMulShape* ms) {
    CHX_REQUIRE(a.ndim >= 2 && b.ndim == a.ndim && y.ndim == a.ndim, "%s: a, b and y must have the same ndim >= 2", op);
    const int nd = a.ndim;
    ms->M = a.shape[nd - 2];
    ms->K = a.shape[nd - 1];
    ms->N = b.shape[nd - 1];
    CHX_REQUIRE(b.shape[nd - 2] == ms->K, "%s: inner dimensions differ (%lld vs %lld)", op, (long long)ms->K,
                (long long)b.shape[nd - 2]);
    CHX_REQUIRE(y.shape[nd - 2] == ms->M && y.shape[nd - 1] == ms->N, "%s: y has the wrong matrix shape", op);
    ms->batch = 1;
    for (int i = 0; i < nd - 2; ++i) {
        CHX_REQUIRE(a.shape[i] == b.shape[i] && a.shape[i] == y.shape[i], "%s: leading dimensions differ", op);
        ms->batch *= a.shape[i];
    }
    auto batch_stride = [&](const chx_hip_tensor& t, int64_t* out) -> int {
        // leading axes must collapse into one
        *out = 0;
        int64_t expect = -1;
        for (int i = nd - 3; i >= 0; --i) {
            if (t.shape[i] == 1) continue;
            if (expect < 0) {
                *out = t.strides[i];
                expect = t.strides[i] * t.shape[i];
            } else {
                CHX_REQUIRE(t.strides[i] == expect, "%s: leading dimensions are not collapsible", op);
                expect *= t.shape[i];
            }
        }
        return CHX_HIP_OK;
    };
    CHX_PROPAGATE(batch_stride(a, &ms->a_batch));
    CHX_PROPAGATE(batch_stride(b, &ms->b_batch));
    CHX_PROPAGATE(batch_stride(y, &ms->y_batch));
    return CHX_HIP_OK;
}

void fill_matmul_args(
        const chx_hip_tensor& a, const chx_hip_tensor& b, const chx_hip_tensor& y, const MatMulShape& ms, MatMulDirectArgs* m) {
    memset(m, 0, sizeof(*m));
    const int nd = a.ndim;
    m->a = static_cast<const char*>(a.data);
    m->b = static_cast<const char*>(b.data);
    m->y = static_cast<char*>(y.data);
    m->a_batch = ms.a_batch; m->a_row = a.strides[nd - 2]; m->a_col = a.strides[nd - 1];
    m->b_batch = ms.b_batch; m->b_row = b.strides[nd - 2]; m->b_col = b.strides[nd - 1];
    m->y_batch = ms.y_batch; m->y_row = y.strides[nd - 2]; m->y_col = y.strides[nd - 1];
    m->M = ms.M; m->K = ms.K; m->N = ms.N;
    m->total = ms.batch * ms.M * ms.N;
    m->a_signed = a.dtype == CHX_HIP_INT8;
    m->b_signed = b.dtype == CHX_HIP_INT8;
}

}  // namespace
}  // namespace chx

using namespace chx;

extern "C" int chx_hip_conv_integer(
        const chx_hip_tensor* x, const chx_hip_tensor* w, int32_t x_zero_point, const chx_hip_tensor* w_zero_point,
        const chx_hip_conv_params* params, chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(x, "ConvInteger x"));
    CHX_PROPAGATE(check_tensor(w, "ConvInteger w"));
    CHX_PROPAGATE(check_tensor(y, "ConvInteger y"));
    CHX_REQUIRE(params != nullptr, "ConvInteger: null params");
    CHX_REQUIRE(y->dtype == CHX_HIP_INT32, "ConvInteger: y must be int32, got %s", dtype_name(y->dtype));
    ConvShape cs;
    CHX_PROPAGATE(conv_shape(*x, *w, *params, *y, "ConvInteger", &cs));
    ConvDirectArgs a;
    fill_conv_args(*x, *w, *params, *y, cs, &a);
    a.x_zp = x_zero_point;
    if (w_zero_point) {
        CHX_PROPAGATE(check_tensor(w_zero_point, "ConvInteger w_zero_point"));
        CHX_REQUIRE(w_zero_point->dtype == w->dtype, "ConvInteger: w_zero_point must have the dtype of w");
        int64_t len, stride;
        CHX_PROPAGATE(param_vector(*w_zero_point, cs.OC, "ConvInteger w_zero_point", &len, &stride));
        a.w_zp = static_cast<const char*>(w_zero_point->data);
        a.w_zp_len = (int32_t)len;
        a.w_zp_stride = stride;
    }
    return launch_conv_direct(a, false, as_stream(stream));
}

extern "C" int chx_hip_matmul_integer(
        const chx_hip_tensor* a, const chx_hip_tensor* b, const chx_hip_tensor* a_zero_point,
        const chx_hip_tensor* b_zero_point, chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(a, "MatMulInteger a"));
    CHX_PROPAGATE(check_tensor(b, "MatMulInteger b"));
    CHX_PROPAGATE(check_tensor(y, "MatMulInteger y"));
    CHX_REQUIRE(is_q8(a->dtype) && is_q8(b->dtype), "MatMulInteger: a and b must be uint8 or int8");
    CHX_REQUIRE(y->dtype == CHX_HIP_INT32, "MatMulInteger: y must be int32, got %s", dtype_name(y->dtype));
    MatMulShape ms;
    CHX_PROPAGATE(matmul_shape(*a, *b, *y, "MatMulInteger", &ms));
    MatMulDirectArgs m;
    fill_matmul_args(*a, *b, *y, ms, &m);
    if (a_zero_point) {
        CHX_PROPAGATE(check_tensor(a_zero_point, "MatMulInteger a_zero_point"));
        CHX_REQUIRE(is_q8(a_zero_point->dtype), "MatMulInteger: a_zero_point must be uint8 or int8");
        int64_t len, stride;
        CHX_PROPAGATE(param_vector(*a_zero_point, ms.K, "MatMulInteger a_zero_point", &len, &stride));  // CHECK_GE(1, ndim)
        m.a_zp = static_cast<const char*>(a_zero_point->data);
        m.a_zp_len = (int32_t)len;
        m.a_zp_stride = stride;
        m.a_zp_signed = a_zero_point->dtype == CHX_HIP_INT8;
    }
    if (b_zero_point) {
        CHX_PROPAGATE(check_tensor(b_zero_point, "MatMulInteger b_zero_point"));
        CHX_REQUIRE(is_q8(b_zero_point->dtype), "MatMulInteger: b_zero_point must be uint8 or int8");
        int64_t len, stride;
        CHX_PROPAGATE(param_vector(*b_zero_point, ms.N, "MatMulInteger b_zero_point", &len, &stride));
        m.b_zp = static_cast<const char*>(b_zero_point->data);
        m.b_zp_len = (int32_t)len;
        m.b_zp_stride = stride;
        m.b_zp_signed = b_zero_point->dtype == CHX_HIP_INT8;
    }
    return launch_matmul_direct(m, false, as_stream(stream));
}

extern "C" int chx_hip_qlinear_matmul(
        const chx_hip_tensor* a, float a_scale, int32_t a_zero_point, const chx_hip_tensor* b, float b_scale,
        int32_t b_zero_point, float y_scale, int32_t y_zero_point, const chx_hip_tensor* bias, uint32_t flags,
        chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(a, "QLinearMatMul a"));
    CHX_PROPAGATE(check_tensor(b, "QLinearMatMul b"));
    CHX_PROPAGATE(check_tensor(y, "QLinearMatMul y"));
    CHX_REQUIRE(is_q8(a->dtype) && is_q8(b->dtype), "QLinearMatMul: a and b must be uint8 or int8");
    MatMulShape ms;
    CHX_PROPAGATE(matmul_shape(*a, *b, *y, "QLinearMatMul", &ms));
    MatMulDirectArgs m;
    fill_matmul_args(*a, *b, *y, ms, &m);
    m.a_zp_imm = a_zero_point;
    m.b_zp_imm = b_zero_point;
    m.requant = 1;
    m.b_scale = b_scale;
    // the extension's bias is always the ONNX kind: int32, added to the accumulator
    CHX_PROPAGATE(fill_requant(a_scale, y_scale, y_zero_point, *y, bias, ms.N, flags | CHX_HIP_BIAS_ONNX_INT32,
                               "QLinearMatMul", &m.rq, &m.bias));
    return launch_matmul_direct(m, (flags & CHX_HIP_ROUND_ONNX_RNE) != 0, as_stream(stream));
}

extern "C" int chx_hip_qlinear_conv(
        const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, const chx_hip_tensor* w,
        const chx_hip_tensor* w_scale, const chx_hip_tensor* w_zero_point, float y_scale, int32_t y_zero_point,
        const chx_hip_tensor* bias, const chx_hip_conv_params* params, uint32_t flags, chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(x, "QLinearConv x"));
    CHX_PROPAGATE(check_tensor(w, "QLinearConv w"));
    CHX_PROPAGATE(check_tensor(w_scale, "QLinearConv w_scale"));
    CHX_PROPAGATE(check_tensor(w_zero_point, "QLinearConv w_zero_point"));
    CHX_PROPAGATE(check_tensor(y, "QLinearConv y"));
    CHX_REQUIRE(params != nullptr, "QLinearConv: null params");
    ConvShape cs;
    CHX_PROPAGATE(conv_shape(*x, *w, *params, *y, "QLinearConv", &cs));
    CHX_REQUIRE(w_scale->dtype == CHX_HIP_FLOAT32, "QLinearConv: w_scale must be float32");
    CHX_REQUIRE(w_zero_point->dtype == w->dtype, "QLinearConv: w_zero_point must have the dtype of w");
    // CHECK_EQ(w_scale.GetTotalSize(), w_zero_point.GetTotalSize()), runtime/ops/quantize.cc:76-77
    int64_t slen, sstride, zlen, zstride;
    CHX_PROPAGATE(param_vector(*w_scale, cs.OC, "QLinearConv w_scale", &slen, &sstride));
    CHX_PROPAGATE(param_vector(*w_zero_point, cs.OC, "QLinearConv w_zero_point", &zlen, &zstride));
    CHX_REQUIRE(slen == zlen && w_scale->ndim == w_zero_point->ndim,
                "QLinearConv: w_scale and w_zero_point must have the same shape");
    CHX_REQUIRE(slen == 1 || sstride == 4, "QLinearConv: w_scale must be contiguous");
    ConvDirectArgs a;
    fill_conv_args(*x, *w, *params, *y, cs, &a);
    a.x_zp = x_zero_point;
    a.w_zp = static_cast<const char*>(w_zero_point->data);
    a.w_zp_len = (int32_t)zlen;
    a.w_zp_stride = zstride;
    a.requant = 1;
    a.w_scale = static_cast<const float*>(w_scale->data);
    a.w_scale_len = (int32_t)slen;
    CHX_PROPAGATE(fill_requant(x_scale, y_scale, y_zero_point, *y, bias, cs.OC, flags, "QLinearConv", &a.rq, &a.bias));
    return launch_conv_direct(a, (flags & CHX_HIP_ROUND_ONNX_RNE) != 0, as_stream(stream));
}
