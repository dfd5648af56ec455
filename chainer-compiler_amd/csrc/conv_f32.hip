// ConvOp::RunImpl (runtime/ops/connection.cc:24-30, GroupedConv runtime/chainerx_util.cc:313-340) on
// float32: the convolutions the quantizer leaves alone (a Conv with a bias, compiler/quantize.cc:376-381).
//
//   y[n, oc, oh, ow] = sum over (c, kh, kw) of x[n, g*Cg + c, oh*sh - ph + kh, ow*sw - pw + kw] * w[oc, c, kh, kw]
//                      (+ b[oc], added last)
//
// float32, the taps in (c, kh, kw) order from an accumulator of 0, one rounding per multiplication and per
// addition, a tap in the padding as the product 0 * w.  That is the order of the CPU restatement this kernel
// is tested against bit for bit (an expanded-matrix product with k ascending); ChainerX's own Conv is not in
// the reference tree.
//
// A coverage kernel: one lane per output element, every operand through its strides; the unit-stride axis
// of y runs along consecutive lanes.  Not tuned and not on the benchmark path.
#include <cstring>

#include "chx_internal.h"

namespace chx {
namespace {

struct ConvF32Args {
    const char* x;
    const char* w;
    const char* b;
    char* y;
    int64_t xs[4], ws[4], ys[4], bs;
    int32_t N, C, H, W, OC, Cg, OCg, KH, KW, OH, OW, sh, sw, ph, pw;
    int64_t total;
    int32_t channels_fastest;
};

__global__ __launch_bounds__(256) void conv_f32_kernel(ConvF32Args a) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= a.total) return;
    int n, oc, oh, ow;
    int64_t r = idx;
    if (a.channels_fastest) {
        oc = (int)(r % a.OC); r /= a.OC;
        ow = (int)(r % a.OW); r /= a.OW;
        oh = (int)(r % a.OH);
        n = (int)(r / a.OH);
    } else {
        ow = (int)(r % a.OW); r /= a.OW;
        oh = (int)(r % a.OH); r /= a.OH;
        oc = (int)(r % a.OC);
        n = (int)(r / a.OC);
    }
    const int c0 = (oc / a.OCg) * a.Cg;
    const char* xn = a.x + n * a.xs[0];
    const char* wo = a.w + oc * a.ws[0];
    float acc = 0.f;
    for (int c = 0; c < a.Cg; ++c)
        for (int kh = 0; kh < a.KH; ++kh) {
            const int ih = oh * a.sh - a.ph + kh;
            for (int kw = 0; kw < a.KW; ++kw) {
                const int iw = ow * a.sw - a.pw + kw;
                float v = 0.f;
                if ((unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W)
                    v = *reinterpret_cast<const float*>(xn + (c0 + c) * a.xs[1] + ih * a.xs[2] + iw * a.xs[3]);
                const float prod = v * *reinterpret_cast<const float*>(wo + c * a.ws[1] + kh * a.ws[2] + kw * a.ws[3]);
                acc = acc + prod;
            }
        }
    if (a.b) acc = acc + *reinterpret_cast<const float*>(a.b + oc * a.bs);
    *reinterpret_cast<float*>(a.y + n * a.ys[0] + oc * a.ys[1] + oh * a.ys[2] + ow * a.ys[3]) = acc;
}

}  // namespace
}  // namespace chx

using namespace chx;

extern "C" int chx_hip_conv_f32(
        const chx_hip_tensor* x, const chx_hip_tensor* w, const chx_hip_tensor* b, const chx_hip_conv_params* params,
        chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(x, "Conv x"));
    CHX_PROPAGATE(check_tensor(w, "Conv w"));
    CHX_PROPAGATE(check_tensor(y, "Conv y"));
    CHX_REQUIRE(params != nullptr, "Conv: params is NULL");
    const chx_hip_conv_params& p = *params;
    CHX_REQUIRE(x->ndim == 4 && w->ndim == 4 && y->ndim == 4, "Conv: x, w and y must be 4-D (2-D convolution only)");
    CHX_REQUIRE(x->dtype == CHX_HIP_FLOAT32 && w->dtype == CHX_HIP_FLOAT32 && y->dtype == CHX_HIP_FLOAT32,
                "Conv: x, w and y must be float32");
    CHX_REQUIRE(p.group >= 1 && p.stride_h >= 1 && p.stride_w >= 1, "Conv: group and strides must be positive");
    CHX_REQUIRE(p.pad_h_begin >= 0 && p.pad_w_begin >= 0 && p.pad_h_end >= 0 && p.pad_w_end >= 0, "Conv: negative padding is not supported");
    for (int i = 0; i < 4; ++i) CHX_REQUIRE(x->shape[i] <= INT32_MAX && w->shape[i] <= INT32_MAX, "Conv: extent too large");
    ConvF32Args a;
    memset(&a, 0, sizeof(a));
    a.N = (int32_t)x->shape[0]; a.C = (int32_t)x->shape[1]; a.H = (int32_t)x->shape[2]; a.W = (int32_t)x->shape[3];
    a.OC = (int32_t)w->shape[0]; a.Cg = (int32_t)w->shape[1]; a.KH = (int32_t)w->shape[2]; a.KW = (int32_t)w->shape[3];
    CHX_REQUIRE(a.C == a.Cg * p.group, "Conv: x has %d channels but w expects %d x group %d", a.C, a.Cg, p.group);
    CHX_REQUIRE(a.OC % p.group == 0, "Conv: %d output channels do not divide into %d groups", a.OC, p.group);
    const int64_t eh = (int64_t)a.H + p.pad_h_begin + p.pad_h_end - a.KH, ew = (int64_t)a.W + p.pad_w_begin + p.pad_w_end - a.KW;
    CHX_REQUIRE(eh >= 0 && ew >= 0, "Conv: kernel %dx%d larger than the padded input", a.KH, a.KW);
    a.OH = (int32_t)(eh / p.stride_h + 1);
    a.OW = (int32_t)(ew / p.stride_w + 1);
    CHX_REQUIRE(y->shape[0] == a.N && y->shape[1] == a.OC && y->shape[2] == a.OH && y->shape[3] == a.OW,
                "Conv: y is [%lld,%lld,%lld,%lld], expected [%d,%d,%d,%d]", (long long)y->shape[0], (long long)y->shape[1],
                (long long)y->shape[2], (long long)y->shape[3], a.N, a.OC, a.OH, a.OW);
    if (b) {
        CHX_PROPAGATE(check_tensor(b, "Conv b"));
        CHX_REQUIRE(b->dtype == CHX_HIP_FLOAT32 && b->ndim == 1 && b->shape[0] == a.OC, "Conv: b must be float32 [%d]", a.OC);
        a.b = static_cast<const char*>(b->data);
        a.bs = b->strides[0];
    }
    a.x = static_cast<const char*>(x->data);
    a.w = static_cast<const char*>(w->data);
    a.y = static_cast<char*>(y->data);
    for (int i = 0; i < 4; ++i) {
        a.xs[i] = x->strides[i];
        a.ws[i] = w->strides[i];
        a.ys[i] = y->strides[i];
    }
    a.OCg = a.OC / p.group;
    a.sh = p.stride_h; a.sw = p.stride_w; a.ph = p.pad_h_begin; a.pw = p.pad_w_begin;
    a.total = (int64_t)a.N * a.OC * a.OH * a.OW;
    if (a.total == 0) return CHX_HIP_OK;
    a.channels_fastest = y->strides[1] == 4 && a.OC > 1;
    conv_f32_kernel<<<(unsigned)((a.total + 255) / 256), 256, 0, as_stream(stream)>>>(a);
    return launch_check("conv_f32_kernel");
}
