// FixedBatchNormalizationOp::RunImpl (runtime/ops/normalization.cc:210-225): the inference form of
// BatchNormalization on float32, for the float layers that stay around integer convolutions (the
// quantizer leaves BatchNormalization nodes in float, compiler/quantize.cc:377-380).
//
//   y[n, c, ...] = ((x[n, c, ...] - mean[c]) * (1 / sqrt(var[c] + eps))) * s[c] + bias[c]
//
// float32, one rounding per operation in this order, the square root and the reciprocal correctly
// rounded.  (ChainerX's FixedBatchNorm is not in the reference tree; this is the order of its generic
// kernel as the CPU restatement states it.)  eps at or below 1e-5 is replaced by (float)(1e-5 + 1e-12),
// as the op does for every device.
//
// One lane per element, x and y addressed through their strides (NCHW, channels-last, views); the unit-stride
// axis of y runs along consecutive lanes.
#include <cstring>

#include "chx_internal.h"

namespace chx {
namespace {

struct BatchNormArgs {
    const char* x;
    char* y;
    const float* s;
    const float* bias;
    const float* mean;
    const float* var;
    int64_t xs[3], ys[3];  // byte strides of (n, c, inner); the inner axes of x and of y are each one dense run
    int64_t N, C, inner, total;
    float eps;
    int32_t channels_fastest;
};

__global__ __launch_bounds__(256) void fixed_batch_norm_f32_kernel(BatchNormArgs a) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= a.total) return;
    int64_t n, c, i;
    if (a.channels_fastest) {
        c = idx % a.C;
        const int64_t r = idx / a.C;
        i = r % a.inner;
        n = r / a.inner;
    } else {
        i = idx % a.inner;
        const int64_t r = idx / a.inner;
        c = r % a.C;
        n = r / a.C;
    }
    const float v = *reinterpret_cast<const float*>(a.x + n * a.xs[0] + c * a.xs[1] + i * a.xs[2]);
    const float inv_std = 1.0f / __builtin_sqrtf(a.var[c] + a.eps);
    float r = v - a.mean[c];
    r = r * inv_std;
    r = r * a.s[c];
    r = r + a.bias[c];
    *reinterpret_cast<float*>(a.y + n * a.ys[0] + c * a.ys[1] + i * a.ys[2]) = r;
}

// The axes after the channel axis as one axis of `inner` elements `stride` bytes apart, if they are laid out so.
bool collapse_inner(const chx_hip_tensor& t, int64_t* inner, int64_t* stride) {
    int64_t count = 1, st = 4;
    bool first = true;
    for (int d = t.ndim - 1; d >= 2; --d) {
        if (t.shape[d] == 1) continue;
        if (first) {
            st = t.strides[d];
            first = false;
        } else if (t.strides[d] != st * count) {
            return false;
        }
        count *= t.shape[d];
    }
    *inner = count;
    *stride = st;
    return true;
}

int check_channel_vector(const chx_hip_tensor* t, int64_t C, const char* name) {
    CHX_PROPAGATE(check_tensor(t, name));
    CHX_REQUIRE(t->dtype == CHX_HIP_FLOAT32, "FixedBatchNormalization: %s must be float32", name);
    int64_t n = 1;
    for (int d = 0; d < t->ndim; ++d) n *= t->shape[d];
    CHX_REQUIRE(n == C, "FixedBatchNormalization: %s has %lld elements, the input has %lld channels", name, (long long)n, (long long)C);
    CHX_REQUIRE(is_contiguous(*t), "FixedBatchNormalization: %s must be contiguous", name);
    return CHX_HIP_OK;
}

}  // namespace
}  // namespace chx

using namespace chx;

extern "C" int chx_hip_fixed_batch_norm_f32(
        const chx_hip_tensor* x, const chx_hip_tensor* s, const chx_hip_tensor* bias, const chx_hip_tensor* mean,
        const chx_hip_tensor* var, float epsilon, chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(x, "FixedBatchNormalization x"));
    CHX_PROPAGATE(check_tensor(y, "FixedBatchNormalization y"));
    CHX_REQUIRE(x->dtype == CHX_HIP_FLOAT32 && y->dtype == CHX_HIP_FLOAT32, "FixedBatchNormalization: x and y must be float32");
    CHX_REQUIRE(x->ndim >= 2 && y->ndim == x->ndim, "FixedBatchNormalization: x needs a batch and a channel axis, y the rank of x");
    for (int d = 0; d < x->ndim; ++d) CHX_REQUIRE(x->shape[d] == y->shape[d], "FixedBatchNormalization: y must have the shape of x");
    const int64_t C = x->shape[1];
    CHX_PROPAGATE(check_channel_vector(s, C, "s"));
    CHX_PROPAGATE(check_channel_vector(bias, C, "bias"));
    CHX_PROPAGATE(check_channel_vector(mean, C, "mean"));
    CHX_PROPAGATE(check_channel_vector(var, C, "var"));
    BatchNormArgs a;
    memset(&a, 0, sizeof(a));
    int64_t inner_y = 1;
    CHX_REQUIRE(collapse_inner(*x, &a.inner, &a.xs[2]) && collapse_inner(*y, &inner_y, &a.ys[2]),
                "FixedBatchNormalization: the axes after the channel axis must be one dense run in x and in y");
    a.x = static_cast<const char*>(x->data);
    a.y = static_cast<char*>(y->data);
    a.s = static_cast<const float*>(s->data);
    a.bias = static_cast<const float*>(bias->data);
    a.mean = static_cast<const float*>(mean->data);
    a.var = static_cast<const float*>(var->data);
    a.xs[0] = x->strides[0]; a.xs[1] = x->strides[1];
    a.ys[0] = y->strides[0]; a.ys[1] = y->strides[1];
    a.N = x->shape[0];
    a.C = C;
    a.total = a.N * a.C * a.inner;
    if (a.total == 0) return CHX_HIP_OK;
    // the op's own adjustment, normalization.cc:217-218
    a.eps = epsilon <= 1e-5f ? (float)(1e-5 + 1e-12) : epsilon;
    a.channels_fastest = y->strides[1] == 4 && a.inner > 1;
    fixed_batch_norm_f32_kernel<<<(unsigned)((a.total + 255) / 256), 256, 0, as_stream(stream)>>>(a);
    return launch_check("fixed_batch_norm_f32_kernel");
}
