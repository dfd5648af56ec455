// SoftmaxOp / LogSoftmaxOp::RunImpl (runtime/ops/activation.cc:66-99) on float32: chainerx::Softmax over one
// axis, or, with ONNX semantics, over the axes from `axis` on taken together.
//
//   m = max over the axis;  e = exp(x - m);  s = sum of e over the axis;  softmax = e * (1 / s)
//   log-softmax = (x - m) - log(s)                                     [not built: only Softmax]
//
// float32, one rounding per operation, exp as the host C library computes it (faithful_math.h), the sum in
// ascending order of the axis from 0.  (ChainerX's Softmax is not in the reference tree: this is the sequence of
// the CPU restatement the kernel is tested against bit for bit.)
//
// One lane per (outer, inner) position walks the axis three times (maximum, sum, result); lanes run along the
// inner positions, or along outer ones when the axis is innermost.  A coverage kernel for classifier heads.
#include <cstring>

#include "chx_internal.h"

#define FM_FN __device__ __forceinline__
#define FM_TABLE_QUALIFIER static __device__ const
#define FM_ANY_LANE(c) (__builtin_amdgcn_ballot_w64(c) != 0ull)
#include "faithful_math.h"

namespace chx {
namespace {

struct SoftmaxArgs {
    const float* x;
    float* y;
    int64_t outer, len, inner;  // x and y as dense [outer][len][inner]
};

template <bool kUseFma>
__global__ __launch_bounds__(256) void softmax_f32_kernel(SoftmaxArgs a) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= a.outer * a.inner) return;
    const int64_t o = idx / a.inner, i = idx - o * a.inner;
    const float* xp = a.x + o * a.len * a.inner + i;
    float* yp = a.y + o * a.len * a.inner + i;
    float m = xp[0];
    for (int64_t k = 1; k < a.len; ++k) {
        const float v = xp[k * a.inner];
        m = v > m ? v : m;
        m = v != v ? v : m;  // a NaN stays (numpy's and ChainerX's maximum)
    }
    float s = 0.f;
    for (int64_t k = 0; k < a.len; ++k) s = s + chx_fm::expf_faithful<kUseFma>(xp[k * a.inner] - m);
    const float r = 1.0f / s;
    for (int64_t k = 0; k < a.len; ++k) yp[k * a.inner] = chx_fm::expf_faithful<kUseFma>(xp[k * a.inner] - m) * r;
}

}  // namespace
}  // namespace chx

using namespace chx;

extern "C" int chx_hip_softmax_f32(const chx_hip_tensor* x, int32_t axis, int32_t is_onnx_semantics, chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(x, "Softmax x"));
    CHX_PROPAGATE(check_tensor(y, "Softmax y"));
    CHX_REQUIRE(x->dtype == CHX_HIP_FLOAT32 && y->dtype == CHX_HIP_FLOAT32, "Softmax: x and y must be float32");
    CHX_REQUIRE(x->ndim >= 1 && same_shape(*x, *y), "Softmax: y must have the shape of x (rank 1 or more)");
    if (axis < 0) axis += x->ndim;
    CHX_REQUIRE(axis >= 0 && axis < x->ndim, "Softmax: axis out of range for rank %d", x->ndim);
    CHX_REQUIRE(is_contiguous(*x) && is_contiguous(*y), "Softmax: x and y must be contiguous");
    SoftmaxArgs a;
    a.x = static_cast<const float*>(x->data);
    a.y = static_cast<float*>(y->data);
    a.outer = 1;
    a.len = 1;
    a.inner = 1;
    for (int d = 0; d < axis; ++d) a.outer *= x->shape[d];
    if (is_onnx_semantics) {
        for (int d = axis; d < x->ndim; ++d) a.len *= x->shape[d];
    } else {
        a.len = x->shape[axis];
        for (int d = axis + 1; d < x->ndim; ++d) a.inner *= x->shape[d];
    }
    if (a.outer * a.len * a.inner == 0) return CHX_HIP_OK;
    const unsigned blocks = (unsigned)((a.outer * a.inner + 255) / 256);
    if (host_libm_uses_fma()) softmax_f32_kernel<true><<<blocks, 256, 0, as_stream(stream)>>>(a);
    else softmax_f32_kernel<false><<<blocks, 256, 0, as_stream(stream)>>>(a);
    return launch_check("softmax_f32_kernel");
}
