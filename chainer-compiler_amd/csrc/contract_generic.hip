// Direct (one thread per output element) integer convolution and matrix product with
// exact int32 accumulation.  These kernels take every case the ops allow -- any
// strides on x, w and y, groups, uint8 or int8 on either side, scalar or per-channel
// weight zero points, asymmetric padding -- and are what runs when a case is outside
// the MFMA kernels' domain.  Results are identical to the MFMA path by construction:
// integer sums do not depend on the order of summation and both share the epilogue in
// quant_math.h.
#include "contract.h"

namespace chx {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ int32_t load8(const char* p, bool is_signed) {
    const uint8_t raw = *reinterpret_cast<const uint8_t*>(p);
    return is_signed ? (int32_t)(int8_t)raw : (int32_t)raw;
}

template <bool kRne>
__global__ __launch_bounds__(kThreads) void conv_direct_kernel(ConvDirectArgs a) {
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= a.total) return;
    // idx enumerates (n, od, oh, ow, oc) with oc fastest: neighbouring lanes share the input window
    const int oc = (int)(idx % a.OC);
    int64_t rest = idx / a.OC;
    const int ow = (int)(rest % a.OW);
    rest /= a.OW;
    const int oh = (int)(rest % a.OH);
    rest /= a.OH;
    const int od = (int)(rest % a.OD);
    const int n = (int)(rest / a.OD);
    const int OCg = a.OC / a.group;
    const int grp = oc / OCg;
    int32_t wz = 0;
    if (a.w_zp_len == 1) wz = load8(a.w_zp, a.w_signed);
    if (a.w_zp_len > 1) wz = load8(a.w_zp + (int64_t)oc * a.w_zp_stride, a.w_signed);
    int32_t acc = 0;
    const char* wbase = a.w + (int64_t)oc * a.ws[0];
    for (int c = 0; c < a.Cg; ++c) {
        const char* xc = a.x + (int64_t)n * a.xs[0] + (int64_t)(grp * a.Cg + c) * a.xs[1];
        const char* wc = wbase + (int64_t)c * a.ws[1];
        for (int kd = 0; kd < a.KD; ++kd) {
            const int id = od * a.sd - a.pd + kd;
            if (id < 0 || id >= a.D) continue;
            for (int kh = 0; kh < a.KH; ++kh) {
                const int ih = oh * a.sh - a.ph + kh;
                if (ih < 0 || ih >= a.H) continue;
                for (int kw = 0; kw < a.KW; ++kw) {
                    const int iw = ow * a.sw - a.pw + kw;
                    if (iw < 0 || iw >= a.W) continue;
                    const int32_t xv = load8(xc + (int64_t)id * a.xsd + (int64_t)ih * a.xs[2] + (int64_t)iw * a.xs[3], a.x_signed) - a.x_zp;
                    const int32_t wv = load8(wc + (int64_t)kd * a.wsd + (int64_t)kh * a.ws[2] + (int64_t)kw * a.ws[3], a.w_signed) - wz;
                    acc += xv * wv;
                }
            }
        }
    }
    char* yp = a.y + (int64_t)n * a.ys[0] + (int64_t)oc * a.ys[1] + (int64_t)od * a.ysd + (int64_t)oh * a.ys[2] + (int64_t)ow * a.ys[3];
    if (!a.requant) {
        *reinterpret_cast<int32_t*>(yp) = acc;
        return;
    }
    const float wsc = a.w_scale_len > 1 ? a.w_scale[oc] : a.w_scale[0];
    const int32_t b = a.bias ? a.bias[oc] : 0;
    *reinterpret_cast<uint8_t*>(yp) = (uint8_t)requantize_value<kRne>(acc, wsc, b, a.rq);
}

template <bool kRne>
__global__ __launch_bounds__(kThreads) void matmul_direct_kernel(MatMulDirectArgs a) {
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= a.total) return;
    const int64_t j = idx % a.N;
    const int64_t rest = idx / a.N;
    const int64_t i = rest % a.M;
    const int64_t bt = rest / a.M;
    const char* ap = a.a + bt * a.a_batch + i * a.a_row;
    const char* bp = a.b + bt * a.b_batch + j * a.b_col;
    int32_t bz = a.b_zp_imm;
    if (a.b_zp_len == 1) bz = load8(a.b_zp, a.b_zp_signed);
    if (a.b_zp_len > 1) bz = load8(a.b_zp + j * a.b_zp_stride, a.b_zp_signed);
    int32_t az0 = a.a_zp_imm;
    if (a.a_zp_len == 1) az0 = load8(a.a_zp, a.a_zp_signed);
    int32_t acc = 0;
    for (int64_t k = 0; k < a.K; ++k) {
        int32_t av = load8(ap + k * a.a_col, a.a_signed) - az0;
        if (a.a_zp_len > 1) av -= load8(a.a_zp + k * a.a_zp_stride, a.a_zp_signed);
        const int32_t bv = load8(bp + k * a.b_row, a.b_signed) - bz;
        acc += av * bv;
    }
    char* yp = a.y + bt * a.y_batch + i * a.y_row + j * a.y_col;
    if (!a.requant) {
        *reinterpret_cast<int32_t*>(yp) = acc;
        return;
    }
    const int32_t b = a.bias ? a.bias[j] : 0;
    *reinterpret_cast<uint8_t*>(yp) = (uint8_t)requantize_value<kRne>(acc, a.b_scale, b, a.rq);
}

}  // namespace

int launch_conv_direct(const ConvDirectArgs& a, bool rne, hipStream_t s) {
    if (a.total == 0) return CHX_HIP_OK;
    const unsigned blocks = (unsigned)((a.total + kThreads - 1) / kThreads);
    if (rne)
        conv_direct_kernel<true><<<blocks, kThreads, 0, s>>>(a);
    else
        conv_direct_kernel<false><<<blocks, kThreads, 0, s>>>(a);
    return launch_check("conv_direct_kernel");
}

int launch_matmul_direct(const MatMulDirectArgs& a, bool rne, hipStream_t s) {
    if (a.total == 0) return CHX_HIP_OK;
    const unsigned blocks = (unsigned)((a.total + kThreads - 1) / kThreads);
    if (rne)
        matmul_direct_kernel<true><<<blocks, kThreads, 0, s>>>(a);
    else
        matmul_direct_kernel<false><<<blocks, kThreads, 0, s>>>(a);
    return launch_check("matmul_direct_kernel");
}

}  // namespace chx
