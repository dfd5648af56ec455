// Internal interface between the contraction entry points (contract_api.hip) and the
// kernels that implement them (contract_generic.hip, conv_mfma.hip).
#pragma once

#include "chx_internal.h"
#include "quant_math.h"

namespace chx {

struct ConvDirectArgs {
    const char* x;
    const char* w;
    char* y;
    int64_t xs[4], ws[4], ys[4];  // byte strides of NCHW / OIHW / NCHW axes
    int32_t N, C, H, W, OC, Cg, KH, KW, OH, OW;
    int32_t sh, sw, ph, pw, group;
    // a third (outermost) spatial axis, for 3-D convolutions; D = KD = OD = 1, sd = 1, pd = 0 otherwise
    int32_t D, KD, OD, sd, pd;
    int64_t xsd, wsd, ysd;  // byte strides of that axis in x, w and y
    int32_t x_signed, w_signed;
    int32_t x_zp;
    const char* w_zp;  // device, dtype of w
    int32_t w_zp_len;  // 0 absent, 1 scalar, OC per channel
    int64_t w_zp_stride;
    int64_t total;
    // epilogue
    int32_t requant;  // 0: int32 output
    const float* w_scale;
    int32_t w_scale_len;
    const int32_t* bias;
    RequantParams rq;
};

struct MatMulDirectArgs {
    const char* a;
    const char* b;
    char* y;
    int64_t a_batch, a_row, a_col;  // byte strides
    int64_t b_batch, b_row, b_col;
    int64_t y_batch, y_row, y_col;
    int64_t M, K, N, total;
    int32_t a_signed, b_signed;
    const char* a_zp;
    const char* b_zp;
    int32_t a_zp_len, b_zp_len;  // 0 absent, 1 scalar, K (a) / N (b) along the last axis
    int64_t a_zp_stride, b_zp_stride;
    int32_t a_zp_signed, b_zp_signed;
    int32_t a_zp_imm, b_zp_imm;  // host-side scalar zero points, subtracted as well
    int32_t requant;
    float b_scale;
    const int32_t* bias;
    RequantParams rq;
};

int launch_conv_direct(const ConvDirectArgs& a, bool rne, hipStream_t s);
int launch_matmul_direct(const MatMulDirectArgs& a, bool rne, hipStream_t s);

}  // namespace chx
