// Interface of the depthwise 3x3 kernel (depthwise.hip) towards the entry points.
#pragma once

#include "chx_internal.h"
#include "quant_math.h"

namespace chx {

struct DepthwiseArgs {
    // activations, channels-last: element (n, c, ih, iw) at x + n*x_n_stride + ih*x_h_stride + iw*x_w_stride + c
    const char* x;
    int64_t x_n_stride, x_h_stride, x_w_stride;
    char* y;  // same convention
    int64_t y_n_stride, y_h_stride, y_w_stride;
    int32_t N, C, H, W, OH, OW, sh, sw, ph, pw;
    int32_t x_signed;       // int8 activations: codes and zero point are shifted by 128
    int32_t x_zp_u;         // zero point in the unsigned range (zp, or zp + 128 for int8)
    const int32_t* rows;    // [C/4][3][4] filter rows as byte triples (pack_depthwise)
    const int32_t* wsum;    // [C] sum of the nine weights of a channel
    const float* w_scale;   // [w_scale_len]
    int32_t w_scale_len;    // 1 or C
    float x_scale;
    const int32_t* bias;    // [C] or null
    int32_t float_bias;     // bias is added as a float after the scale multiply (reference mode), else to the accumulator
    QuantParams q;
    float inv_y_scale;
    float lo_folded;
    uint32_t y_flip;        // 0x80808080: every stored byte is the uint8 code minus 128 (CHX_HIP_STORE_MINUS_128), else 0
    int32_t oh_blocks;      // filled by the launcher
    // The launch is one-dimensional: work-group b of the device's dispatch order (which deals work-groups out to the 8
    // XCDs in turn) takes block (b % 8) * xcd_chunk + b / 8 of the (x blocks of a row strip, row strips, images) order, so
    // that each XCD works through a contiguous run of blocks and the input lines that neighbouring blocks share (the
    // filter's three columns, the halo rows of a strip) are found in that XCD's own L2.  Filled by the launcher.
    uint32_t grid_x, grid_xy, blocks, xcd_chunk;
    int64_t total;          // filled by the launcher
};

int pack_depthwise(const chx_hip_tensor& w, int32_t* rows, int32_t* wsum, hipStream_t s);
int launch_depthwise3x3(DepthwiseArgs a, bool rne, hipStream_t s);

}  // namespace chx
