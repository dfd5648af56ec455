// Interface of the MFMA implicit-GEMM kernel (conv_mfma.hip) and the layout helpers
// (layout.hip) towards the entry points.
#pragma once

#include "chx_internal.h"
#include "quant_math.h"

namespace chx {

// A residual sum fused behind the requantization: the 8-bit code c of the convolution is not
// written; the kernel writes  Q_out( act( DQ_y(c) + DQ_r(r) ) )  instead, which is what a
// QLinearConv followed by the element-wise group {DequantizeLinear, DequantizeLinear, Add,
// [Relu], QuantizeLinear} computes, operation by operation.  A signed code is read as
// (byte ^ 0x80) - 128, so the flips and the "+128" below make one code path serve both types.
struct ResidualAdd {
    const char* r;         // pixel-major like y: element (m, oc) at r + m*r_px_stride + oc
    int64_t r_px_stride;
    int32_t r_vec_ok;      // 16-byte loads allowed
    uint32_t c_flip;       // 0x80808080 when the convolution's code is int8
    uint32_t r_flip;       // ... when r is int8
    float c_zpf;           // y_zero_point (+128 for int8), as float
    float c_scale;         // y_scale
    float r_zpf;           // r's zero point (+128 for int8)
    float r_scale;
    int32_t relu;
    QuantParams out;       // quantization of the sum
    float inv_out_scale;
    float big;             // 2^40 * out.scale: the dividend is limited to +-big (both sides saturate beyond)
    int32_t guard;         // 0 when the operand scales already keep every sum far inside +-big
    int32_t lean;          // uint8 result with zero point 0 and r with zero point 0: see add_residual16
    // The sum as two fused multiply-adds, floor((c * kc + (r * kr + k0))) saturated to [0, 255] (and not below
    // floor_pre when a Relu is part of the group): set only after find_affine_residual has found constants for which
    // this gives the byte of the operation-by-operation arithmetic for every one of the 65536 pairs of codes.
    int32_t affine;
    float kc, kr, k0, floor_pre;
};

// Number of constant triples find_affine_residual tries: the float32 neighbours of the real-valued constants.
constexpr int kAffineCandidates = 5 * 5 * 13;

struct ConvMfmaArgs {
    // activations, channels-last: element (n, c, ih, iw) at x + n*x_n_stride + ih*x_h_stride + iw*x_w_stride + c
    // The bytes [x, x + x_bytes) hold every element of x and nothing the kernel may not read; x_bytes and every
    // stride are below 2^31 (the kernel addresses x with 32-bit offsets through a buffer resource).
    const char* x;
    int64_t x_n_stride, x_h_stride, x_w_stride;
    uint32_t x_bytes;
    uint32_t x_bias;  // filled by the launcher: what the kernel adds to every offset into x so that taps in the padding stay non-negative
    int32_t C16;  // channels rounded up to 16; the pixel pitch covers at least this many bytes
    int32_t C64;  // channels rounded up to 64 (K bytes per filter tap in the packed weights)
    int32_t H, W, OH, OW, KH, KW, sh, sw, ph, pw;
    int64_t M;    // N * OH * OW
    int32_t OC;
    int32_t bk;   // K bytes per step: 64, or 128 when C64 is a multiple of 128
    int32_t nk;   // K steps: KP / bk
    int32_t KP;   // packed row length: KH * KW * C64
    const int8_t* wp;     // [OCpad / 64][nk][64][bk]
    const int32_t* wsum;  // [OCpad]
    // [16][OCpad]: the sum of a filter's weights over the taps of its first row (class bit 3), last row (bit 2), first
    // column (bit 1) and last column (bit 0), each tap once: what a pixel whose window leaves the image on those sides
    // misses when the taps outside arrive as zeros (pack_weights); null when the packing did not compute it
    const int32_t* padsum;
    int32_t padsum_stride;  // channels per class of padsum
    int32_t x_zp;
    int32_t corr_mult;    // (128 - x_zp) for uint8 x, (-x_zp) for int8 x
    int32_t tap_corr;     // not 0: taps outside the image arrive as zeros although the zero point is not the byte 0, and the accumulators start from the pixel's class of padsum; the number of classes other than 0 that occur (launcher)
    uint64_t tap_classes; // those classes (at most eight), four bits each from bit 0 up (launcher)
    uint64_t tap_rows;    // per class (four bits each, class c at bit 4c): its row of the work-group's seed table, the class's place in tap_classes + 1; 0 for class 0 (launcher)
    // output, pixel-major: element (m, oc) at y + m*y_px_stride + oc*elemsize
    char* y;
    int64_t y_px_stride;
    int32_t y_vec_ok;     // 16-byte stores allowed (base and pitch aligned)
    uint32_t y_flip;      // 0x80808080: every stored byte is the code minus 128 (CHX_HIP_STORE_MINUS_128), else 0
    // epilogue
    const float* w_scale;
    int32_t w_scale_len;
    const int32_t* bias;
    RequantParams rq;
    float inv_y_scale;           // 1 / y_scale, for the division-free requantization
    float lo_folded;             // lower clamp bound with the fused Relu folded in (fold_relu_floor)
    int32_t tiles_oc, tiles_px;  // filled by the launcher
    uint32_t ow_mul, ow_shift, oh_mul, oh_shift;  // magic_divisor(OW), magic_divisor(OH), filled by the launcher
    uint32_t row_unit;           // bit i*KW set for every filter row i (when KH*KW <= 32), filled by the launcher
    uint32_t tiles_oc_mul, tiles_oc_shift;  // magic_divisor(tiles_oc), filled by the launcher
    int32_t px_slots;                       // pixel-tile slots per XCD of the launch's grid: gridDim.x / 8 / tiles_oc (launcher)
    uint32_t px_slots_mul, px_slots_shift;  // magic_divisor(px_slots)
    uint32_t tap_step_col, tap_step_row;  // what the scalar offset into x gains from the last K step of a filter tap to the first of the next: one pixel to the right, or to the first column of the next filter row (launcher)
    int32_t px_linear;           // 1x1, stride 1, no padding over a dense image: input pixel m is at x + m * x_w_stride (launcher)
    ResidualAdd res;             // res.r == nullptr: plain QLinearConv
    // Two convolutions of the same input in one launch (oc_split > 0): the weights hold both filter sets one after the
    // other; output channels [0, oc_split) are the first convolution's and go to y with rq.q / inv_y_scale /
    // lo_folded, channels [oc_split, OC) are the second's and go to y2 (its channel oc - oc_split) with the set below.
    // oc_split is a multiple of the tile's output channels, so a tile belongs to one of the two whole.
    int32_t oc_split;
    char* y2;
    int64_t y2_px_stride;
    int32_t y2_vec_ok;
    uint32_t y2_flip;
    QuantParams q2;
    float inv_y_scale2;
    float lo_folded2;
};

// Direct convolution over planar activations with few channels (conv_stem.hip).
struct ConvStemArgs {
    // activations, rows contiguous: element (n, c, ih, iw) at x + n*x_n_stride + c*x_c_stride + ih*x_h_stride + iw
    const char* x;
    int64_t x_n_stride, x_c_stride, x_h_stride;
    int32_t N, C, H, W, OH, OW, KH, KW, sh, sw, ph, pw;
    int32_t OC;
    const int8_t* wd;     // pack_weights_stem
    const int32_t* wsum;  // [OC padded]
    int32_t x_zp;
    int32_t x_unsigned;
    int32_t corr_mult;    // (128 - x_zp) for uint8 x, (-x_zp) for int8 x
    char* y;              // pixel-major, as for ConvMfmaArgs
    int64_t y_px_stride;
    int32_t y_vec_ok;
    const float* w_scale;
    int32_t w_scale_len;
    const int32_t* bias;
    RequantParams rq;
    float inv_y_scale;
    float lo_folded;
    // filled by the launcher
    int32_t KB, tiles_h, tiles_w, tiles;
    uint32_t m_ppw, m_ph, m_kh;
    uint32_t tpi_mul, tpi_shift, tw_mul, tw_shift;  // magic_divisor(tiles per image), magic_divisor(tiles_w)
};

struct Im2colArgs {
    const char* x;
    int64_t xs[4];  // byte strides of N, C, H, W
    int32_t C, H, W, OH, OW, KH, KW, sh, sw, ph, pw;
    int32_t Kd;     // row length of the expanded matrix, a multiple of 64
    int32_t fill;   // the activation zero point (raw code)
    int64_t M;
    char* col;      // [M][Kd]
};

// Multiplier and shift with n / d == (mulhi(n, mul) + n) >> shift for every n < 2^31 (d >= 1).
inline void magic_divisor(uint32_t d, uint32_t* mul, uint32_t* shift) {
    uint32_t l = 0;
    while ((uint64_t(1) << l) < d) ++l;
    *mul = (uint32_t)((((uint64_t(1) << l) - d) << 32) / d + 1);
    *shift = l;
}

int pack_weights_dense(const chx_hip_tensor& w, int Kd, int BK, int OCpad, int8_t* wp, int32_t* wsum, hipStream_t s);
int launch_im2col_dense(const Im2colArgs& a, hipStream_t s);
int pack_weights(const chx_hip_tensor& w, int C64, int BK, int OCpad, int8_t* wp, int32_t* wsum, int32_t* padsum, hipStream_t s);
// the stem kernel: weights [C][KH][KW] with C*KH <= 32 and KW <= 8; patch = LDS bytes of a tile's input rows
bool stem_shape_fits(int C, int KH, int KW);
bool stem_patch_fits(int C, int KH, int KW, int sh, int sw);
int stem_k_blocks(int C, int KH, int KW);
int pack_weights_stem(const chx_hip_tensor& w, int OCpad64, int8_t* wd, hipStream_t s);
int launch_conv_stem(ConvStemArgs a, bool rne, hipStream_t s);
// max_wgs_per_cu caps the persistent grid (0: as many work-groups as the device holds at once); waves: 4, or 8
// for the tiles 128x128, 128x256 and 64x128 (output channels x pixels)
// Looks for constants (kc, kr, k0) with which the two-multiply-add form of the residual sum equals the
// operation-by-operation one on all 65536 code pairs: every candidate is checked on the device against
// add_residual16, the mismatch counts come back to the host (synchronizes the stream).  Returns CHX_HIP_OK and sets
// p->affine (1 when a candidate without mismatch exists; then kc, kr, k0, floor_pre are filled in).  Only for uint8
// sums without the range guard; otherwise p->affine stays 0.  `scratch` holds kAffineCandidates int32 on the device.
int find_affine_residual(ResidualAdd* p, int32_t* scratch, hipStream_t s);

// One launcher per tile shape (FM x FN MFMA tiles per wavefront, K bytes per step, wavefronts along the pixels), each
// in a translation unit of its own (conv_mfma_t*.hip).
#define CHX_CONV_MFMA_TILES(X) \
    X(2, 1, 128, 4) X(2, 1, 64, 4) X(2, 2, 128, 4) X(1, 1, 128, 4) X(2, 2, 128, 2) X(2, 2, 64, 2) X(1, 2, 128, 2) X(1, 2, 64, 2) \
    X(2, 1, 128, 2) X(2, 1, 64, 2) X(1, 1, 128, 2) X(1, 1, 64, 2)
#define CHX_CONV_MFMA_DECLARE(FM, FN, BK, NWN) \
    int launch_conv_mfma_##FM##_##FN##_##BK##_##NWN(const ConvMfmaArgs& a, bool x_unsigned, bool out_int32, bool rne, int max_wgs_per_cu, hipStream_t s);
CHX_CONV_MFMA_TILES(CHX_CONV_MFMA_DECLARE)
#undef CHX_CONV_MFMA_DECLARE

int launch_conv_mfma(ConvMfmaArgs a, int tile_oc, int tile_px, int max_wgs_per_cu, int waves, bool x_unsigned, bool out_int32, bool rne,
                     hipStream_t s);

// [N][C][HW] bytes -> [N][HW][pitch] bytes (lanes c >= C of a pixel are zero filled) and back
int launch_nchw_to_nhwc_u8(const char* src, char* dst, int N, int C, int64_t HW, int pitch, hipStream_t s);
int launch_nhwc_to_nchw_u8(const char* src, char* dst, int N, int C, int64_t HW, int pitch, hipStream_t s);

}  // namespace chx
