// int8 implicit-GEMM convolution / matrix product on the gfx950 matrix cores.
//
//   D[oc, m] = sum_k  Wp[oc, k] * Xcol[m, k]        m = (n, oh, ow),  k = (kh, kw, c)
//
// computed with v_mfma_i32_32x32x32_i8 (exact int32 accumulation), where
//   - Wp is the weight tensor repacked once to [OC'][KH*KW][C64] int8 (C64 = C rounded
//     up to 64, zero filled), so every 64-byte K slice of a row is contiguous;
//   - Xcol is never materialised: activations are channels-last, so for a fixed
//     (kh, kw) the 64 channels of a K slice are 64 contiguous bytes of x, or the
//     padding value when the tap falls outside the image;
//   - uint8 activations are turned into int8 by flipping the top bit (x - 128) on the
//     way into LDS; the exact result is restored per output channel in the epilogue:
//         sum (x - zp) w = sum (x - 128) w + (128 - zp) * sum_k w[oc, k]
//     Out-of-image taps are filled with the zero point itself, which makes them
//     contribute (zp - zp) * w = 0, the reference's zero padding of the already
//     zero-point-subtracted tensor (runtime/chainerx_util.cc:232-274, 313-340).
//
// Work-group tile: (64*WM) output channels x (64*WN) pixels x 64 K-bytes per step,
// one wavefront per 64x64 sub-tile (2x2 MFMA tiles, 64 accumulator registers).
// Both operand tiles are staged through LDS in double buffers; the 16-byte chunks of a
// row are XOR-swizzled with bits 2..3 of the row index so that the 128-bit LDS reads
// of a wavefront's 16-lane groups fall on distinct banks.
//
// Epilogue: the requantization of quant_math.h per element, codes packed four output
// channels at a time, transposed through LDS into [pixel][oc] rows and written as
// 128-bit stores to the channels-last output.  With an int32 output (ConvInteger,
// MatMulInteger) the accumulators are stored directly.
#include "contract.h"
#include "conv_mfma.h"

namespace chx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kBK = 64;  // K bytes per step

// ---------------------------------------------------------------------------------------------
// Weight repacking: w [OC][C][KH][KW] (any strides) -> Wp [OCpad][KH*KW][C64] and
// wsum[oc] = sum of the row.  One work-group per output channel.
__global__ __launch_bounds__(256) void pack_weights_kernel(
        const char* __restrict__ w, int64_t s_oc, int64_t s_c, int64_t s_kh, int64_t s_kw, int OC, int C, int KH, int KW,
        int C64, int8_t* __restrict__ wp, int32_t* __restrict__ wsum) {
    const int oc = blockIdx.x;
    const int KP = KH * KW * C64;
    int8_t* dst = wp + (int64_t)oc * KP;
    int32_t local = 0;
    for (int k = threadIdx.x; k < KP; k += 256) {
        const int c = k % C64;
        const int pos = k / C64;
        int8_t v = 0;
        if (oc < OC && c < C) {
            const int kh = pos / KW, kw = pos % KW;
            v = *reinterpret_cast<const int8_t*>(w + oc * s_oc + c * s_c + kh * s_kh + kw * s_kw);
        }
        dst[k] = v;
        local += v;
    }
    __shared__ int32_t red[256];
    red[threadIdx.x] = local;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) wsum[oc] = red[0];
}

// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ int lds_chunk_offset(int row, int kc) {
    return row * kBK + ((kc ^ ((row >> 2) & 3)) << 4);
}

template <int WM, int WN, bool kXUnsigned, bool kOutInt32, bool kRne>
__global__ __launch_bounds__(64 * WM * WN) void conv_mfma_kernel(ConvMfmaArgs a) {
    constexpr int T = 64 * WM * WN;
    constexpr int TM = 64 * WM;  // output channels per tile
    constexpr int TN = 64 * WN;  // pixels per tile
    constexpr int A_PER_THREAD = TM * 4 / T;
    constexpr int B_PER_THREAD = TN * 4 / T;
    constexpr int STAGE_BYTES = (TM + TN) * kBK;
    constexpr int OUT_PITCH = TM + 16;  // staging row pitch in bytes, keeps 16-byte alignment
    constexpr int LDS_MAIN = 2 * STAGE_BYTES;
    constexpr int LDS_OUT = TN * OUT_PITCH;
    constexpr int LDS_BYTES = LDS_MAIN > LDS_OUT ? LDS_MAIN : LDS_OUT;
    __shared__ __attribute__((aligned(16))) char lds[LDS_BYTES];
    __shared__ float s_scale[TM];
    __shared__ int32_t s_add[TM];
    __shared__ float s_fbias[TM];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;

    // tile coordinates; consecutive work-group ids go round-robin over the 8 XCDs, so ids are
    // regrouped to keep the oc-tiles of one pixel tile on one XCD (they share its L2)
    int bid = blockIdx.x;
    const int nblk = gridDim.x;
    if ((nblk & 7) == 0) bid = (bid & 7) * (nblk >> 3) + (bid >> 3);
    const int oc_tile = bid % a.tiles_oc;
    const int px_tile = bid / a.tiles_oc;
    const int oc0 = oc_tile * TM;
    const int64_t m0 = (int64_t)px_tile * TN;

    // per-channel epilogue constants
    for (int i = tid; i < TM; i += T) {
        const int oc = oc0 + i;
        float sc = 0.f, fb = 0.f;
        int32_t add = 0;
        if (oc < a.OC) {
            add = a.corr_mult * a.wsum[oc];
            if (!kOutInt32) {
                const float wsc = a.w_scale_len > 1 ? a.w_scale[oc] : a.w_scale[0];
                sc = a.rq.x_scale * wsc;
                if (a.bias) {
                    if (a.rq.bias_mode == kBiasOnnxInt32) add += a.bias[oc];
                    if (a.rq.bias_mode == kBiasReferenceFloat) fb = (float)a.bias[oc];
                }
            }
        }
        s_scale[i] = sc;
        s_add[i] = add;
        s_fbias[i] = fb;
    }

    // activation chunks this thread stages: row (pixel) and 16-byte K chunk
    int b_row[B_PER_THREAD], b_ih0[B_PER_THREAD], b_iw0[B_PER_THREAD];
    int64_t b_base[B_PER_THREAD];
    bool b_ok[B_PER_THREAD];
    const int b_kc = tid & 3;
#pragma unroll
    for (int j = 0; j < B_PER_THREAD; ++j) {
        const int row = (tid + j * T) >> 2;
        b_row[j] = row;
        const int64_t m = m0 + row;
        b_ok[j] = m < a.M;
        const int64_t mm = b_ok[j] ? m : 0;
        const int ow = (int)(mm % a.OW);
        const int64_t r = mm / a.OW;
        const int oh = (int)(r % a.OH);
        const int n = (int)(r / a.OH);
        b_ih0[j] = oh * a.sh - a.ph;
        b_iw0[j] = ow * a.sw - a.pw;
        b_base[j] = (int64_t)n * a.x_n_stride;
    }
    const int8_t* wp_row[A_PER_THREAD];
    int a_row[A_PER_THREAD];
    const int a_kc = tid & 3;
#pragma unroll
    for (int j = 0; j < A_PER_THREAD; ++j) {
        a_row[j] = (tid + j * T) >> 2;
        wp_row[j] = a.wp + (int64_t)(oc0 + a_row[j]) * a.KP + a_kc * 16;
    }

    const int fill_byte = kXUnsigned ? ((a.x_zp ^ 0x80) & 0xff) : (a.x_zp & 0xff);
    const int fill_word = (int)((unsigned)fill_byte * 0x01010101u);
    const v4i fill = {fill_word, fill_word, fill_word, fill_word};

    v4i ra[A_PER_THREAD], rb[B_PER_THREAD];
    int kh = 0, kw = 0, c0 = 0;
    int kofs = 0;

    auto load_global = [&]() {
#pragma unroll
        for (int j = 0; j < A_PER_THREAD; ++j) ra[j] = *reinterpret_cast<const v4i*>(wp_row[j] + kofs);
        const int cc = c0 + b_kc * 16;
#pragma unroll
        for (int j = 0; j < B_PER_THREAD; ++j) {
            const int ih = b_ih0[j] + kh, iw = b_iw0[j] + kw;
            const bool ok = b_ok[j] && cc < a.C16 && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W;
            v4i v = fill;
            if (ok) {
                v = *reinterpret_cast<const v4i*>(a.x + b_base[j] + (int64_t)ih * a.x_h_stride + (int64_t)iw * a.x_w_stride + cc);
                if (kXUnsigned) v ^= (int)0x80808080;
            }
            rb[j] = v;
        }
        // advance (kh, kw, c0) to the next K step
        kofs += kBK;
        c0 += kBK;
        if (c0 >= a.C64) {
            c0 = 0;
            if (++kw == a.KW) {
                kw = 0;
                ++kh;
            }
        }
    };
    auto store_lds = [&](int buf) {
        char* sa = lds + buf * STAGE_BYTES;
        char* sb = sa + TM * kBK;
#pragma unroll
        for (int j = 0; j < A_PER_THREAD; ++j) *reinterpret_cast<v4i*>(sa + lds_chunk_offset(a_row[j], a_kc)) = ra[j];
#pragma unroll
        for (int j = 0; j < B_PER_THREAD; ++j) *reinterpret_cast<v4i*>(sb + lds_chunk_offset(b_row[j], b_kc)) = rb[j];
    };

    v16i acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

    const int nk = a.nk;
    load_global();
    store_lds(0);
    __syncthreads();
    const int frag_row = lane & 31;
    const int frag_kc = lane >> 5;
    for (int ks = 0; ks < nk; ++ks) {
        const int cur = ks & 1;
        if (ks + 1 < nk) load_global();
        const char* sa = lds + cur * STAGE_BYTES;
        const char* sb = sa + TM * kBK;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            v4i fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                fa[i] = *reinterpret_cast<const v4i*>(sa + lds_chunk_offset(wm * 64 + i * 32 + frag_row, sub * 2 + frag_kc));
#pragma unroll
            for (int j = 0; j < 2; ++j)
                fb[j] = *reinterpret_cast<const v4i*>(sb + lds_chunk_offset(wn * 64 + j * 32 + frag_row, sub * 2 + frag_kc));
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (ks + 1 < nk) store_lds(cur ^ 1);
        __syncthreads();
    }

    // ---- epilogue ----
    // lane holds, per 32x32 tile: pixel column (lane & 31), output-channel rows
    // (v / 4) * 8 + (lane >> 5) * 4 + (v % 4)
    if (kOutInt32) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int64_t m = m0 + wn * 64 + j * 32 + (lane & 31);
                if (m >= a.M) continue;
                char* yrow = a.y + m * a.y_px_stride;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int ocl = wm * 64 + i * 32 + g * 8 + (lane >> 5) * 4;
                    const int oc = oc0 + ocl;
                    v4i out;
#pragma unroll
                    for (int e = 0; e < 4; ++e) out[e] = acc[i][j][g * 4 + e] + s_add[ocl + e];
                    if (a.y_vec_ok && oc + 4 <= a.OC) {
                        *reinterpret_cast<v4i*>(yrow + (int64_t)oc * 4) = out;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (oc + e < a.OC) *reinterpret_cast<int32_t*>(yrow + (int64_t)(oc + e) * 4) = out[e];
                    }
                }
            }
        return;
    }

    // all waves are past their last LDS read (the loop ends with a barrier): reuse the buffers
    char* so = lds;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int pxl = wn * 64 + j * 32 + (lane & 31);
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int ocl = wm * 64 + i * 32 + g * 8 + (lane >> 5) * 4;
                uint32_t packed = 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int32_t accv = acc[i][j][g * 4 + e] + s_add[ocl + e];
                    float v = (float)accv * s_scale[ocl + e];
                    if (a.rq.bias_mode == kBiasReferenceFloat) v = v + s_fbias[ocl + e];
                    int32_t code = quantize_value<kRne>(v, a.rq.q);
                    code = code < a.rq.relu_floor ? a.rq.relu_floor : code;
                    packed |= ((uint32_t)code & 0xffu) << (8 * e);
                }
                *reinterpret_cast<uint32_t*>(so + pxl * OUT_PITCH + ocl) = packed;
            }
        }
    __syncthreads();
    constexpr int CHUNKS_PER_ROW = TM / 16;
    for (int q = tid; q < TN * CHUNKS_PER_ROW; q += T) {
        const int pxl = q / CHUNKS_PER_ROW;
        const int ch = q % CHUNKS_PER_ROW;
        const int64_t m = m0 + pxl;
        const int oc = oc0 + ch * 16;
        if (m >= a.M || oc >= a.OC) continue;
        const v4i val = *reinterpret_cast<const v4i*>(so + pxl * OUT_PITCH + ch * 16);
        char* dst = a.y + m * a.y_px_stride + oc;
        if (a.y_vec_ok && oc + 16 <= a.OC) {
            *reinterpret_cast<v4i*>(dst) = val;
        } else {
            const char* src = so + pxl * OUT_PITCH + ch * 16;
            for (int e = 0; e < 16 && oc + e < a.OC; ++e) dst[e] = src[e];
        }
    }
}

template <int WM, int WN>
int launch_config(const ConvMfmaArgs& a, bool x_unsigned, bool out_int32, bool rne, hipStream_t s) {
    const unsigned grid = (unsigned)(a.tiles_oc * a.tiles_px);
    const unsigned threads = 64 * WM * WN;
#define CHX_LAUNCH(XU, OI, RN) conv_mfma_kernel<WM, WN, XU, OI, RN><<<grid, threads, 0, s>>>(a)
    if (out_int32) {
        if (x_unsigned) CHX_LAUNCH(true, true, false);
        else CHX_LAUNCH(false, true, false);
    } else if (rne) {
        if (x_unsigned) CHX_LAUNCH(true, false, true);
        else CHX_LAUNCH(false, false, true);
    } else {
        if (x_unsigned) CHX_LAUNCH(true, false, false);
        else CHX_LAUNCH(false, false, false);
    }
#undef CHX_LAUNCH
    return launch_check("conv_mfma_kernel");
}

}  // namespace

int pack_weights(
        const chx_hip_tensor& w, int C64, int OCpad, int8_t* wp, int32_t* wsum, hipStream_t s) {
    pack_weights_kernel<<<OCpad, 256, 0, s>>>(
            static_cast<const char*>(w.data), w.strides[0], w.strides[1], w.strides[2], w.strides[3], (int)w.shape[0],
            (int)w.shape[1], (int)w.shape[2], (int)w.shape[3], C64, wp, wsum);
    return launch_check("pack_weights_kernel");
}

int launch_conv_mfma(ConvMfmaArgs a, int tile_oc, int tile_px, bool x_unsigned, bool out_int32, bool rne, hipStream_t s) {
    a.tiles_oc = (a.OC + tile_oc - 1) / tile_oc;
    a.tiles_px = (int)((a.M + tile_px - 1) / tile_px);
    if (a.M == 0 || a.OC == 0) return CHX_HIP_OK;
    if (tile_oc == 128 && tile_px == 128) return launch_config<2, 2>(a, x_unsigned, out_int32, rne, s);
    if (tile_oc == 64 && tile_px == 128) return launch_config<1, 2>(a, x_unsigned, out_int32, rne, s);
    if (tile_oc == 128 && tile_px == 64) return launch_config<2, 1>(a, x_unsigned, out_int32, rne, s);
    if (tile_oc == 64 && tile_px == 64) return launch_config<1, 1>(a, x_unsigned, out_int32, rne, s);
    CHX_FAIL(CHX_HIP_EINVAL, "conv_mfma: no kernel for a %dx%d tile", tile_oc, tile_px);
}

}  // namespace chx
