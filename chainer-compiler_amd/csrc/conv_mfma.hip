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
// Work-group: four wavefronts in a 2x2 grid over a tile of (64*FM) output channels x
// (64*FN) pixels, 64 K-bytes per step; each wavefront owns FM x FN MFMA tiles of 32x32.
// Global memory latency is covered by keeping three K steps in flight in registers
// ahead of the double-buffered LDS stage that is being consumed.  The 16-byte chunks of
// an LDS row are XOR-swizzled with bits 2..3 of the row index so that the 128-bit LDS
// reads of a wavefront's 16-lane groups fall on distinct banks.
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

// Few input channels (the 3-channel stem): padding each filter tap to 64 K-bytes would waste
// most of the matrix-core work, so the taps are packed densely instead.  The weights become
// [OCpad][Kd] with k = (kh*KW + kw)*C + c, Kd = KH*KW*C rounded up to 64, and the activations
// are expanded once into an explicit [M][Kd] matrix (im2col) that the MFMA kernel then reads
// as a 1x1 convolution over Kd "channels".  Out-of-image taps hold the zero point, K padding
// holds anything (its weights are zero).
__global__ __launch_bounds__(256) void pack_weights_dense_kernel(
        const char* __restrict__ w, int64_t s_oc, int64_t s_c, int64_t s_kh, int64_t s_kw, int OC, int C, int KH, int KW,
        int Kd, int8_t* __restrict__ wp, int32_t* __restrict__ wsum) {
    const int oc = blockIdx.x;
    int8_t* dst = wp + (int64_t)oc * Kd;
    const int K = KH * KW * C;
    int32_t local = 0;
    for (int k = threadIdx.x; k < Kd; k += 256) {
        int8_t v = 0;
        if (oc < OC && k < K) {
            const int c = k % C;
            const int pos = k / C;
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

// One lane writes one 16-byte chunk of one row of the [M][Kd] matrix.
__global__ __launch_bounds__(256) void im2col_dense_kernel(Im2colArgs a) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int chunks = a.Kd / 16;
    if (idx >= a.M * chunks) return;
    const int ch = (int)(idx % chunks);
    const int64_t m = idx / chunks;
    const int ow = (int)(m % a.OW);
    const int64_t r = m / a.OW;
    const int oh = (int)(r % a.OH);
    const int n = (int)(r / a.OH);
    const int K = a.KH * a.KW * a.C;
    const char* xn = a.x + (int64_t)n * a.xs[0];
    const int ih0 = oh * a.sh - a.ph, iw0 = ow * a.sw - a.pw;
    // (kh, kw, c) of the chunk's first element; then walk c fastest, kw, kh
    int k = ch * 16;
    int c = k % a.C;
    int pos = k / a.C;
    int kh = pos / a.KW, kw = pos % a.KW;
    uint32_t out[4] = {0, 0, 0, 0};
#pragma unroll
    for (int e = 0; e < 16; ++e, ++k) {
        uint32_t v = (uint32_t)a.fill & 0xffu;
        if (k < K) {
            const int ih = ih0 + kh, iw = iw0 + kw;
            if ((unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W)
                v = *reinterpret_cast<const uint8_t*>(xn + (int64_t)c * a.xs[1] + (int64_t)ih * a.xs[2] + (int64_t)iw * a.xs[3]);
        }
        out[e >> 2] |= v << (8 * (e & 3));
        if (++c == a.C) {
            c = 0;
            if (++kw == a.KW) {
                kw = 0;
                ++kh;
            }
        }
    }
    v4i o = {(int)out[0], (int)out[1], (int)out[2], (int)out[3]};
    *reinterpret_cast<v4i*>(a.col + m * a.Kd + ch * 16) = o;
}

// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ int lds_chunk_offset(int row, int kc) {
    return row * kBK + ((kc ^ ((row >> 2) & 3)) << 4);
}

// FM x FN MFMA tiles (32x32) per wavefront; four wavefronts in a 2x2 grid per work-group.
// Tile = (64*FM) output channels x (64*FN) pixels.
//
// Work-groups are persistent: each owns one output-channel tile and walks over pixel tiles
// px_first, px_first + px_step, ...  The sequence of (pixel tile, K step) pairs is one flat
// pipeline: global loads run D steps ahead of the MFMAs and cross tile boundaries, so the
// loads of the next tile are in flight while the current tile is finished and written out.
//
// kPad: some filter tap can fall outside the image, or the channel count is not a multiple
// of 64.  Then each staged row carries a bit mask of its valid taps (computed once per pixel
// tile) and invalid chunks are replaced by the zero point on their way into LDS.  Without
// kPad (1x1 and other unpadded convolutions on 64-multiple channels, matrix products) every
// load is valid and the per-step work on the vector ALU is one address add and the sign flip.
template <int FM, int FN, bool kXUnsigned, bool kOutInt32, bool kRne, bool kPad>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void conv_mfma_kernel(ConvMfmaArgs a) {
    constexpr int T = 256;
    constexpr int TM = 64 * FM;  // output channels per tile
    constexpr int TN = 64 * FN;  // pixels per tile
    constexpr int D = 3;         // K steps in flight between global memory and LDS
    constexpr int STAGE_BYTES = (TM + TN) * kBK;
    constexpr int OUT_PITCH = TM + 16;  // staging row pitch in bytes, keeps 16-byte alignment
    constexpr int LDS_OUT = kOutInt32 ? 16 : TN * OUT_PITCH;
    __shared__ __attribute__((aligned(16))) char lds[2 * STAGE_BYTES];
    __shared__ __attribute__((aligned(16))) char lds_out[LDS_OUT];
    __shared__ float s_scale[TM];
    __shared__ int32_t s_add[TM];
    __shared__ float s_fbias[TM];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // Work-group ids go round-robin over the 8 XCDs, each with its own L2.  Every XCD gets one
    // contiguous range of pixel tiles (neighbouring tiles share halo rows) and runs all
    // output-channel tiles of a pixel tile side by side, so an activation tile is fetched into
    // that L2 once and reused by tiles_oc work-groups; only the small weight tensor is read by
    // every XCD.
    const int xcd = blockIdx.x & 7;
    const int idx = blockIdx.x >> 3;
    const int oc_tile = idx % a.tiles_oc;
    const int slot = idx / a.tiles_oc;
    const int px_step = (gridDim.x >> 3) / a.tiles_oc;  // pixel-tile slots per XCD
    const int px_lo = (int)(((int64_t)a.tiles_px * xcd) >> 3);
    const int px_hi = (int)(((int64_t)a.tiles_px * (xcd + 1)) >> 3);
    const int px_first = px_lo + slot;
    const int oc0 = oc_tile * TM;
    const int my_tiles = px_first < px_hi ? (px_hi - px_first + px_step - 1) / px_step : 0;
    const int nk = a.nk;
    const int total_stages = my_tiles * nk;

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

    // chunks this thread stages per K step: FM of the weight tile, FN of the activation tile;
    // chunk q = tid + j*256 -> row q/4, 16-byte K chunk q%4
    const int kc = tid & 3;
    const int row0 = tid >> 2;  // rows row0 + 64*j
    const int8_t* wp_row[FM];
#pragma unroll
    for (int j = 0; j < FM; ++j) wp_row[j] = a.wp + (int64_t)(oc0 + row0 + 64 * j) * a.KP + kc * 16;

    const int fill_byte = kXUnsigned ? ((a.x_zp ^ 0x80) & 0xff) : (a.x_zp & 0xff);
    const int fill_word = (int)((unsigned)fill_byte * 0x01010101u);

    // ---- load side state: which (pixel tile, K step) the next global load fetches ----
    const char* xb[FN];
    int ld_tile = px_first;
    int ld_k = 0, kh = 0, kw = 0, c0 = 0, kofs = 0;
    int64_t tap_off = 0;  // kh * x_h_stride + kw * x_w_stride

    uint64_t tapmask[FN];  // kPad: bit (kh*KW + kw) set when that tap of the row's pixel is inside the image
    int tap = 0;

    auto set_load_tile = [&]() {
        const int64_t mbase = (int64_t)ld_tile * TN + row0;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const int64_t m = mbase + 64 * j;
            const bool row_ok = m < a.M && ld_tile < px_hi;
            // rows past the end re-read the last pixel; they are never written back
            const uint32_t mm = m < a.M ? (uint32_t)m : (uint32_t)(a.M - 1);  // M fits 31 bits (checked on the host)
            const uint32_t ow = mm % (uint32_t)a.OW;
            const uint32_t r = mm / (uint32_t)a.OW;
            const uint32_t oh = r % (uint32_t)a.OH;
            const uint32_t n = r / (uint32_t)a.OH;
            const int ih0 = (int)oh * a.sh - a.ph;
            const int iw0 = (int)ow * a.sw - a.pw;
            xb[j] = a.x + (int64_t)n * a.x_n_stride + (int64_t)ih0 * a.x_h_stride + (int64_t)iw0 * a.x_w_stride + kc * 16;
            if (kPad) {
                uint64_t mask = 0;
                if (row_ok) {
                    for (int t = 0, i = 0; i < a.KH; ++i)
                        for (int jj = 0; jj < a.KW; ++jj, ++t)
                            if ((unsigned)(ih0 + i) < (unsigned)a.H && (unsigned)(iw0 + jj) < (unsigned)a.W)
                                mask |= (uint64_t)1 << t;
                }
                tapmask[j] = mask;
            }
        }
    };
    set_load_tile();

    // Loads are unconditional (an invalid chunk reads the tensor's first bytes instead) and
    // nothing consumes a loaded value here; the fill value and the sign flip are applied when
    // the stage is written to LDS, several K steps later, so the loads stay in flight.
    auto load_global = [&](v4i* pa, v4i* pb, uint32_t& okmask) {
#pragma unroll
        for (int j = 0; j < FM; ++j) pa[j] = *reinterpret_cast<const v4i*>(wp_row[j] + kofs);
        okmask = 0;
        if (kPad) {
            const bool c_ok = c0 + kc * 16 < a.C16;
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const bool ok = c_ok && ((tapmask[j] >> tap) & 1u);
                const char* src = ok ? xb[j] + tap_off + c0 : a.x;
                pb[j] = *reinterpret_cast<const v4i*>(src);
                okmask |= (ok ? 1u : 0u) << j;
            }
        } else {
#pragma unroll
            for (int j = 0; j < FN; ++j) pb[j] = *reinterpret_cast<const v4i*>(xb[j] + tap_off + c0);
        }
        // advance to the next K step, or to the first K step of this work-group's next pixel tile
        if (++ld_k == nk) {
            ld_k = 0; kh = 0; kw = 0; c0 = 0; kofs = 0; tap_off = 0; tap = 0;
            ld_tile += px_step;
            set_load_tile();
        } else {
            kofs += kBK;
            c0 += kBK;
            if (c0 >= a.C64) {
                c0 = 0;
                ++tap;
                tap_off += a.x_w_stride;
                if (++kw == a.KW) {
                    kw = 0;
                    ++kh;
                    tap_off = (int64_t)kh * a.x_h_stride;
                }
            }
        }
    };
    auto store_lds = [&](int buf, const v4i* pa, const v4i* pb, uint32_t okmask) {
        char* sa = lds + buf * STAGE_BYTES;
        char* sb = sa + TM * kBK;
#pragma unroll
        for (int j = 0; j < FM; ++j) *reinterpret_cast<v4i*>(sa + lds_chunk_offset(row0 + 64 * j, kc)) = pa[j];
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            v4i v = pb[j];
            if (kXUnsigned) v ^= (int)0x80808080;
            if (kPad) {
                const bool ok = (okmask >> j) & 1u;
                v[0] = ok ? v[0] : fill_word;
                v[1] = ok ? v[1] : fill_word;
                v[2] = ok ? v[2] : fill_word;
                v[3] = ok ? v[3] : fill_word;
            }
            *reinterpret_cast<v4i*>(sb + lds_chunk_offset(row0 + 64 * j, kc)) = v;
        }
    };

    v16i acc[FM][FN];
    auto zero_acc = [&]() {
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
    };
    zero_acc();

    // ---- epilogue of one finished pixel tile ----
    // lane holds, per 32x32 MFMA tile: pixel column (lane & 31), output-channel rows
    // (v / 4) * 8 + (lane >> 5) * 4 + (v % 4)
    auto epilogue = [&](int px_tile) {
        const int64_t m0 = (int64_t)px_tile * TN;
        if (kOutInt32) {
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    const int64_t m = m0 + wn * 32 * FN + j * 32 + (lane & 31);
                    if (m >= a.M) continue;
                    char* yrow = a.y + m * a.y_px_stride;
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int ocl = wm * 32 * FM + i * 32 + g * 8 + (lane >> 5) * 4;
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
        const bool float_bias = a.rq.bias_mode == kBiasReferenceFloat;  // uniform
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int ocl = wm * 32 * FM + i * 32 + g * 8 + (lane >> 5) * 4;
                float sc[4], fb[4];
                int32_t ad[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    sc[e] = s_scale[ocl + e];
                    ad[e] = s_add[ocl + e];
                    fb[e] = float_bias ? s_fbias[ocl + e] : 0.f;
                }
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    const int pxl = wn * 32 * FN + j * 32 + (lane & 31);
                    int32_t code[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int32_t accv = acc[i][j][g * 4 + e] + ad[e];
                        float v = (float)accv * sc[e];
                        // the reference adds a float bias after the scale multiply; x + 0.0f
                        // changes nothing the quantization can see, so no branch is needed
                        v = v + fb[e];
                        const int32_t c = quantize_value_fast<kRne>(v, a.rq.q, a.inv_y_scale);
                        code[e] = c < a.rq.relu_floor ? a.rq.relu_floor : c;
                    }
                    const uint32_t packed = ((uint32_t)code[0] & 0xffu) | (((uint32_t)code[1] & 0xffu) << 8) |
                                            (((uint32_t)code[2] & 0xffu) << 16) | ((uint32_t)code[3] << 24);
                    *reinterpret_cast<uint32_t*>(lds_out + pxl * OUT_PITCH + ocl) = packed;
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
            const v4i val = *reinterpret_cast<const v4i*>(lds_out + pxl * OUT_PITCH + ch * 16);
            char* dst = a.y + m * a.y_px_stride + oc;
            if (a.y_vec_ok && oc + 16 <= a.OC) {
                *reinterpret_cast<v4i*>(dst) = val;
            } else {
                const char* src = lds_out + pxl * OUT_PITCH + ch * 16;
#pragma nounroll
                for (int e = 0; e < 16 && oc + e < a.OC; ++e) dst[e] = src[e];
            }
        }
    };

    if (total_stages == 0) return;
    v4i ra[D][FM], rb[D][FN];
    uint32_t okm[D];
    // Every iteration issues the same number of loads and none of it is conditional, so the
    // compiler can wait for exactly the stage it is about to store (vmcnt counts in order) and
    // leave the younger stages in flight.  Iterations past the end (the loop runs a multiple
    // of D) recompute a finished tile's stale LDS contents into accumulators nobody reads and
    // load from valid addresses; a tile boundary they reach belongs to no tile of this work-group and is skipped.
    // prologue: stages 0 .. D-1 in flight, stage 0 into LDS, its registers refilled with stage D
#pragma unroll
    for (int d = 0; d < D; ++d) load_global(ra[d], rb[d], okm[d]);
    store_lds(0, ra[0], rb[0], okm[0]);
    load_global(ra[0], rb[0], okm[0]);
    __syncthreads();

    const int frag_row = lane & 31;
    const int frag_kc = lane >> 5;
    int ck = 0;               // K step within the tile being computed
    int c_tile = px_first;    // pixel tile being computed
    const int iters = (total_stages + D - 1) / D * D;
    for (int s0 = 0; s0 < iters; s0 += D) {
#pragma unroll
        for (int u = 0; u < D; ++u) {
            const int cur = (s0 + u) & 1;
            const char* sa = lds + cur * STAGE_BYTES;
            const char* sb = sa + TM * kBK;
            v4i fa[2][FM], fb[2][FN];
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
                for (int i = 0; i < FM; ++i)
                    fa[sub][i] = *reinterpret_cast<const v4i*>(
                            sa + lds_chunk_offset(wm * 32 * FM + i * 32 + frag_row, sub * 2 + frag_kc));
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    fb[sub][j] = *reinterpret_cast<const v4i*>(
                            sb + lds_chunk_offset(wn * 32 * FN + j * 32 + frag_row, sub * 2 + frag_kc));
            }
#pragma unroll
            for (int sub = 0; sub < 2; ++sub)
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int j = 0; j < FN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[sub][i], fb[sub][j], acc[i][j], 0, 0, 0);
            const int nxt = (u + 1) % D;  // register set holding the next stage (static after unrolling)
            store_lds(cur ^ 1, ra[nxt], rb[nxt], okm[nxt]);
            load_global(ra[nxt], rb[nxt], okm[nxt]);
            if (++ck == nk) {
                if (c_tile < px_hi) epilogue(c_tile);  // iterations past the end own no tile
                zero_acc();
                ck = 0;
                c_tile += px_step;
            }
            __syncthreads();
        }
    }
}

template <int FM, int FN>
int launch_config(const ConvMfmaArgs& a, bool x_unsigned, bool out_int32, bool rne, hipStream_t s) {
    // persistent work-groups: as many as the device holds at once, a whole number per
    // output-channel tile
    static int resident = 0;  // per (FM, FN); the variants of one tile shape use about the same resources
    if (resident == 0) {
        int dev = 0, cus = 256, per_cu = 2;
        if (hipGetDevice(&dev) == hipSuccess) {
            hipDeviceProp_t prop;
            if (hipGetDeviceProperties(&prop, dev) == hipSuccess) cus = prop.multiProcessorCount;
        }
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(
                    &per_cu, reinterpret_cast<const void*>(&conv_mfma_kernel<FM, FN, true, false, false, true>), 256, 0) !=
                    hipSuccess ||
            per_cu < 1)
            per_cu = 2;
        resident = cus * per_cu;
    }
    int slots = (a.tiles_px + 7) / 8;  // pixel-tile slots per XCD
    const int cap = resident / (8 * a.tiles_oc) > 0 ? resident / (8 * a.tiles_oc) : 1;
    if (slots > cap) slots = cap;
    const unsigned grid = (unsigned)(8 * a.tiles_oc * slots);
    // padding-free variant: no tap can leave the image and channels fill whole 64-byte K steps
    const bool pad = a.ph != 0 || a.pw != 0 || (a.C16 % 64) != 0 ||
                     (int64_t)(a.OH - 1) * a.sh + a.KH > a.H || (int64_t)(a.OW - 1) * a.sw + a.KW > a.W;
#define CHX_LAUNCH(XU, OI, RN)                                                           \
    do {                                                                                 \
        if (pad)                                                                         \
            conv_mfma_kernel<FM, FN, XU, OI, RN, true><<<grid, 256, 0, s>>>(a);          \
        else                                                                             \
            conv_mfma_kernel<FM, FN, XU, OI, RN, false><<<grid, 256, 0, s>>>(a);         \
    } while (0)
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

int pack_weights_dense(const chx_hip_tensor& w, int Kd, int OCpad, int8_t* wp, int32_t* wsum, hipStream_t s) {
    pack_weights_dense_kernel<<<OCpad, 256, 0, s>>>(
            static_cast<const char*>(w.data), w.strides[0], w.strides[1], w.strides[2], w.strides[3], (int)w.shape[0],
            (int)w.shape[1], (int)w.shape[2], (int)w.shape[3], Kd, wp, wsum);
    return launch_check("pack_weights_dense_kernel");
}

int launch_im2col_dense(const Im2colArgs& a, hipStream_t s) {
    const int64_t total = a.M * (a.Kd / 16);
    if (total == 0) return CHX_HIP_OK;
    im2col_dense_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(a);
    return launch_check("im2col_dense_kernel");
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
