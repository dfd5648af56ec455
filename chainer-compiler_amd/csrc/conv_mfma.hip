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
//     fragments read back from LDS; the exact result is restored by the accumulator seed:
//         sum (x - zp) w = sum (x - 128) w + (128 - zp) * sum_k w[oc, k]
//     Out-of-image taps are filled with the zero point itself, which makes them
//     contribute (zp - zp) * w = 0, the reference's zero padding of the already
//     zero-point-subtracted tensor (runtime/chainerx_util.cc:232-274, 313-340).
//
// Work-group: four wavefronts in a 2x2 grid over a tile of (64*FM) output channels x
// (64*FN) pixels; each wavefront owns FM x FN MFMA tiles of 32x32.  Both operands reach LDS by
// asynchronous global->LDS copies (nothing passes through registers) into a ring of two or
// three stages of 64 or 128 K-bytes; the copies run ahead of the MFMAs across tile boundaries.
// The 16-byte chunks of a staged row are XOR-swizzled with row bits so that the 128-bit
// fragment reads of a wavefront fall on distinct banks (lds_chunk_offset).
//
// Epilogue: the requantization of quant_math.h per element, codes packed four output
// channels at a time, transposed through the ring slot just consumed into [pixel][oc] rows
// and written as 128-bit stores to the channels-last output; optionally the residual sum of
// the element-wise group behind the convolution (ResidualAdd).  With an int32 output
// (ConvInteger, MatMulInteger) the accumulators are stored directly.
#include <cmath>
#include <type_traits>
#include <vector>

#include "contract.h"
#include "conv_mfma.h"
#include "conv_device.h"

namespace chx {
namespace {

// Packed weights are stored in blocks that one K step of the kernel reads as whole cache
// lines: Wp[oc / 64][k / BK][oc % 64][k % BK] with BK = 64 or 128 K-bytes per step, i.e. the 64
// rows of a block are BK contiguous bytes each and a block is 64 * BK contiguous bytes.
__host__ __device__ __forceinline__ int64_t packed_offset(int oc, int k, int KP, int BK) {
    return ((int64_t)(oc >> 6) * (KP / BK) + k / BK) * (64 * BK) + (oc & 63) * BK + k % BK;
}

// ---------------------------------------------------------------------------------------------
// Weight repacking: w [OC][C][KH][KW] (any strides) -> Wp, K index k = (kh*KW + kw)*C64 + c with
// C64 = C rounded up to 64 (zero filled), and wsum[oc] = sum of the row.  One work-group per
// output channel.  padsum (when not null; at most 32 taps): [16][gridDim.x] sums of the row over the taps of the
// filter's border rows and columns that the class names (ConvMfmaArgs::padsum).
__global__ __launch_bounds__(256) void pack_weights_kernel(
        const char* __restrict__ w, int64_t s_oc, int64_t s_c, int64_t s_kh, int64_t s_kw, int OC, int C, int KH, int KW,
        int C64, int BK, int8_t* __restrict__ wp, int32_t* __restrict__ wsum, int32_t* __restrict__ padsum) {
    const int oc = blockIdx.x;
    const int KP = KH * KW * C64;
    __shared__ int32_t tap_sum[32];
    if (threadIdx.x < 32) tap_sum[threadIdx.x] = 0;
    __syncthreads();
    int32_t local = 0;
    int32_t run = 0, run_pos = 0;  // this thread's sum over its elements of tap run_pos so far
    for (int k = threadIdx.x; k < KP; k += 256) {
        const int c = k % C64;
        const int pos = k / C64;
        int8_t v = 0;
        if (oc < OC && c < C) {
            const int kh = pos / KW, kw = pos % KW;
            v = *reinterpret_cast<const int8_t*>(w + oc * s_oc + c * s_c + kh * s_kh + kw * s_kw);
        }
        wp[packed_offset(oc, k, KP, BK)] = v;
        local += v;
        if (padsum) {
            if (pos != run_pos) {
                if (run != 0) atomicAdd(&tap_sum[run_pos], run);
                run = 0;
                run_pos = pos;
            }
            run += v;
        }
    }
    if (padsum && run != 0) atomicAdd(&tap_sum[run_pos], run);
    __shared__ int32_t red[256];
    red[threadIdx.x] = local;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) wsum[oc] = red[0];
    if (padsum && threadIdx.x < 16) {
        const int cls = threadIdx.x;
        int32_t sum = 0;
        for (int i = 0; i < KH; ++i)
            for (int j = 0; j < KW; ++j) {
                const bool outside = ((cls & 8) && i == 0) || ((cls & 4) && i == KH - 1) || ((cls & 2) && j == 0) || ((cls & 1) && j == KW - 1);
                if (outside) sum += tap_sum[i * KW + j];
            }
        padsum[(int64_t)cls * gridDim.x + oc] = sum;
    }
}

// Few input channels (the 3-channel stem): padding each filter tap to 64 K-bytes would waste
// most of the matrix-core work, so the taps are packed densely instead.  The weights become
// [OCpad][Kd] with k = (kh*KW + kw)*C + c, Kd = KH*KW*C rounded up to 64, and the activations
// are expanded once into an explicit [M][Kd] matrix (im2col) that the MFMA kernel then reads
// as a 1x1 convolution over Kd "channels".  Out-of-image taps hold the zero point, K padding
// holds anything (its weights are zero).
__global__ __launch_bounds__(256) void pack_weights_dense_kernel(
        const char* __restrict__ w, int64_t s_oc, int64_t s_c, int64_t s_kh, int64_t s_kw, int OC, int C, int KH, int KW,
        int Kd, int BK, int8_t* __restrict__ wp, int32_t* __restrict__ wsum) {
    const int oc = blockIdx.x;
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
        wp[packed_offset(oc, k, Kd, BK)] = v;
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

// The same matrix, staged through LDS: a work-group takes kIm2colPx consecutive output pixels of
// one output row, copies the C x KH input row segments they touch into LDS once (coalesced,
// out-of-image bytes replaced by the zero point), and then every lane assembles 16-byte chunks
// of the [M][Kd] rows from LDS bytes; consecutive lanes write consecutive chunks.  A table maps
// k = (kh*KW + kw)*C + c to the LDS offset of the pixel-independent part of the address.
constexpr int kIm2colPx = 64;
constexpr int kIm2colPatchMax = 24 * 1024;  // bytes of LDS for the input patch

__global__ __launch_bounds__(256) void im2col_dense_lds_kernel(Im2colArgs a, int row_len) {
    extern __shared__ __attribute__((aligned(16))) unsigned char im2col_lds[];
    const int K = a.KH * a.KW * a.C;
    uint16_t* tab = reinterpret_cast<uint16_t*>(im2col_lds);  // [Kd]
    unsigned char* patch = im2col_lds + a.Kd * 2;             // [C*KH][row_len]
    const int tid = threadIdx.x;
    const int ow0 = blockIdx.x * kIm2colPx;
    const int oh = blockIdx.y;
    const int n = blockIdx.z;
    for (int k = tid; k < a.Kd; k += 256) {
        int v = 0xffff;
        if (k < K) {
            const int c = k % a.C, pos = k / a.C;
            const int kh = pos / a.KW, kw = pos % a.KW;
            v = (c * a.KH + kh) * row_len + kw;
        }
        tab[k] = (uint16_t)v;
    }
    const int ih0 = oh * a.sh - a.ph, iw0 = ow0 * a.sw - a.pw;
    const char* xn = a.x + (int64_t)n * a.xs[0];
    const int rows = a.C * a.KH;
    for (int idx = tid; idx < rows * row_len; idx += 256) {
        const int rr = idx / row_len, col = idx - rr * row_len;
        const int c = rr / a.KH, kh = rr - c * a.KH;
        const int ih = ih0 + kh, iw = iw0 + col;
        unsigned char v = (unsigned char)a.fill;
        if ((unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W)
            v = *reinterpret_cast<const unsigned char*>(xn + (int64_t)c * a.xs[1] + (int64_t)ih * a.xs[2] + (int64_t)iw * a.xs[3]);
        patch[idx] = v;
    }
    __syncthreads();
    const int chunks = a.Kd / 16;
    const int npx = min(kIm2colPx, a.OW - ow0);
    const int64_t m0 = ((int64_t)n * a.OH + oh) * a.OW + ow0;
    const uint32_t fill = (uint32_t)a.fill & 0xffu;
    for (int q = tid; q < npx * chunks; q += 256) {
        const int p = q / chunks, ch = q - p * chunks;
        const unsigned char* src = patch + p * a.sw;
        const v4i t0 = *reinterpret_cast<const v4i*>(tab + ch * 16);
        const v4i t1 = *reinterpret_cast<const v4i*>(tab + ch * 16 + 8);
        uint32_t out[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            uint32_t word = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int k = d * 4 + e;  // two 16-bit offsets per dword of the table
                const uint32_t pair = (uint32_t)(k < 8 ? t0[k >> 1] : t1[(k - 8) >> 1]);
                const uint32_t off = (k & 1) ? pair >> 16 : pair & 0xffffu;
                const uint32_t v = off == 0xffffu ? fill : (uint32_t)src[off];
                word |= v << (8 * e);
            }
            out[d] = word;
        }
        const v4i o = {(int)out[0], (int)out[1], (int)out[2], (int)out[3]};
        *reinterpret_cast<v4i*>(a.col + (m0 + p) * a.Kd + ch * 16) = o;
    }
}

}  // namespace

int pack_weights(
        const chx_hip_tensor& w, int C64, int BK, int OCpad, int8_t* wp, int32_t* wsum, int32_t* padsum, hipStream_t s) {
    pack_weights_kernel<<<OCpad, 256, 0, s>>>(
            static_cast<const char*>(w.data), w.strides[0], w.strides[1], w.strides[2], w.strides[3], (int)w.shape[0],
            (int)w.shape[1], (int)w.shape[2], (int)w.shape[3], C64, BK, wp, wsum, padsum);
    return launch_check("pack_weights_kernel");
}

int pack_weights_dense(const chx_hip_tensor& w, int Kd, int BK, int OCpad, int8_t* wp, int32_t* wsum, hipStream_t s) {
    pack_weights_dense_kernel<<<OCpad, 256, 0, s>>>(
            static_cast<const char*>(w.data), w.strides[0], w.strides[1], w.strides[2], w.strides[3], (int)w.shape[0],
            (int)w.shape[1], (int)w.shape[2], (int)w.shape[3], Kd, BK, wp, wsum);
    return launch_check("pack_weights_dense_kernel");
}

int launch_im2col_dense(const Im2colArgs& a, hipStream_t s) {
    const int64_t total = a.M * (a.Kd / 16);
    if (total == 0) return CHX_HIP_OK;
    // LDS-staged variant when the input patch of a pixel group fits (the offsets are 16-bit)
    const int row_len = (kIm2colPx - 1) * a.sw + a.KW;
    const int64_t patch = (int64_t)a.C * a.KH * row_len;
    const int64_t N = a.M / ((int64_t)a.OH * a.OW);
    if (patch <= kIm2colPatchMax && patch < 0xffff && a.OH <= 65535 && N <= 65535) {
        const dim3 grid((unsigned)((a.OW + kIm2colPx - 1) / kIm2colPx), (unsigned)a.OH, (unsigned)N);
        im2col_dense_lds_kernel<<<grid, 256, (size_t)(a.Kd * 2 + patch), s>>>(a, row_len);
        return launch_check("im2col_dense_lds_kernel");
    }
    im2col_dense_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(a);
    return launch_check("im2col_dense_kernel");
}

namespace {

// One work-group per candidate, one thread per residual code r, all 256 convolution codes c in turn (sixteen at a
// time, as the epilogue processes them): counts the pairs on which the two forms differ.
__global__ __launch_bounds__(256) void affine_residual_search_kernel(ResidualAdd exact, const float* __restrict__ cand, int32_t* __restrict__ mismatches) {
    ResidualAdd p = exact;
    p.kc = cand[blockIdx.x * 3 + 0];
    p.kr = cand[blockIdx.x * 3 + 1];
    p.k0 = cand[blockIdx.x * 3 + 2];
    const uint32_t r = threadIdx.x;
    const v4i rw = {(int)(r * 0x01010101u), (int)(r * 0x01010101u), (int)(r * 0x01010101u), (int)(r * 0x01010101u)};
    int bad = 0;
    for (uint32_t c0 = 0; c0 < 256; c0 += 16) {
        v4i cw;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const uint32_t b = c0 + 4 * w;
            cw[w] = (int)(b | ((b + 1) << 8) | ((b + 2) << 16) | ((b + 3) << 24));
        }
        const v4i want = add_residual16_any(cw, rw, exact);
        const v4i got = exact.affine == 2 ? affine_residual16<true>(cw, rw, p) : affine_residual16<false>(cw, rw, p);
#pragma unroll
        for (int w = 0; w < 4; ++w) bad |= want[w] != got[w] ? 1 : 0;
    }
    const int total = __syncthreads_count(bad);  // threads (residual codes) with a difference anywhere
    if (threadIdx.x == 0) mismatches[blockIdx.x] = total;
}

}  // namespace

int find_affine_residual(ResidualAdd* p, int32_t* scratch, hipStream_t s) {
    p->affine = 0;
    // uint8 sums only (the floor-mode conversion saturates to [0, 255]); with the range guard active the scales are
    // extreme and the sum stays with the guarded arithmetic
    if (p->out.lo != 0.f || p->guard) return CHX_HIP_OK;
    const double so = (double)p->out.scale;
    const double kc = (double)p->c_scale / so, kr = (double)p->r_scale / so;
    const double k0 = -(double)p->c_zpf * kc - (double)p->r_zpf * kr + (double)p->out.zpf + 0.5;
    if (!(fabs(kc) < 1e6 && fabs(kr) < 1e6 && fabs(k0) < 1e6)) return CHX_HIP_OK;
    const int mode = (p->relu && p->out.zpf != 0.f) ? 2 : 1;
    std::vector<float> cand((size_t)kAffineCandidates * 3);
    auto step = [](float x, int n) {
        for (int i = 0; i < (n < 0 ? -n : n); ++i) x = nextafterf(x, n > 0 ? INFINITY : -INFINITY);
        return x;
    };
    int idx = 0;
    // nearest neighbours first: the order of preference
    static const int order5[5] = {0, -1, 1, -2, 2};
    static const int order13[13] = {0, -1, 1, -2, 2, -3, 3, -4, 4, -5, 5, -6, 6};
    for (int a = 0; a < 5; ++a)
        for (int b = 0; b < 5; ++b)
            for (int c = 0; c < 13; ++c) {
                cand[idx * 3 + 0] = step((float)kc, order5[a]);
                cand[idx * 3 + 1] = step((float)kr, order5[b]);
                cand[idx * 3 + 2] = step((float)k0, order13[c]);
                ++idx;
            }
    float* dcand = nullptr;
    CHX_HIP_CALL(hipMalloc(reinterpret_cast<void**>(&dcand), cand.size() * sizeof(float)));
    ResidualAdd probe = *p;
    probe.affine = mode;
    probe.floor_pre = p->out.zpf + 0.5f;
    int rc = CHX_HIP_OK;
    std::vector<int32_t> bad((size_t)kAffineCandidates, 1);
    if (hipMemcpyAsync(dcand, cand.data(), cand.size() * sizeof(float), hipMemcpyHostToDevice, s) != hipSuccess) rc = CHX_HIP_ERUNTIME;
    if (rc == CHX_HIP_OK) {
        affine_residual_search_kernel<<<kAffineCandidates, 256, 0, s>>>(probe, dcand, scratch);
        rc = launch_check("affine_residual_search_kernel");
    }
    if (rc == CHX_HIP_OK && (hipMemcpyAsync(bad.data(), scratch, bad.size() * sizeof(int32_t), hipMemcpyDeviceToHost, s) != hipSuccess ||
                             hipStreamSynchronize(s) != hipSuccess))
        rc = CHX_HIP_ERUNTIME;
    (void)hipFree(dcand);
    if (rc != CHX_HIP_OK) {
        (void)hipGetLastError();
        CHX_FAIL(rc, "checking the two-multiply-add form of a residual sum failed");
    }
    for (int i = 0; i < kAffineCandidates; ++i)
        if (bad[i] == 0) {
            p->affine = mode;
            p->kc = cand[i * 3 + 0];
            p->kr = cand[i * 3 + 1];
            p->k0 = cand[i * 3 + 2];
            p->floor_pre = probe.floor_pre;
            break;
        }
    return CHX_HIP_OK;
}

int launch_conv_mfma(ConvMfmaArgs a, int tile_oc, int tile_px, int max_wgs_per_cu, int waves, bool x_unsigned, bool out_int32, bool rne,
                     hipStream_t s) {
    a.tiles_oc = (a.OC + tile_oc - 1) / tile_oc;
    a.tiles_px = (int)((a.M + tile_px - 1) / tile_px);
    if (a.M == 0 || a.OC == 0) return CHX_HIP_OK;
    if (a.oc_split != 0 && (a.oc_split < 0 || a.oc_split >= a.OC || a.oc_split % tile_oc != 0 || out_int32 || a.res.r))
        CHX_FAIL(CHX_HIP_EINVAL, "conv_mfma: two outputs split at channel %d do not fit tiles of %d output channels", a.oc_split, tile_oc);
    // 32-bit offsets into x: the bias keeps the offset of a tap in the padding of the first image non-negative
    // (and leaves room for the immediates the copies subtract); a tap that is fetched lies inside x
    const int64_t bias = 4096 + (int64_t)a.ph * a.x_h_stride + (int64_t)a.pw * a.x_w_stride;
    if (a.x_h_stride < 0 || a.x_w_stride < 0 || a.x_n_stride < 0 || bias < 0 || (int64_t)a.x_bytes + bias >= (int64_t(1) << 31) ||
        a.x_n_stride >= (int64_t(1) << 31) || a.x_h_stride >= (int64_t(1) << 31) || a.x_w_stride >= (int64_t(1) << 31))
        CHX_FAIL(CHX_HIP_EUNSUPPORTED, "conv_mfma: the activations span 2 GB or more");
    a.x_bias = (uint32_t)bias;
    // the scalar offset has advanced by C64 - bk inside the tap when it moves on
    a.tap_step_col = (uint32_t)(a.x_w_stride - (a.C64 - a.bk));
    a.tap_step_row = (uint32_t)(a.x_h_stride - (int64_t)(a.KW - 1) * a.x_w_stride - (a.C64 - a.bk));
    magic_divisor((uint32_t)a.OW, &a.ow_mul, &a.ow_shift);
    magic_divisor((uint32_t)a.OH, &a.oh_mul, &a.oh_shift);
    a.px_linear = a.KH == 1 && a.KW == 1 && a.sh == 1 && a.sw == 1 && a.ph == 0 && a.pw == 0 && a.OH == a.H && a.OW == a.W &&
                  a.x_h_stride == (int64_t)a.W * a.x_w_stride && a.x_n_stride == (int64_t)a.H * a.x_h_stride;
    a.row_unit = 0;
    if (a.KH * a.KW <= 32)
        for (int i = 0; i < a.KH; ++i) a.row_unit |= 1u << (i * a.KW);
    if (waves == 8) {
        // eight wavefronts: the pixels of the tile are split four ways
        if (tile_oc == 128 && tile_px == 128) return a.bk == 128 ? launch_conv_mfma_2_1_128_4(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s)
                               : launch_conv_mfma_2_1_64_4(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s);
        if (tile_oc == 128 && tile_px == 256 && a.bk == 128) return launch_conv_mfma_2_2_128_4(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s);
        if (tile_oc == 64 && tile_px == 128 && a.bk == 128) return launch_conv_mfma_1_1_128_4(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s);
        CHX_FAIL(CHX_HIP_EINVAL, "conv_mfma: no eight-wavefront kernel for a %dx%d tile with %d K bytes per step", tile_oc, tile_px, a.bk);
    }
    if (waves != 4) CHX_FAIL(CHX_HIP_EINVAL, "conv_mfma: work-groups have 4 or 8 wavefronts, not %d", waves);
    if (tile_oc == 128 && tile_px == 128) return a.bk == 128 ? launch_conv_mfma_2_2_128_2(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s)
                           : launch_conv_mfma_2_2_64_2(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s);
    if (tile_oc == 64 && tile_px == 128) return a.bk == 128 ? launch_conv_mfma_1_2_128_2(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s)
                           : launch_conv_mfma_1_2_64_2(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s);
    if (tile_oc == 128 && tile_px == 64) return a.bk == 128 ? launch_conv_mfma_2_1_128_2(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s)
                           : launch_conv_mfma_2_1_64_2(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s);
    if (tile_oc == 64 && tile_px == 64) return a.bk == 128 ? launch_conv_mfma_1_1_128_2(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s)
                           : launch_conv_mfma_1_1_64_2(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s);
    CHX_FAIL(CHX_HIP_EINVAL, "conv_mfma: no kernel for a %dx%d tile", tile_oc, tile_px);
}

}  // namespace chx
