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
// output channel.
__global__ __launch_bounds__(256) void pack_weights_kernel(
        const char* __restrict__ w, int64_t s_oc, int64_t s_c, int64_t s_kh, int64_t s_kw, int OC, int C, int KH, int KW,
        int C64, int BK, int8_t* __restrict__ wp, int32_t* __restrict__ wsum) {
    const int oc = blockIdx.x;
    const int KP = KH * KW * C64;
    int32_t local = 0;
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

// ---------------------------------------------------------------------------------------------
// Byte offset of K chunk kc (16 bytes) of a staged row.  The chunks of a row are XOR-swizzled
// with row bits so that 128-bit fragment reads of consecutive rows fall on distinct banks:
// rows of 64 bytes (4 chunks) with bits 2..3, rows of 128 bytes (8 chunks) with bits 1..3.
template <int BK>
__device__ __forceinline__ int lds_chunk_offset(int row, int kc) {
    return BK == 64 ? row * 64 + ((kc ^ ((row >> 2) & 3)) << 4) : row * 128 + ((kc ^ ((row >> 1) & 7)) << 4);
}

// 128-bit LDS read whose completion the caller waits for itself (wait_fragments): the compiler
// would otherwise wait for every outstanding LDS operation at the first use, because it cannot
// see through the inline assembly of the copies issued in between.
__device__ __forceinline__ v4i lds_read16_nowait(uint32_t lds_addr) {
    v4i v;
    asm volatile("ds_read_b128 %0, %1" : "=&v"(v) : "v"(lds_addr) : "memory");
    return v;
}

// Wait until at most N LDS/scalar-memory operations of this wave are outstanding; the fragment
// registers pass through so that their uses are ordered after the wait.
template <int N, int FM, int FN>
__device__ __forceinline__ void wait_fragments(v4i (&fa)[FM], v4i (&fb)[FN]) {
    if constexpr (FM == 2 && FN == 2)
        asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fb[0]), "+v"(fb[1]) : "n"(N) : "memory");
    else if constexpr (FM == 2 && FN == 1)
        asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fb[0]) : "n"(N) : "memory");
    else if constexpr (FM == 1 && FN == 2)
        asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(fa[0]), "+v"(fb[0]), "+v"(fb[1]) : "n"(N) : "memory");
    else
        asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(fa[0]), "+v"(fb[0]) : "n"(N) : "memory");
}

// Touch every 64-byte line of the kernel arguments at once.  The argument block of a fresh launch
// is not in any cache, and the compiler fetches the fields in several dependent batches that
// each touch new lines: one round trip to memory per batch.  After this, one round trip.
template <int BYTES>
__device__ __forceinline__ void warm_kernel_arguments() {
    const uint64_t ka = (uint64_t)__builtin_amdgcn_kernarg_segment_ptr();
    constexpr int LINES = (BYTES + 63) / 64;
    static_assert(LINES >= 4 && LINES <= 6, "between four and six lines are touched");
    // offsets of the last lines, clamped into the block so that nothing outside it is read
    constexpr int L4 = LINES > 4 ? 0x100 : 0xc0, L5 = LINES > 5 ? 0x140 : L4;
    int t0, t1, t2, t3, t4, t5;
    asm volatile(
            "s_load_dword %0, %6, 0x0\n\t"
            "s_load_dword %1, %6, 0x40\n\t"
            "s_load_dword %2, %6, 0x80\n\t"
            "s_load_dword %3, %6, 0xc0\n\t"
            "s_load_dword %4, %6, %7\n\t"
            "s_load_dword %5, %6, %8\n\t"
            "s_waitcnt lgkmcnt(0)"
            : "=&s"(t0), "=&s"(t1), "=&s"(t2), "=&s"(t3), "=&s"(t4), "=&s"(t5)
            : "s"(ka), "n"(L4), "n"(L5)
            : "memory");
}

// LDS ring stages of a work-group: what fits the budget, between 2 and the cap.  The bytes in
// flight towards a compute unit, (stages - 1) * stage bytes * resident work-groups, set the copy
// rate that the memory latency allows.
#ifndef CHX_CONV_LDS_BUDGET
#define CHX_CONV_LDS_BUDGET (80 * 1024)
#endif
#ifndef CHX_CONV_NS_MAX
#define CHX_CONV_NS_MAX 3
#endif
constexpr int ring_stages(int stage_bytes, int lds_budget) {
    const int fit = lds_budget / stage_bytes;
    return fit < 2 ? 2 : fit > CHX_CONV_NS_MAX ? CHX_CONV_NS_MAX : fit;
}

// FM x FN MFMA tiles (32x32) per wavefront; four wavefronts in a 2x2 grid per work-group.
// Tile = (64*FM) output channels x (64*FN) pixels.
//
// Work-groups are persistent: each owns one output-channel tile and walks over pixel tiles
// px_first, px_first + px_step, ...  The sequence of (pixel tile, K step) pairs is one flat
// pipeline over a ring of NS LDS stages: the asynchronous copies run NS-1 steps ahead of the
// MFMAs and cross tile boundaries, so the operands of the next tile are in flight while the
// current tile is requantized and written out.  Per K step (BK = 64 or 128 K-bytes) a wave
// issues (FM + FN) * BK/64 copy instructions, reads its fragments back with 128-bit LDS loads,
// flips the sign bits of uint8 activations on the fragments, and feeds FM*FN*BK/32 MFMAs; one
// barrier per step.
//
// LDS stage: rows of BK K-bytes, weight rows first, then pixel rows.  A copy instruction fills
// 1 KB = 1024/BK consecutive rows; a lane lands in a fixed (row, slot) and fetches the K chunk
// that the XOR swizzle of lds_chunk_offset() places there, so the 128-bit fragment reads are
// free of bank conflicts.  BK = 128 is used when the channel count is a multiple of 128: then a
// pixel's 128 K-bytes of one filter tap are one whole cache line, where two 64-byte steps
// would each fetch the line and use half of it (the weight blocks are contiguous either way).
//
// kPad: some filter tap can fall outside the image, or the channel count is not a multiple
// of 64.  Then each staged row carries a bit mask of its valid taps (computed once per pixel
// tile) and an invalid chunk is fetched from a 64-byte row holding the zero point instead
// (g_fill_rows), which makes it contribute (zp - zp) * w = 0.  Without kPad (1x1 and other
// unpadded convolutions on 64-multiple channels, matrix products) every chunk is valid.
//
// NWN: wavefronts along the pixel axis (two along the output channels).  2: four wavefronts, two
// work-groups per compute unit as a rule.  4: eight wavefronts on the same tile, each with half the
// pixels; a work-group then has the compute unit to itself (and the whole LDS for a deeper ring).  The
// K loop of a wavefront is bound by the instructions it has to issue (fragment reads, sign flips,
// copy addresses: about 200 for 16 MFMAs with four wavefronts on a 128x128 tile), so when a layer has
// no second work-group to put on the compute unit, twice the wavefronts on the same tile halve what
// each has to issue and the two of a SIMD fill each other's gaps.
template <int FM, int FN, int BK, bool kXUnsigned, bool kOutInt32, bool kRne, bool kPad, bool kRes, int NWN = 2>
__global__ __launch_bounds__(128 * NWN) __attribute__((amdgpu_waves_per_eu(2))) void conv_mfma_kernel(ConvMfmaArgs a) {
    constexpr int NW = 2 * NWN;  // wavefronts
    constexpr int T = 64 * NW;
    constexpr int TM = 64 * FM;        // output channels per tile
    constexpr int TN = 32 * NWN * FN;  // pixels per tile
    constexpr int STAGE_BYTES = (TM + TN) * BK;
    constexpr int NS = ring_stages(STAGE_BYTES, NWN == 2 ? CHX_CONV_LDS_BUDGET : 2 * CHX_CONV_LDS_BUDGET - 8 * 1024);
    constexpr int CH = BK / 16;          // 16-byte chunks per staged row
    constexpr int RPI = 64 / CH;         // rows one copy instruction fills
    constexpr int CA = TM / RPI / NW;    // copy instructions per wave and stage, weight rows
    constexpr int CB = TN / RPI / NW;    //   ... pixel rows
    static_assert(CA >= 1 && CB >= 1 && CA * RPI * NW == TM && CB * RPI * NW == TN, "every wavefront copies whole instructions of both operands");
    constexpr int COPIES = CA + CB;
    constexpr int OUT_CHUNKS = TM / 16;  // 16-byte chunks per staged output row
    static_assert(TN * TM <= STAGE_BYTES, "the output tile is staged in one ring slot");
    __shared__ __attribute__((aligned(16))) char ring[NS * STAGE_BYTES];
    __shared__ __attribute__((aligned(16))) float s_scale[TM];
    __shared__ __attribute__((aligned(16))) int32_t s_add[TM];
    __shared__ __attribute__((aligned(16))) float s_fbias[TM];

    warm_kernel_arguments<sizeof(ConvMfmaArgs)>();
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / NWN, wn = wave % NWN;

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
    if (total_stages == 0) return;

    // rows this thread copies per stage: row0 + 4*RPI*j of the weight tile and of the pixel tile,
    // K chunk kc of each (the chunk whose swizzled slot is lane % CH; it is the same for all j)
    const int row0 = wave * RPI + lane / CH;
    const int kc = BK == 64 ? (lane & 3) ^ ((lane >> 4) & 3) : (lane & 7) ^ ((((wave & 1) << 2) + (lane >> 4)) & 7);
    const int8_t* wp_row[CA];
#pragma unroll
    for (int j = 0; j < CA; ++j) wp_row[j] = a.wp + packed_offset(oc0 + row0 + NW * RPI * j, kc * 16, a.KP, BK);
    const char* fill_src = reinterpret_cast<const char*>(g_fill_rows) + (a.x_zp & 0xff) * 64 + (kc & 3) * 16;
    const uint32_t ring_base = (uint32_t)(uintptr_t)ring;             // LDS byte address
    const uint32_t ring_addr = ring_base + (uint32_t)wave * 1024u;

    // ---- copy side state: which (pixel tile, K step) the next stage fetches ----
    const char* xb[CB];
    int ld_tile = px_first;
    int ld_k = 0, kh = 0, kw = 0, c0 = 0, kofs = 0;
    int64_t tap_off = 0;  // kh * x_h_stride + kw * x_w_stride

    uint64_t tapmask[CB];  // kPad: bit (kh*KW + kw) set when that tap of the row's pixel is inside the image
    int tap = 0;

    auto set_load_tile = [&]() {
        const int64_t mbase = (int64_t)ld_tile * TN + row0;
#pragma unroll
        for (int j = 0; j < CB; ++j) {
            const int64_t m = mbase + NW * RPI * j;
            const bool row_ok = m < a.M && ld_tile < px_hi;
            // rows past the end re-read the last pixel; they are never written back
            const uint32_t mm = m < a.M ? (uint32_t)m : (uint32_t)(a.M - 1);  // M fits 31 bits (checked on the host)
            if (a.px_linear) {
                // output pixel m reads input pixel m: no decomposition into (n, oh, ow), one multiplication
                xb[j] = a.x + (int64_t)mm * a.x_w_stride + kc * 16;
                if (kPad) tapmask[j] = row_ok ? 1u : 0u;  // the one tap is inside the image
                continue;
            }
            const uint32_t r = fast_div(mm, a.ow_mul, a.ow_shift);
            const uint32_t ow = mm - r * (uint32_t)a.OW;
            const uint32_t n = fast_div(r, a.oh_mul, a.oh_shift);
            const uint32_t oh = r - n * (uint32_t)a.OH;
            const int ih0 = (int)oh * a.sh - a.ph;
            const int iw0 = (int)ow * a.sw - a.pw;
            xb[j] = a.x + (int64_t)n * a.x_n_stride + (int64_t)ih0 * a.x_h_stride + (int64_t)iw0 * a.x_w_stride + kc * 16;
            if (kPad) {
                // taps (i, jj) inside the image: i in [r_lo, r_hi), jj in [c_lo, c_hi)
                const int c_lo = min(max(-iw0, 0), a.KW), c_hi = min(max(a.W - iw0, 0), a.KW);
                const int r_lo = min(max(-ih0, 0), a.KH), r_hi = min(max(a.H - ih0, 0), a.KH);
                uint64_t mask = 0;
                if (a.KH * a.KW <= 32) {
                    // up to 32 taps (3x3, 5x5): the column bits repeated in every filter row by one
                    // multiplication with the bits KW apart, then the rows outside the image cut off
                    const uint32_t cols = c_hi > c_lo ? ((1u << c_hi) - 1u) & ~((1u << c_lo) - 1u) : 0u;
                    const uint32_t lo_bit = (uint32_t)(r_lo * a.KW), hi_bit = (uint32_t)(r_hi * a.KW);
                    const uint32_t below_hi = hi_bit >= 32 ? ~0u : (1u << hi_bit) - 1u;
                    const uint32_t rows = r_hi > r_lo ? below_hi & ~((1u << lo_bit) - 1u) : 0u;
                    mask = (cols * a.row_unit) & rows;
                } else {
                    const uint64_t below_hi = c_hi >= 64 ? ~(uint64_t)0 : ((uint64_t)1 << c_hi) - 1;  // a 1x64 filter fills the mask
                    const uint64_t cols = c_hi > c_lo ? below_hi & ~(((uint64_t)1 << c_lo) - 1) : 0;
                    for (int i = 0; i < a.KH; ++i)
                        if (i >= r_lo && i < r_hi) mask |= cols << (i * a.KW);
                }
                tapmask[j] = row_ok ? mask : 0;
            }
        }
    };
    set_load_tile();

    // Every stage issues the same number of copies and none is conditional, so a fixed
    // vector-memory count identifies the stage about to be consumed.  Stages past the end of
    // this work-group's list re-read the last K step into a ring slot nobody reads again.
    // copy number q of the stage being fetched: the weight rows come first, then the pixel rows
    auto issue_copy = [&](int buf, int q) {
        const uint32_t dst = ring_addr + (uint32_t)buf * STAGE_BYTES;
        if (q < CA) {
            async_copy16(wp_row[q] + kofs, dst + q * (NW * 1024));
        } else {
            const int j = q - CA;
            bool ok = true;
            if (kPad) ok = c0 + kc * 16 < a.C16 && ((tapmask[j] >> tap) & 1u);
            async_copy16(ok ? xb[j] + tap_off + c0 : fill_src, dst + TM * BK + j * (NW * 1024));
        }
    };
    // advance to the next K step, or to the first K step of this work-group's next pixel tile
    auto advance_stage = [&]() {
        if (++ld_k == nk) {
            if (ld_tile + px_step < px_hi) {
                ld_k = 0; kh = 0; kw = 0; c0 = 0; kofs = 0; tap_off = 0; tap = 0;
                ld_tile += px_step;
                set_load_tile();
            } else {
                --ld_k;  // nothing follows: keep fetching the last step
            }
        } else {
            kofs += 64 * BK;  // next block of the packed weights
            c0 += BK;
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

    // the first NS-1 stages go out before anything else touches memory
#pragma unroll
    for (int d = 0; d < NS - 1; ++d) {
#pragma unroll
        for (int q = 0; q < COPIES; ++q) issue_copy(d, q);
        advance_stage();
    }

    // per-channel epilogue constants; s_add seeds the accumulators
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
    __syncthreads();

    // lane holds, per 32x32 MFMA tile: pixel column (lane & 31), output-channel rows
    // (v / 4) * 8 + (lane >> 5) * 4 + (v % 4)
    v16i acc[FM][FN];
    auto seed_acc = [&]() {
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const v4i ad = *reinterpret_cast<const v4i*>(&s_add[wm * 32 * FM + i * 32 + g * 8 + (lane >> 5) * 4]);
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[i][j][g * 4 + e] = ad[e];
            }
    };
    seed_acc();

    // ---- epilogue of one finished pixel tile ----
    // The 8-bit tile is transposed through the ring slot that was just consumed (the copies in
    // flight target the other slots): rows of TM bytes per pixel, the 16-byte chunks of a row
    // XOR-swizzled with bits 1.. of the pixel index so that neither the 4-byte writes of the
    // accumulator layout nor the 16-byte reads of the store loop pile up on a bank.
    auto staged = [&](char* slot, int pxl, int ocl) -> char* {
        return slot + pxl * TM + ((((ocl >> 4) ^ (pxl >> 1)) & (OUT_CHUNKS - 1)) << 4) + (ocl & 15);
    };
    auto epilogue = [&](int px_tile, char* lds_out) {
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
                        for (int e = 0; e < 4; ++e) out[e] = acc[i][j][g * 4 + e];
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
        // requantize: one instance of the element loop per bias mode and per conversion path (the
        // branches are uniform).  kPath 0: any 8-bit type and rounding; 1: uint8 in the reference's
        // rounding through floor_sat_u8x16; 2: the same with a lower bound above 0 (a folded Relu);
        // 3: as 1 with a zero point of 0.
        auto requantize_tile = [&](auto float_bias_tag, auto path_tag) {
            constexpr bool kFloatBias = decltype(float_bias_tag)::value;
            constexpr int kPath = decltype(path_tag)::value;
            // a block of 32 output channels that lies beyond OC altogether (OC = 96 in a 128-wide tile, say) is not
            // requantized: nobody reads its staged bytes (the test is the same for the whole wavefront)
            if constexpr (kPath == 0) {
#pragma unroll
                for (int i = 0; i < FM; ++i) {
                    if (oc0 + wm * 32 * FM + i * 32 >= a.OC) continue;
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int ocl = wm * 32 * FM + i * 32 + g * 8 + (lane >> 5) * 4;
                        const v4f sc = *reinterpret_cast<const v4f*>(&s_scale[ocl]);
                        v4f fb = {0.f, 0.f, 0.f, 0.f};
                        if (kFloatBias) fb = *reinterpret_cast<const v4f*>(&s_fbias[ocl]);
#pragma unroll
                        for (int j = 0; j < FN; ++j) {
                            const int pxl = wn * 32 * FN + j * 32 + (lane & 31);
                            int32_t code[4];
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                float v = (float)acc[i][j][g * 4 + e] * sc[e];
                                if (kFloatBias) v = v + fb[e];  // reference mode: float bias after the scale multiply
                                code[e] = quantize_value_folded<kRne>(v, a.rq.q, a.inv_y_scale, a.lo_folded);
                            }
                            *reinterpret_cast<uint32_t*>(staged(lds_out, pxl, ocl)) = pack4(code[0], code[1], code[2], code[3]);
                        }
                    }
                }
            } else {
                // sixteen values (4 / FN row groups of the accumulator) per switch of the rounding mode
                constexpr int G = 4 / FN;
#pragma unroll
                for (int i = 0; i < FM; ++i) {
                    if (oc0 + wm * 32 * FM + i * 32 >= a.OC) continue;
#pragma unroll
                    for (int gb = 0; gb < 4; gb += G) {
                        float pre[16];
#pragma unroll
                        for (int gl = 0; gl < G; ++gl) {
                            const int g = gb + gl;
                            const int ocl = wm * 32 * FM + i * 32 + g * 8 + (lane >> 5) * 4;
                            const v4f sc = *reinterpret_cast<const v4f*>(&s_scale[ocl]);
                            v4f fb = {0.f, 0.f, 0.f, 0.f};
                            if (kFloatBias) fb = *reinterpret_cast<const v4f*>(&s_fbias[ocl]);
#pragma unroll
                            for (int j = 0; j < FN; ++j)
#pragma unroll
                                for (int e = 0; e < 4; ++e) {
                                    float v = (float)acc[i][j][g * 4 + e] * sc[e];
                                    if (kFloatBias) v = v + fb[e];
                                    pre[(gl * FN + j) * 4 + e] =
                                            quantize_prefloor_u8<kPath == 2, kPath != 3>(v, a.rq.q, a.inv_y_scale, a.lo_folded);
                                }
                        }
                        uint32_t word[4];
                        floor_sat_u8x16(pre, word);
#pragma unroll
                        for (int gl = 0; gl < G; ++gl) {
                            const int ocl = wm * 32 * FM + i * 32 + (gb + gl) * 8 + (lane >> 5) * 4;
#pragma unroll
                            for (int j = 0; j < FN; ++j)
                                *reinterpret_cast<uint32_t*>(staged(lds_out, wn * 32 * FN + j * 32 + (lane & 31), ocl)) = word[gl * FN + j];
                        }
                    }
                }
            }
        };
        // The residual chunks this thread will add are requested now: their latency runs under the
        // requantization instead of in front of every store.
        constexpr int ITER = TN * OUT_CHUNKS / T;
        v4i rres[ITER];
        // A tile that lies inside the output altogether, with 16-byte accesses allowed, needs no test per lane
        // (the operands of this test are the same for the whole work-group); per-lane branches in the loops
        // below cost far more than the instructions they skip.
        // (in 32-bit scalar terms: every pixel tile but the last is full, and the last one is when TN divides M)
        const bool tile_inside = (px_tile + 1 < a.tiles_px || a.M % TN == 0) && oc0 + TM <= a.OC && a.y_vec_ok && (!kRes || a.res.r_vec_ok);
        if (kRes && tile_inside) {
#pragma unroll
            for (int it = 0; it < ITER; ++it) {
                const int q = tid + it * T;
                rres[it] = *reinterpret_cast<const v4i*>(a.res.r + (m0 + q / OUT_CHUNKS) * a.res.r_px_stride + oc0 + (q % OUT_CHUNKS) * 16);
            }
        } else if (kRes) {
#pragma unroll
            for (int it = 0; it < ITER; ++it) {
                const int q = tid + it * T;
                const int64_t m = m0 + q / OUT_CHUNKS;
                const int oc = oc0 + (q % OUT_CHUNKS) * 16;
                rres[it] = v4i{0, 0, 0, 0};
                if (m < a.M && oc + 16 <= a.OC && a.res.r_vec_ok)
                    rres[it] = *reinterpret_cast<const v4i*>(a.res.r + m * a.res.r_px_stride + oc);
            }
        }
        __syncthreads();  // every wave is done reading the slot's operands
        {
            using P0 = std::integral_constant<int, 0>;
            using P1 = std::integral_constant<int, 1>;
            using P2 = std::integral_constant<int, 2>;
            using P3 = std::integral_constant<int, 3>;
            const bool u8_reference = !kRne && a.rq.q.lo == 0.f && a.rq.q.hi == 255.f;
            const bool float_bias = a.rq.bias_mode == kBiasReferenceFloat;
            if (!u8_reference) {
                if (float_bias) requantize_tile(std::true_type(), P0());
                else requantize_tile(std::false_type(), P0());
            } else if (a.lo_folded > 0.f) {
                if (float_bias) requantize_tile(std::true_type(), P2());
                else requantize_tile(std::false_type(), P2());
            } else if (a.rq.q.zpf == 0.f) {
                if (float_bias) requantize_tile(std::true_type(), P3());
                else requantize_tile(std::false_type(), P3());
            } else {
                if (float_bias) requantize_tile(std::true_type(), P1());
                else requantize_tile(std::false_type(), P1());
            }
        }
        __syncthreads();
        if (tile_inside) {
            auto store_all = [&](auto mode_tag) {
                constexpr int kMode = decltype(mode_tag)::value;  // 0: no residual, 1 / 2: the two-multiply-add forms, 3: the exact chain
#pragma unroll
                for (int it = 0; it < ITER; ++it) {
                    const int q = tid + it * T;
                    const int pxl = q / OUT_CHUNKS;
                    const int ch = q % OUT_CHUNKS;
                    v4i val = *reinterpret_cast<const v4i*>(staged(lds_out, pxl, ch * 16));
                    if constexpr (kMode == 1) val = affine_residual16<false>(val, rres[it], a.res);
                    if constexpr (kMode == 2) val = affine_residual16<true>(val, rres[it], a.res);
                    if constexpr (kMode == 3) val = add_residual16_any(val, rres[it], a.res);
                    *reinterpret_cast<v4i*>(a.y + (m0 + pxl) * a.y_px_stride + oc0 + ch * 16) = val;
                }
            };
            if (!kRes) store_all(std::integral_constant<int, 0>());
            else if (a.res.affine == 1) store_all(std::integral_constant<int, 1>());
            else if (a.res.affine == 2) store_all(std::integral_constant<int, 2>());
            else store_all(std::integral_constant<int, 3>());
            return;
        }
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
            const int q = tid + it * T;
            const int pxl = q / OUT_CHUNKS;
            const int ch = q % OUT_CHUNKS;
            const int64_t m = m0 + pxl;
            const int oc = oc0 + ch * 16;
            if (m >= a.M || oc >= a.OC) continue;
            char* src = staged(lds_out, pxl, ch * 16);
            v4i val = *reinterpret_cast<const v4i*>(src);
            const bool whole = oc + 16 <= a.OC;
            if (kRes) {
                v4i rv = rres[it];
                if (!(a.res.r_vec_ok && whole)) {
                    const char* rsrc = a.res.r + m * a.res.r_px_stride + oc;
#pragma nounroll
                    for (int w = 0; w < 4; ++w) {
                        uint32_t word = 0;
                        for (int e = 0; e < 4; ++e)
                            if (oc + w * 4 + e < a.OC) word |= (uint32_t)(uint8_t)rsrc[w * 4 + e] << (8 * e);
                        rv[w] = (int)word;
                    }
                }
                if (a.res.affine == 1) val = affine_residual16<false>(val, rv, a.res);
                else if (a.res.affine == 2) val = affine_residual16<true>(val, rv, a.res);
                else val = add_residual16_any(val, rv, a.res);
                if (!(a.y_vec_ok && whole)) *reinterpret_cast<v4i*>(src) = val;  // the byte loop below reads LDS
            }
            char* dst = a.y + m * a.y_px_stride + oc;
            if (a.y_vec_ok && whole) {
                *reinterpret_cast<v4i*>(dst) = val;
            } else {
#pragma nounroll
                for (int e = 0; e < 16 && oc + e < a.OC; ++e) dst[e] = src[e];
            }
        }
    };

    const int frag_row = lane & 31;
    const int frag_kc = lane >> 5;
    int ck = 0;             // K step within the tile being computed
    int c_tile = px_first;  // pixel tile being computed
    int cbuf = 0;           // ring slot being computed
    int lbuf = NS - 1;      // ring slot the next copy fills
    for (int s = 0; s < total_stages; ++s) {
        // this wave's copies of stage s have landed when at most the NS-2 younger stages are
        // outstanding; the barrier extends that to every wave's copies, and also says that
        // everybody is done reading the slot the next copies overwrite
        wait_vmcnt<(NS - 2) * COPIES>();
        __syncthreads();

        char* slot = ring + cbuf * STAGE_BYTES;
        cbuf = cbuf + 1 == NS ? 0 : cbuf + 1;
        // The copies of the stage NS-1 steps ahead are issued between the MFMA groups rather than
        // in one burst: the copy unit takes a 1 KB instruction every 16 cycles or so, and a wave
        // that issues them back to back sits in the queue instead of feeding the matrix cores.
        constexpr int SUBS = BK / 32;  // MFMA K extents per stage
        constexpr int PER_SUB = (COPIES + SUBS - 1) / SUBS;
        v4i fa[SUBS][FM], fb[SUBS][FN];
        const uint32_t sa_addr = ring_base + (uint32_t)(slot - ring);
        auto read_fragments = [&](int sub) {
#pragma unroll
            for (int i = 0; i < FM; ++i)
                fa[sub][i] = lds_read16_nowait(sa_addr + lds_chunk_offset<BK>(wm * 32 * FM + i * 32 + frag_row, sub * 2 + frag_kc));
#pragma unroll
            for (int j = 0; j < FN; ++j)
                fb[sub][j] = lds_read16_nowait(sa_addr + TM * BK +
                                               lds_chunk_offset<BK>(wn * 32 * FN + j * 32 + frag_row, sub * 2 + frag_kc));
        };
        // all reads of the stage go out at once; LDS reads complete in order, so extent sub is
        // there when at most the reads of the later extents are outstanding
#pragma unroll
        for (int sub = 0; sub < SUBS; ++sub) read_fragments(sub);
#pragma unroll
        for (int sub = 0; sub < SUBS; ++sub) {
            if (sub == 0) wait_fragments<(SUBS - 1) * (FM + FN)>(fa[sub], fb[sub]);
            else if (sub == 1) wait_fragments<(SUBS > 2 ? SUBS - 2 : 0) * (FM + FN)>(fa[sub], fb[sub]);
            else if (sub == 2) wait_fragments<(SUBS > 3 ? SUBS - 3 : 0) * (FM + FN)>(fa[sub], fb[sub]);
            else wait_fragments<0>(fa[sub], fb[sub]);
#pragma unroll
            for (int j = 0; j < FN; ++j)
                if (kXUnsigned) fb[sub][j] ^= (int)0x80808080;  // uint8 code - 128 as int8
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[sub][i], fb[sub][j], acc[i][j], 0, 0, 0);
#pragma unroll
            for (int q = sub * PER_SUB; q < (sub + 1) * PER_SUB && q < COPIES; ++q) issue_copy(lbuf, q);
            __builtin_amdgcn_sched_barrier(0);  // keep the read / MFMA / copy interleaving as written
        }
        advance_stage();
        lbuf = lbuf + 1 == NS ? 0 : lbuf + 1;
        if (++ck == nk) {
            epilogue(c_tile, slot);
            seed_acc();
            ck = 0;
            c_tile += px_step;
        }
    }
    wait_vmcnt<0>();  // the copies past the end still target this work-group's LDS
}

template <int FM, int FN, int BK, int NWN = 2>
int launch_config(const ConvMfmaArgs& a, bool x_unsigned, bool out_int32, bool rne, int max_wgs_per_cu, hipStream_t s) {
    // persistent work-groups: as many as the device holds at once, a whole number per
    // output-channel tile
    static int cus = 256, per_cu = 0;  // per (FM, FN); the variants of one tile shape use about the same resources
    if (per_cu == 0) {
        int dev = 0;
        per_cu = 2;
        if (hipGetDevice(&dev) == hipSuccess) {
            hipDeviceProp_t prop;
            if (hipGetDeviceProperties(&prop, dev) == hipSuccess) cus = prop.multiProcessorCount;
        }
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(
                    &per_cu, reinterpret_cast<const void*>(&conv_mfma_kernel<FM, FN, BK, true, false, false, true, false, NWN>), 128 * NWN, 0) !=
                    hipSuccess ||
            per_cu < 1)
            per_cu = 2;
    }
    const int resident = cus * (max_wgs_per_cu > 0 && max_wgs_per_cu < per_cu ? max_wgs_per_cu : per_cu);
    int slots = (a.tiles_px + 7) / 8;  // pixel-tile slots per XCD
    const int cap = resident / (8 * a.tiles_oc) > 0 ? resident / (8 * a.tiles_oc) : 1;
    if (slots > cap) slots = cap;
    const unsigned grid = (unsigned)(8 * a.tiles_oc * slots);
    // padding-free variant: no tap can leave the image and channels fill whole 64-byte K steps
    const bool pad = a.ph != 0 || a.pw != 0 || (a.C16 % BK) != 0 ||
                     (int64_t)(a.OH - 1) * a.sh + a.KH > a.H || (int64_t)(a.OW - 1) * a.sw + a.KW > a.W;
#define CHX_LAUNCH_R(XU, OI, RN, RS)                                                       \
    do {                                                                                   \
        if (pad)                                                                           \
            conv_mfma_kernel<FM, FN, BK, XU, OI, RN, true, RS, NWN><<<grid, 128 * NWN, 0, s>>>(a);    \
        else                                                                               \
            conv_mfma_kernel<FM, FN, BK, XU, OI, RN, false, RS, NWN><<<grid, 128 * NWN, 0, s>>>(a);   \
    } while (0)
#define CHX_LAUNCH(XU, OI, RN) CHX_LAUNCH_R(XU, OI, RN, false)
    if (a.res.r) {
        // the fused residual sum exists for 8-bit results in the reference's rounding
        if (out_int32 || rne) CHX_FAIL(CHX_HIP_EUNSUPPORTED, "conv_mfma: a fused residual sum needs an 8-bit result and the reference rounding");
        if (x_unsigned) CHX_LAUNCH_R(true, false, false, true);
        else CHX_LAUNCH_R(false, false, false, true);
    } else if (out_int32) {
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
#undef CHX_LAUNCH_R
    return launch_check("conv_mfma_kernel");
}

}  // namespace

int pack_weights(
        const chx_hip_tensor& w, int C64, int BK, int OCpad, int8_t* wp, int32_t* wsum, hipStream_t s) {
    pack_weights_kernel<<<OCpad, 256, 0, s>>>(
            static_cast<const char*>(w.data), w.strides[0], w.strides[1], w.strides[2], w.strides[3], (int)w.shape[0],
            (int)w.shape[1], (int)w.shape[2], (int)w.shape[3], C64, BK, wp, wsum);
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
    magic_divisor((uint32_t)a.OW, &a.ow_mul, &a.ow_shift);
    magic_divisor((uint32_t)a.OH, &a.oh_mul, &a.oh_shift);
    a.px_linear = a.KH == 1 && a.KW == 1 && a.sh == 1 && a.sw == 1 && a.ph == 0 && a.pw == 0 && a.OH == a.H && a.OW == a.W &&
                  a.x_h_stride == (int64_t)a.W * a.x_w_stride && a.x_n_stride == (int64_t)a.H * a.x_h_stride;
    a.row_unit = 0;
    if (a.KH * a.KW <= 32)
        for (int i = 0; i < a.KH; ++i) a.row_unit |= 1u << (i * a.KW);
    if (waves == 8) {
        // eight wavefronts: the pixels of the tile are split four ways
        if (tile_oc == 128 && tile_px == 128) return a.bk == 128 ? launch_config<2, 1, 128, 4>(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s)
                               : launch_config<2, 1, 64, 4>(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s);
        if (tile_oc == 128 && tile_px == 256 && a.bk == 128) return launch_config<2, 2, 128, 4>(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s);
        if (tile_oc == 64 && tile_px == 128 && a.bk == 128) return launch_config<1, 1, 128, 4>(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s);
        CHX_FAIL(CHX_HIP_EINVAL, "conv_mfma: no eight-wavefront kernel for a %dx%d tile with %d K bytes per step", tile_oc, tile_px, a.bk);
    }
    if (waves != 4) CHX_FAIL(CHX_HIP_EINVAL, "conv_mfma: work-groups have 4 or 8 wavefronts, not %d", waves);
    if (tile_oc == 128 && tile_px == 128) return a.bk == 128 ? launch_config<2, 2, 128>(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s)
                           : launch_config<2, 2, 64>(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s);
    if (tile_oc == 64 && tile_px == 128) return a.bk == 128 ? launch_config<1, 2, 128>(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s)
                           : launch_config<1, 2, 64>(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s);
    if (tile_oc == 128 && tile_px == 64) return a.bk == 128 ? launch_config<2, 1, 128>(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s)
                           : launch_config<2, 1, 64>(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s);
    if (tile_oc == 64 && tile_px == 64) return a.bk == 128 ? launch_config<1, 1, 128>(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s)
                           : launch_config<1, 1, 64>(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s);
    CHX_FAIL(CHX_HIP_EINVAL, "conv_mfma: no kernel for a %dx%d tile", tile_oc, tile_px);
}

}  // namespace chx
