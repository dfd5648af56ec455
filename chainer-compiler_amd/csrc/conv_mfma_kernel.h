// The matrix-core convolution kernel and its launcher as templates: one translation unit per tile shape
// (conv_mfma_t*.hip) instantiates them, so that the shapes compile side by side.
#pragma once

#include <type_traits>

#include "contract.h"
#include "conv_mfma.h"
#include "conv_device.h"

namespace chx {
namespace {

// ---------------------------------------------------------------------------------------------
// 128-bit LDS read at lds_addr + OFF whose completion the caller waits for itself (wait_fragments): the
// compiler would otherwise wait for every outstanding LDS operation at the first use, because it cannot
// see through the inline assembly of the copies issued in between.
template <int OFF>
__device__ __forceinline__ v4i lds_read16_nowait(uint32_t lds_addr) {
    v4i v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(v) : "v"(lds_addr), "n"(OFF) : "memory");
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

// f(integral_constant<int, I>) for I = 0 .. N-1, unrolled: the index is a compile-time constant inside f.
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>());
        static_for<I + 1, N>(f);
    }
}

// Touch every 64-byte line of the kernel arguments at once.  The argument block of a fresh launch
// is not in any cache, and the compiler fetches the fields in several dependent batches that
// each touch new lines: one round trip to memory per batch.  After this, one round trip.
template <int BYTES>
__device__ __forceinline__ void warm_kernel_arguments() {
    const uint64_t ka = (uint64_t)__builtin_amdgcn_kernarg_segment_ptr();
    constexpr int LINES = (BYTES + 63) / 64;
    static_assert(LINES >= 4 && LINES <= 8, "between four and eight lines are touched");
    // offsets of the last lines, clamped into the block so that nothing outside it is read
    constexpr int L4 = LINES > 4 ? 0x100 : 0xc0, L5 = LINES > 5 ? 0x140 : L4, L6 = LINES > 6 ? 0x180 : L5, L7 = LINES > 7 ? 0x1c0 : L6;
    int t0, t1, t2, t3, t4, t5, t6, t7;
    asm volatile(
            "s_load_dword %0, %8, 0x0\n\t"
            "s_load_dword %1, %8, 0x40\n\t"
            "s_load_dword %2, %8, 0x80\n\t"
            "s_load_dword %3, %8, 0xc0\n\t"
            "s_load_dword %4, %8, %9\n\t"
            "s_load_dword %5, %8, %10\n\t"
            "s_load_dword %6, %8, %11\n\t"
            "s_load_dword %7, %8, %12\n\t"
            "s_waitcnt lgkmcnt(0)"
            : "=&s"(t0), "=&s"(t1), "=&s"(t2), "=&s"(t3), "=&s"(t4), "=&s"(t5), "=&s"(t6), "=&s"(t7)
            : "s"(ka), "n"(L4), "n"(L5), "n"(L6), "n"(L7)
            : "memory");
}

// The kernel arguments, fetched again from the argument block.  The arguments a pixel tile needs once (geometry for the
// addresses, requantization and residual parameters for the epilogue) would otherwise stay in scalar registers
// throughout the K loop, which has none to spare; the loads hit the scalar cache.
template <class Args>
__device__ __forceinline__ Args kernel_arguments_again() {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef const Args __attribute__((address_space(4))) * ConstantArgs;
    uint64_t p = (uint64_t)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(p));  // not the pointer the compiler already knows: nothing is kept from earlier loads
    Args r;
    __builtin_memcpy(&r, (ConstantArgs)p, sizeof(Args));
    return r;
#else
    return Args();  // the host pass only parses the kernel
#endif
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

// Bits of a staged row's index that the 16-byte chunks of the row are XOR-swizzled with.
template <int BK>
__device__ __forceinline__ int row_swizzle(int row) {
    return BK == 64 ? (row >> 2) & 3 : (row >> 1) & 7;
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
// Copies.  Both operands are fetched through buffer resources: a lane's byte offset into the
// resource is fixed for a pixel tile (a vector register per copy instruction), the K step moves
// through a scalar offset, and the LDS destinations of a wave's copies of one operand are
// consecutive kilobytes reached by the immediate of the instruction, so a K step costs no
// vector instruction per copy and two writes of M0 per wave.  What a lane must not fetch (pixel
// rows past the end of the matrix, stages past the end of the work-group's list, the channel
// tail of the tensor's last pixel) lies outside the resource and arrives in LDS as zeros.
//
// LDS stage: rows of BK K-bytes, weight rows first, then pixel rows.  A copy instruction fills
// 1 KB = 1024/BK consecutive rows; wave w's copies of an operand fill consecutive kilobytes; a
// lane lands in a fixed (row, slot) and fetches the K chunk that the XOR swizzle places there, so
// the 128-bit fragment reads are free of bank conflicts.  BK = 128 is used when the channel
// count is a multiple of 128: then a pixel's 128 K-bytes of one filter tap are one whole cache
// line, where two 64-byte steps would each fetch the line and use half of it (the weight blocks
// are contiguous either way).
//
// Fragments are double-buffered in registers and requested one K extent (32 K-bytes) ahead, also
// across the stage barrier: the barrier of stage s sits in front of the MFMAs of its last extent,
// which therefore run while the first fragments of stage s+1 travel from LDS.  The copies of
// stage s+NS go out once that barrier has said that every wave is done reading stage s.
//
// kPad: 0, no filter tap can fall outside the image.  Otherwise each staged pixel row carries a bit
// mask of its taps (computed once per pixel tile).  1: at most 32 taps and the activation zero point is the byte 0, so
// a tap outside the image is fetched from outside the resource (one shift and one and-or on the
// lane's offset): zeros contribute (0 - 0) * w, the reference's zero padding of the already
// zero-point-subtracted tensor.  With another zero point z each such zero stands for a z and the sum misses z * w
// per tap outside: the accumulators of a pixel then start from z times the sum of the weights of its taps outside
// (ConvMfmaArgs::tap_corr; the copy side leaves each staged pixel's class of taps in LDS, the seeding reads it).
// 2: any zero point, any window; the pixel copies use flat addresses and fetch
// an invalid chunk from a 64-byte row holding the zero point instead (g_fill_rows).
//
// NWN: wavefronts along the pixel axis (two along the output channels).  2: four wavefronts, two
// work-groups per compute unit as a rule.  4: eight wavefronts on the same tile, each with half the
// pixels; a work-group then has the compute unit to itself (and the whole LDS for a deeper ring).
template <int FM, int FN, int BK, bool kXUnsigned, bool kOutInt32, bool kRne, int kPad, bool kRes, int NWN = 2>
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
    static_assert(CA <= 4 && CB <= 4, "the copies of one operand are reached by the 12-bit immediate");
    constexpr int COPIES = CA + CB;
    constexpr int SUBS = BK / 32;        // MFMA K extents per stage
    constexpr int PER_SUB = (COPIES + SUBS - 1) / SUBS;  // copies issued per extent
    constexpr int OUT_CHUNKS = TM / 16;  // 16-byte chunks per staged output row
    static_assert(TN * TM <= STAGE_BYTES, "the output tile is staged in one ring slot");
    __shared__ __attribute__((aligned(16))) char ring[NS * STAGE_BYTES];
    __shared__ __attribute__((aligned(16))) float s_scale[TM];
    // what the accumulators start from, per output channel; kPad 1: up to nine rows, one per class of taps outside the
    // image that occurs (ConvMfmaArgs::padsum), row 0 for a pixel whose taps are all inside, and each staged pixel's row
    constexpr int ADD_ROW = TM + 8;  // (rows 32 bytes off a multiple of the bank width: lanes that read different rows do not meet on a bank)
    __shared__ __attribute__((aligned(16))) int32_t s_add[kPad == 1 ? 9 * ADD_ROW : TM];
    __shared__ int32_t s_cls[kPad == 1 ? TN : 1];
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
    // (divisions by numbers the launcher knows go through its multipliers: an integer division costs a wave
    // some 150 cycles, and nothing can be fetched before these are known)
    const int slot = (int)fast_div((uint32_t)idx, a.tiles_oc_mul, a.tiles_oc_shift);
    const int oc_tile = idx - slot * a.tiles_oc;
    const int px_step = a.px_slots;  // pixel-tile slots per XCD: (gridDim.x / 8) / tiles_oc
    const int px_lo = (int)(((int64_t)a.tiles_px * xcd) >> 3);
    const int px_hi = (int)(((int64_t)a.tiles_px * (xcd + 1)) >> 3);
    const int px_first = px_lo + slot;
    const int oc0 = oc_tile * TM;
    const int my_tiles = px_first < px_hi ? (int)fast_div((uint32_t)(px_hi - px_first + px_step - 1), a.px_slots_mul, a.px_slots_shift) : 0;
    const int nk = a.nk;
    const int total_stages = my_tiles * nk;
    if (total_stages == 0) return;

    const uint32_t ring_base = (uint32_t)(uintptr_t)ring;  // LDS byte address
    // A lane of a copy instruction lands in row `rl` of the instruction's RPI rows, chunk position `pos`.
    const int rl = lane / CH, pos = lane % CH;

    // ---- copy side: weights.  The tile's rows are TM/64 blocks of nk * 64 * BK bytes; a K step is 64 * BK bytes on.
    // Offsets carry a bias of 4 KB (and the resource starts 4 KB early) so that subtracting the immediate of copy q,
    // which the instruction adds back, cannot take an offset below zero.
    constexpr uint32_t kBiasW = 4096;
    const v4i srd_w = buffer_resource(a.wp + (int64_t)oc_tile * TM * a.KP - kBiasW, (uint32_t)TM * (uint32_t)a.KP + kBiasW);
    uint32_t voffA[4] = {kOutOfRange, kOutOfRange, kOutOfRange, kOutOfRange};
#pragma unroll
    for (int q = 0; q < CA; ++q) {
        const int r = (wave * CA + q) * RPI + rl;
        const int kc = pos ^ row_swizzle<BK>(r);
        voffA[q] = kBiasW + (uint32_t)(r >> 6) * (uint32_t)(nk * 64 * BK) + (uint32_t)((r & 63) * BK + kc * 16) - (uint32_t)(q * 1024);
    }
    uint32_t soff_w = 0;  // K step * 64 * BK

    // ---- copy side: activations
    const v4i srd_x = buffer_resource(a.x - a.x_bias, a.x_bytes + a.x_bias);
    uint32_t voffB[4] = {kOutOfRange, kOutOfRange, kOutOfRange, kOutOfRange};
    uint32_t nmask[CB];      // kPad 1: bit (kh*KW + kw) set when that tap of the row's pixel is outside the image (at most 32 taps)
    const char* xb[CB];      // kPad 2: flat address of the row's tap (0, 0), channel chunk of this lane
    uint64_t tapmask[CB];    // kPad 2: bit (kh*KW + kw) set when that tap is inside the image
    int32_t c_end[CB];       // kPad 2: the lane's chunk holds channels of the tensor while the step's first channel is below this
    const char* fill_src = reinterpret_cast<const char*>(g_fill_rows) + (a.x_zp & 0xff) * 64;
    int ld_tile = px_first;  // which (pixel tile, K step) the next stage fetches
    int ld_k = 0, kw = 0, c0 = 0, tap = 0;
    uint32_t soff_x = 0;     // kh * x_h_stride + kw * x_w_stride + c0
    int lslot = 0;           // ring slot the next stage's copies fill
    keep_scalar(soff_w);
    keep_scalar(soff_x);
    keep_scalar(lslot);
    keep_scalar(tap);

    auto set_load_tile = [&]() {
        const ConvMfmaArgs a = kernel_arguments_again<ConvMfmaArgs>();
#pragma unroll
        for (int j = 0; j < CB; ++j) {
            const int rowB = (wave * CB + j) * RPI + rl;
            const int kc = pos ^ row_swizzle<BK>(rowB);
            const int64_t m = (int64_t)ld_tile * TN + rowB;
            const bool row_ok = m < a.M;
            // rows past the end fetch nothing (kPad 2: they re-read the last pixel); they are never written back
            const uint32_t mm = row_ok ? (uint32_t)m : (uint32_t)(a.M - 1);  // M fits 31 bits (checked on the host)
            int32_t off;           // byte offset of tap (0, 0), channel 0 of the row's pixel; may be negative with padding
            uint64_t mask = 1u;    // taps inside the image
            if (a.px_linear) {
                // output pixel m reads input pixel m: no decomposition into (n, oh, ow), one multiplication
                off = (int32_t)(mm * (uint32_t)a.x_w_stride);
            } else {
                const uint32_t r = fast_div(mm, a.ow_mul, a.ow_shift);
                const uint32_t ow = mm - r * (uint32_t)a.OW;
                const uint32_t n = fast_div(r, a.oh_mul, a.oh_shift);
                const uint32_t oh = r - n * (uint32_t)a.OH;
                const int ih0 = (int)oh * a.sh - a.ph;
                const int iw0 = (int)ow * a.sw - a.pw;
                // the extent of x is below 2^31 bytes (checked on the host), so 32-bit arithmetic is exact
                off = (int32_t)n * (int32_t)a.x_n_stride + ih0 * (int32_t)a.x_h_stride + iw0 * (int32_t)a.x_w_stride;
                if (kPad) {
                    // taps (i, jj) inside the image: i in [r_lo, r_hi), jj in [c_lo, c_hi)
                    const int c_lo = min(max(-iw0, 0), a.KW), c_hi = min(max(a.W - iw0, 0), a.KW);
                    const int r_lo = min(max(-ih0, 0), a.KH), r_hi = min(max(a.H - ih0, 0), a.KH);
                    if (kPad == 1 || a.KH * a.KW <= 32) {
                        // up to 32 taps (3x3, 5x5): the column bits repeated in every filter row by one
                        // multiplication with the bits KW apart, then the rows outside the image cut off
                        const uint32_t cols = c_hi > c_lo ? ((1u << c_hi) - 1u) & ~((1u << c_lo) - 1u) : 0u;
                        const uint32_t lo_bit = (uint32_t)(r_lo * a.KW), hi_bit = (uint32_t)(r_hi * a.KW);
                        const uint32_t below_hi = hi_bit >= 32 ? ~0u : (1u << hi_bit) - 1u;
                        const uint32_t rows = r_hi > r_lo ? below_hi & ~((1u << lo_bit) - 1u) : 0u;
                        mask = (cols * a.row_unit) & rows;
                        if constexpr (kPad == 1) {
                            // which sides the window leaves the image on (at most one row or column per side: the launcher
                            // has checked); every lane of the row writes the same word
                            s_cls[rowB] = a.tap_corr ? (int)((a.tap_rows >> (4 * (r_lo * 8 + (a.KH - r_hi) * 4 + c_lo * 2 + (a.KW - c_hi)))) & 15) : 0;
                        }
                    } else {
                        const uint64_t below_hi = c_hi >= 64 ? ~(uint64_t)0 : ((uint64_t)1 << c_hi) - 1;  // a 1x64 filter fills the mask
                        const uint64_t cols = c_hi > c_lo ? below_hi & ~(((uint64_t)1 << c_lo) - 1) : 0;
                        mask = 0;
                        for (int i = 0; i < a.KH; ++i)
                            if (i >= r_lo && i < r_hi) mask |= cols << (i * a.KW);
                    }
                }
            }
            if constexpr (kPad == 2) {
                xb[j] = a.x + (int64_t)off + kc * 16;
                tapmask[j] = row_ok ? mask : 0;
                c_end[j] = a.C16 - kc * 16;
            } else {
                voffB[j] = row_ok ? a.x_bias + (uint32_t)off + (uint32_t)(kc * 16) - (uint32_t)(j * 1024) : kOutOfRange;
                if constexpr (kPad == 1) nmask[j] = row_ok ? ~(uint32_t)mask : ~0u;
            }
        }
    };

    // Copies Q0 .. Q0+N-1 of the weight rows / of the pixel rows of the stage being fetched, into ring slot lslot.
    auto issue_weights = [&](auto q0_c, auto n_c) {
        constexpr int Q0 = decltype(q0_c)::value, N = decltype(n_c)::value;
        if constexpr (N > 0)
            buffer_copy16_run<N, Q0>(voffA, srd_w, soff_w, ring_base + (uint32_t)lslot * STAGE_BYTES + (uint32_t)wave * (CA * 1024));
    };
    auto issue_pixels = [&](auto j0_c, auto n_c) {
        constexpr int J0 = decltype(j0_c)::value, N = decltype(n_c)::value;
        if constexpr (N > 0) {
            const uint32_t dst = ring_base + (uint32_t)lslot * STAGE_BYTES + TM * BK + (uint32_t)wave * (CB * 1024);
            if constexpr (kPad == 2) {
#pragma unroll
                for (int j = J0; j < J0 + N; ++j) {
                    const bool ok = c0 < c_end[j] && ((tapmask[j] >> tap) & 1u);
                    async_copy16(ok ? xb[j] + soff_x : fill_src, dst + j * 1024);
                }
            } else if constexpr (kPad == 1) {
                // bit `tap` of the row's mask moves to the top of the offset: a tap outside the image fetches zeros
                uint32_t run[4] = {voffB[0], voffB[1], voffB[2], voffB[3]};
#pragma unroll
                for (int j = J0; j < J0 + N; ++j) run[j] |= (nmask[j] << (31 - tap)) & kOutOfRange;
                buffer_copy16_run<N, J0>(run, srd_x, soff_x, dst);
            } else {
                buffer_copy16_run<N, J0>(voffB, srd_x, soff_x, dst);
            }
        }
    };
    // the part of a stage's copies that is issued in one K extent: copies [c*PER_SUB, (c+1)*PER_SUB) of the
    // sequence weight rows 0..CA-1, pixel rows 0..CB-1
    auto issue_chunk = [&](auto chunk_c) {
        constexpr int c = decltype(chunk_c)::value;
        constexpr int g0 = c * PER_SUB < COPIES ? c * PER_SUB : COPIES, g1 = (c + 1) * PER_SUB < COPIES ? (c + 1) * PER_SUB : COPIES;
        constexpr int a0 = g0 < CA ? g0 : CA, a1 = g1 < CA ? g1 : CA;
        constexpr int b0 = (g0 > CA ? g0 : CA) - CA, b1 = (g1 > CA ? g1 : CA) - CA;
        issue_weights(std::integral_constant<int, a0>(), std::integral_constant<int, a1 - a0>());
        issue_pixels(std::integral_constant<int, b0>(), std::integral_constant<int, b1 - b0>());
    };
    // advance to the next K step, or to the first K step of this work-group's next pixel tile
    auto advance_stage = [&]() {
        lslot = lslot + 1 == NS ? 0 : lslot + 1;
        if (++ld_k == nk) {
            if (ld_tile + px_step < px_hi) {
                ld_k = 0; kw = 0; c0 = 0; tap = 0; soff_w = 0; soff_x = 0;
                ld_tile += px_step;
                set_load_tile();
            } else {
                // nothing follows: the remaining stages of the ring fetch nothing (zeros into slots nobody reads);
                // with flat pixel addresses they re-read the last step
                --ld_k;
#pragma unroll
                for (int q = 0; q < 4; ++q) voffA[q] = kOutOfRange;
                soff_w = 0;
                if constexpr (kPad != 2) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) voffB[j] = kOutOfRange;
                    soff_x = 0;
                }
            }
        } else {
            soff_w += 64 * BK;  // next block of the packed weights
            c0 += BK;
            if (c0 < a.C64) {
                soff_x += BK;
            } else {
                // next filter tap: one pixel to the right, or back to the first column of the next filter row
                c0 = 0;
                ++tap;
                ++kw;
                const bool row_done = kw == a.KW;
                kw = row_done ? 0 : kw;
                soff_x += row_done ? a.tap_step_row : a.tap_step_col;
            }
        }
        // the operands of the copies that must sit in scalar registers
        keep_scalar(soff_w);
        keep_scalar(soff_x);
        keep_scalar(lslot);
        keep_scalar(tap);
    };

    // kPad 1 with a zero point that is not the byte 0: the sums over the border taps of each class in use
    // (a.tap_classes: their numbers, four bits each; a.tap_corr: how many), requested first of all so that they travel
    // together with the first copies.  The T / TM threads of an output channel share the classes out (a wavefront
    // holds one share); every instruction here delays the work-group's first matrix instruction.
    constexpr int SHARES = T / TM;
    constexpr int SHARE_MAX = (8 + SHARES - 1) / SHARES;
    static_assert(T % TM == 0 && TM % 64 == 0, "whole wavefronts per share of the classes");
    int32_t border[SHARE_MAX];
    if constexpr (kPad == 1) {
        if (a.tap_corr) {
            const int share = __builtin_amdgcn_readfirstlane(tid / TM);
            const int32_t* mine = a.padsum + min(oc0 + tid % TM, a.OC - 1);
#pragma unroll
            for (int k = 0; k < SHARE_MAX; ++k) {
                border[k] = 0;
                if (k * SHARES + share < a.tap_corr) border[k] = mine[(int64_t)((a.tap_classes >> (4 * (k * SHARES + share))) & 15) * a.padsum_stride];
            }
        }
    }
    // the first NS-1 stages go out before anything else touches memory; the weight rows of the very first one
    // do not wait for the pixel addresses
    issue_weights(std::integral_constant<int, 0>(), std::integral_constant<int, CA>());
    set_load_tile();
    issue_pixels(std::integral_constant<int, 0>(), std::integral_constant<int, CB>());
    advance_stage();
#pragma unroll
    for (int d = 1; d < NS - 1; ++d) {
        issue_weights(std::integral_constant<int, 0>(), std::integral_constant<int, CA>());
        issue_pixels(std::integral_constant<int, 0>(), std::integral_constant<int, CB>());
        advance_stage();
    }

    // per-channel epilogue constants; s_add seeds the accumulators.  One thread per output channel; with class rows
    // to fill (kPad 1, see `border`) every share of the threads works the channel's constant out for itself.
    const bool all_shares = kPad == 1 && a.tap_corr;
    if (tid < TM || all_shares) {
        const int i = tid % TM;
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
        if (tid < TM) {
            s_scale[i] = sc;
            s_add[i] = add;
            s_fbias[i] = fb;
        }
        if constexpr (kPad == 1) {
            // taps outside the image arrive as the byte 0 where the tensor would hold the zero point: each contributes
            // w * x_zp too little.  Row c of s_add = row 0 + x_zp * the border sums of class c.
            if (a.tap_corr) {
                const int share = __builtin_amdgcn_readfirstlane(tid / TM);
#pragma unroll
                for (int k = 0; k < SHARE_MAX; ++k)
                    if (k * SHARES + share < a.tap_corr)
                        s_add[(k * SHARES + share + 1) * ADD_ROW + i] = add + a.x_zp * border[k];  // the class's row: its place in the list + 1
            }
        }
    }
    __syncthreads();

    // lane holds, per 32x32 MFMA tile: pixel column (lane & 31), output-channel rows
    // (v / 4) * 8 + (lane >> 5) * 4 + (v % 4)
    v16i acc[FM][FN];
    auto seed_acc = [&]() {
        if constexpr (kPad == 1) {
            // the row of the pixel's class (s_cls holds the classes of the tile about to be computed: the copy side wrote
            // them when it turned to that tile, at least one barrier ago, and turns to the tile after it only once this
            // one is under way)
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const int32_t* row = &s_add[s_cls[wn * 32 * FN + j * 32 + (lane & 31)] * ADD_ROW + wm * 32 * FM + (lane >> 5) * 4];
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const v4i ad = *reinterpret_cast<const v4i*>(&row[i * 32 + g * 8]);
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[i][j][g * 4 + e] = ad[e];
                    }
            }
            return;
        }
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
    // The 8-bit tile is transposed through the ring slot that was just consumed (every wave is done reading
    // its operands: the stage barrier said so; the copies in flight target the other slots, and the caller
    // lets the next copies into this one only behind a barrier of its own): rows of TM bytes per pixel, the 16-byte chunks of a row
    // XOR-swizzled with bits 1.. of the pixel index so that neither the 4-byte writes of the
    // accumulator layout nor the 16-byte reads of the store loop pile up on a bank.
    auto staged = [&](char* slot, int pxl, int ocl) -> char* {
        return slot + pxl * TM + ((((ocl >> 4) ^ (pxl >> 1)) & (OUT_CHUNKS - 1)) << 4) + (ocl & 15);
    };
    auto epilogue = [&](int px_tile, char* lds_out) {
        ConvMfmaArgs a = kernel_arguments_again<ConvMfmaArgs>();
        if (a.oc_split > 0) {
            // two convolutions in this launch: the tile is one of the second's (its output and quantization take the
            // first's place, its channel 0 is this launch's channel oc_split), or the first's channels end at oc_split
            if (oc0 >= a.oc_split) {
                a.y = a.y2 - a.oc_split;
                a.y_px_stride = a.y2_px_stride;
                a.y_vec_ok = a.y2_vec_ok;
                a.y_flip = a.y2_flip;
                a.rq.q = a.q2;
                a.inv_y_scale = a.inv_y_scale2;
                a.lo_folded = a.lo_folded2;
            } else {
                a.OC = a.oc_split;
            }
        }
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
        // the constants of the per-element arithmetic in vector registers (in_vector_register says why)
        const QuantParams rq_q = in_vector_registers(a.rq.q);
        const float inv_y_scale = in_vector_register(a.inv_y_scale);
        const float lo_folded = in_vector_register(a.lo_folded);
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
                                code[e] = quantize_value_folded<kRne>(v, rq_q, inv_y_scale, lo_folded);
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
                                            quantize_prefloor_u8<kPath == 2, kPath != 3>(v, rq_q, inv_y_scale, lo_folded);
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
                ResidualAdd res;
                if constexpr (kMode != 0) res = in_vector_registers(a.res);
                const int store_flip = (int)in_vector_register(a.y_flip);
#pragma unroll
                for (int it = 0; it < ITER; ++it) {
                    const int q = tid + it * T;
                    const int pxl = q / OUT_CHUNKS;
                    const int ch = q % OUT_CHUNKS;
                    v4i val = *reinterpret_cast<const v4i*>(staged(lds_out, pxl, ch * 16));
                    if constexpr (kMode == 1) val = affine_residual16<false>(val, rres[it], res);
                    if constexpr (kMode == 2) val = affine_residual16<true>(val, rres[it], res);
                    if constexpr (kMode == 3) val = add_residual16_any(val, rres[it], res);
                    val ^= store_flip;
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
            }
            val ^= (int)a.y_flip;
            if (!(a.y_vec_ok && whole)) *reinterpret_cast<v4i*>(src) = val;  // the byte loop below reads LDS
            char* dst = a.y + m * a.y_px_stride + oc;
            if (a.y_vec_ok && whole) {
                *reinterpret_cast<v4i*>(dst) = val;
            } else {
#pragma nounroll
                for (int e = 0; e < 16 && oc + e < a.OC; ++e) dst[e] = src[e];
            }
        }
    };

    // ---- the pipeline ----
    // Fragment reads: the lane's part of the address is fixed per K extent (row of the 32x32 tile and the swizzled
    // chunk), the wave's part is scalar, the 32-row blocks of a wave's rows are reached by the immediate.
    const int frag_row = lane & 31;
    const int frag_kc = lane >> 5;
    uint32_t lane_off[SUBS];
#pragma unroll
    for (int sub = 0; sub < SUBS; ++sub) lane_off[sub] = (uint32_t)(frag_row * BK + (((sub * 2 + frag_kc) ^ row_swizzle<BK>(frag_row)) << 4));
    const uint32_t wave_a = ring_base + (uint32_t)(wm * 32 * FM * BK);
    const uint32_t wave_b = ring_base + (uint32_t)(TM * BK + wn * 32 * FN * BK);
    // Fragments live in NB register buffers and are requested D K extents (of 32 K-bytes) ahead of their MFMAs, also
    // across the stage barrier: with four extents per stage two ahead (an LDS read takes longer than the MFMAs of one
    // extent), buffer = extent; with two extents per stage one ahead.
#ifndef CHX_CONV_FRAGMENT_LEAD
#define CHX_CONV_FRAGMENT_LEAD 2
#endif
    constexpr int D = SUBS >= 4 ? CHX_CONV_FRAGMENT_LEAD : 1;
    constexpr int NB = SUBS >= 4 ? SUBS : 2;
    constexpr int NM = FM * FN;          // MFMAs per extent
    constexpr int READS = FM + FN;       // fragment reads per extent
    v4i fa[NB][FM], fb[NB][FN];
    int flip;  // in a vector register: a literal would make every flip an eight-byte instruction, a scalar register a four-cycle one
    asm volatile("v_mov_b32 %0, 0x80808080" : "=v"(flip));
    auto read_one = [&](auto buf_c, auto sub_c, auto r_c, uint32_t slot_off) {
        constexpr int buf = decltype(buf_c)::value, sub = decltype(sub_c)::value, r = decltype(r_c)::value;
        if constexpr (r < FM) fa[buf][r] = lds_read16_nowait<r * 32 * BK>(wave_a + slot_off + lane_off[sub]);
        else fb[buf][r - FM] = lds_read16_nowait<(r - FM) * 32 * BK>(wave_b + slot_off + lane_off[sub]);
    };
    auto read_fragments = [&](auto buf_c, auto sub_c, uint32_t slot_off) {
        static_for<0, READS>([&](auto r_c) { read_one(buf_c, sub_c, r_c, slot_off); });
    };
    auto flip_one = [&](auto buf_c, auto j_c) {
        constexpr int buf = decltype(buf_c)::value, j = decltype(j_c)::value;
        if (kXUnsigned) fb[buf][j] ^= flip;  // uint8 code - 128 as int8
    };

    // Stage 0 has landed when at most the NS-2 younger stages of this wave's copies are outstanding; the barrier
    // extends that to every wave's copies.  Every stage issues the same number of copies and none is
    // conditional, so a fixed vector-memory count identifies the stage about to be consumed.
    wait_vmcnt<(NS - 2) * COPIES>();
    __builtin_amdgcn_s_barrier();
    // the pipeline starts with extent 0 in its buffer, flipped, and the next D-1 extents requested
    read_fragments(std::integral_constant<int, 0>(), std::integral_constant<int, 0>(), 0u);
    if constexpr (D == 2) read_fragments(std::integral_constant<int, 1>(), std::integral_constant<int, 1>(), 0u);
    if constexpr (D == 2) wait_fragments<READS>(fa[0], fb[0]);
    else wait_fragments<0>(fa[0], fb[0]);
    static_for<0, FN>([&](auto j_c) { flip_one(std::integral_constant<int, 0>(), j_c); });

    // The copies of a stage go out in SUBS parts, one per extent, starting in the extent that holds the barrier
    // (extent SUBS-D of the stage whose slot they overwrite); the first D parts of stage NS-1 go out here.
    constexpr int BAR = SUBS - D;  // the extent whose beginning holds the stage barrier
    static_for<0, D>([&](auto part_c) { issue_chunk(part_c); });
    int ck = 0;             // K step within the tile being computed
    int c_tile = px_first;  // pixel tile being computed
    int cbuf = 0;           // ring slot being computed
    for (int s = 0; s < total_stages; ++s) {
        const uint32_t slot_off = (uint32_t)cbuf * STAGE_BYTES;
        cbuf = cbuf + 1 == NS ? 0 : cbuf + 1;
        const uint32_t next_off = (uint32_t)cbuf * STAGE_BYTES;
        const bool last_k = ck + 1 == nk;  // the tile is finished behind this stage: its slot stages the output
        static_for<0, SUBS>([&](auto sub_c) {
            constexpr int sub = decltype(sub_c)::value;
            constexpr int cur = sub % NB;              // buffer of this extent: ready and flipped
            constexpr int nxt = (sub + 1) % NB;        // buffer of the next extent: requested, or (D == 1) about to be
            constexpr int far = (sub + D) % NB;        // buffer requested in this extent
            constexpr int far_sub = (sub + D) % SUBS;  // ... which is this extent of this stage or of the next
            constexpr bool far_next = sub + D >= SUBS;
            if constexpr (sub == BAR) {
                // This wave's copies of stage s+1 have landed when at most the NS-2 younger stages are outstanding, and
                // its reads of stage s are complete (the last of them were requested an extent ago); the barrier
                // extends both to every wave: stage s+1 can be read, and the slot of stage s can be overwritten.
                wait_vmcnt<(NS - 2) * COPIES>();
                wait_fragments<0>(fa[nxt], fb[nxt]);
                __builtin_amdgcn_s_barrier();
            }
            // MFMA m of this extent, then a share of what prepares the extents behind it: the reads of extent sub+D,
            // the wait for extent sub+1, its sign flips
            constexpr int ITEMS = READS + 1 + FN;
            constexpr int PER = (ITEMS + NM - 1) / NM;
            static_for<0, NM>([&](auto m_c) {
                constexpr int m = decltype(m_c)::value;
                acc[m / FN][m % FN] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[cur][m / FN], fb[cur][m % FN], acc[m / FN][m % FN], 0, 0, 0);
                static_for<m * PER, ((m + 1) * PER < ITEMS ? (m + 1) * PER : ITEMS)>([&](auto it_c) {
                    constexpr int it = decltype(it_c)::value;
                    if constexpr (it < READS) {
                        read_one(std::integral_constant<int, far>(), std::integral_constant<int, far_sub>(), it_c, far_next ? next_off : slot_off);
                    } else if constexpr (it == READS) {
                        // extent sub+1 is there when at most the reads just issued are outstanding (with D == 1 they are
                        // the ones waited for)
                        if constexpr (D == 2) wait_fragments<READS>(fa[nxt], fb[nxt]);
                        else wait_fragments<0>(fa[nxt], fb[nxt]);
                    } else {
                        flip_one(std::integral_constant<int, nxt>(), std::integral_constant<int, it - READS - 1>());
                    }
                });
                __builtin_amdgcn_sched_barrier(0);  // keep the MFMA / read / flip interleaving as written
            });
            // copies: part (sub - BAR) mod SUBS of the stage that overwrites the slot freed by the last barrier
            constexpr int part = (sub - BAR + SUBS) % SUBS;
            if constexpr (sub >= BAR) {
                // of stage s+NS, into the slot of stage s; when that slot stages the output tile they wait for the epilogue
                if (!last_k) issue_chunk(std::integral_constant<int, part>());
            } else {
                issue_chunk(std::integral_constant<int, part>());
            }
            if constexpr (part == SUBS - 1) advance_stage();
            __builtin_amdgcn_sched_barrier(0);
        });
        if (last_k) {
            epilogue(c_tile, ring + slot_off);
            seed_acc();
            ck = 0;
            c_tile += px_step;
            // the staged tile has been read by every wave before the copies held back above overwrite the slot
            if (!kOutInt32) __builtin_amdgcn_s_barrier();
            static_for<0, D>([&](auto part_c) {
                issue_chunk(part_c);
                if constexpr (decltype(part_c)::value == SUBS - 1) advance_stage();
            });
        } else {
            ++ck;
        }
    }
    // the fragments requested past the end, and the copies past the end, still target this work-group's registers and LDS
    wait_fragments<0>(fa[0], fb[0]);
    wait_vmcnt<0>();
}

template <int FM, int FN, int BK, int NWN = 2>
int launch_config(const ConvMfmaArgs& a_in, bool x_unsigned, bool out_int32, bool rne, int max_wgs_per_cu, hipStream_t s) {
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
                    &per_cu, reinterpret_cast<const void*>(&conv_mfma_kernel<FM, FN, BK, true, false, false, 2, false, NWN>), 128 * NWN, 0) !=
                    hipSuccess ||
            per_cu < 1)
            per_cu = 2;
    }
    const int resident = cus * (max_wgs_per_cu > 0 && max_wgs_per_cu < per_cu ? max_wgs_per_cu : per_cu);
    int slots = (a_in.tiles_px + 7) / 8;  // pixel-tile slots per XCD
    const int cap = resident / (8 * a_in.tiles_oc) > 0 ? resident / (8 * a_in.tiles_oc) : 1;
    if (slots > cap) slots = cap;
    const unsigned grid = (unsigned)(8 * a_in.tiles_oc * slots);
    ConvMfmaArgs a = a_in;
    a.px_slots = slots;
    magic_divisor((uint32_t)slots, &a.px_slots_mul, &a.px_slots_shift);
    magic_divisor((uint32_t)a.tiles_oc, &a.tiles_oc_mul, &a.tiles_oc_shift);
    // no tap can leave the image: 0; else 1 when the zero point is the byte 0 and 32 bits hold a pixel's tap mask (a tap
    // outside the image is fetched as zeros), 2 otherwise (it is fetched from a row of zero points)
    const bool pad = a.ph != 0 || a.pw != 0 || (int64_t)(a.OH - 1) * a.sh + a.KH > a.H || (int64_t)(a.OW - 1) * a.sw + a.KW > a.W;
    // (with another zero point still 1 when the accumulators can start from what the zeros miss: border sums packed, the
    // window leaves the image by at most one row or column per side, and enough K steps per tile that the copy side is
    // never more than one tile ahead of the seeding, which reads the classes it leaves in LDS)
    const int last_ih0 = (a.OH - 1) * a.sh - a.ph, last_iw0 = (a.OW - 1) * a.sw - a.pw;
    const int below = a.KH - (a.H - last_ih0 < 0 ? 0 : a.H - last_ih0 > a.KH ? a.KH : a.H - last_ih0);
    const int right = a.KW - (a.W - last_iw0 < 0 ? 0 : a.W - last_iw0 > a.KW ? a.KW : a.W - last_iw0);
    a.tap_corr = 0;
    a.tap_classes = 0;
    a.tap_rows = 0;
    bool class_seeds = pad && (a.x_zp & 0xff) != 0 && a.KH * a.KW <= 32 && a.padsum != nullptr && a.ph <= 1 && a.pw <= 1 && below <= 1 &&
                       right <= 1 && a.nk >= 4;
    if (class_seeds) {
        // the classes in use: 4 * (2 * rows outside above + rows outside below) + 2 * columns outside left + columns outside
        // right, over the output rows and columns that can differ from the interior (the first and the last few)
        auto sides = [](int O, int stride, int p, int I, int K) {
            uint32_t seen = 0;
            for (int o = 0; o < O; ++o) {
                if (o == 4 && O > 8) o = O - 4;
                const int i0 = o * stride - p;
                const int lo = -i0 < 0 ? 0 : -i0 > K ? K : -i0, hi = I - i0 < 0 ? 0 : I - i0 > K ? K : I - i0;
                seen |= 1u << ((lo * 2 + (K - hi)) & 3);
            }
            return seen;
        };
        const uint32_t rows = sides(a.OH, a.sh, a.ph, a.H, a.KH), cols = sides(a.OW, a.sw, a.pw, a.W, a.KW);
        int count = 0;
        uint64_t classes = 0, table_rows = 0;
        for (int cls = 1; cls < 16; ++cls)
            if (((rows >> (cls >> 2)) & 1) && ((cols >> (cls & 3)) & 1)) {
                classes |= (uint64_t)cls << (4 * count);
                ++count;
                table_rows |= (uint64_t)(count & 15) << (4 * cls);
            }
        // (padding means that some pixel has a tap outside: at least one class besides 0; more than eight only where a
        // window leaves the image on opposite sides at once, images one or two pixels high or wide)
        class_seeds = count >= 1 && count <= 8;
        if (class_seeds) {
            a.tap_corr = count;
            a.tap_classes = classes;
            a.tap_rows = table_rows;
        }
    }
    const int pad_mode = !pad ? 0 : (a.KH * a.KW <= 32 && ((a.x_zp & 0xff) == 0 || class_seeds)) ? 1 : 2;
#define CHX_LAUNCH_R(XU, OI, RN, RS)                                                    \
    do {                                                                                \
        if (pad_mode == 0)                                                              \
            conv_mfma_kernel<FM, FN, BK, XU, OI, RN, 0, RS, NWN><<<grid, 128 * NWN, 0, s>>>(a); \
        else if (pad_mode == 1)                                                         \
            conv_mfma_kernel<FM, FN, BK, XU, OI, RN, 1, RS, NWN><<<grid, 128 * NWN, 0, s>>>(a); \
        else                                                                            \
            conv_mfma_kernel<FM, FN, BK, XU, OI, RN, 2, RS, NWN><<<grid, 128 * NWN, 0, s>>>(a); \
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
}  // namespace chx
