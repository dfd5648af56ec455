// Direct int8 convolution for a handful of input channels read from planar (NCHW) activations:
// the first layer of an image network (3 x 7 x 7 stride 2, 3 x 3 x 3 stride 2).
//
// With so few channels a filter tap is not a usable K slice, and expanding the activations into
// an explicit [pixels][C*KH*KW] matrix costs a pass over memory several times the size of the
// input.  Here the K axis is made of the filter *rows* instead: group g = (c, kh) contributes
// the KW consecutive input bytes of one image row, padded to KWP = 4 or 8 bytes (the weights of
// the padding bytes are zero).  A work-group copies the C x PH input rows under its 8 x 16 tile
// of output pixels into LDS once; each lane then assembles its 16 K-bytes of a
// v_mfma_i32_32x32x32_i8 operand from the LDS bytes at (row of group) * pitch + ocol * stride_w
// (aligned dword reads and a byte shift: unaligned LDS reads are slow).  The packed weights of the work-group's 64 output
// channels sit in LDS in operand order for the whole kernel.
//
// Out-of-image bytes are filled with the activation zero point, which makes them contribute
// (zp - zp) * w = 0 (runtime/chainerx_util.cc:232-274); uint8 codes become int8 by flipping the
// top bit, and the accumulators are seeded with (128 - zp) * sum_k w[oc, k] as in conv_mfma.hip.
// The epilogue is the requantization of quant_math.h, codes transposed through a wave-private
// LDS area into [pixel][oc] rows and written as 128-bit stores to the channels-last output.
#include <type_traits>

#include "contract.h"
#include "conv_mfma.h"

namespace chx {
namespace {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kTileH = 8;    // output rows per work-group: two per wavefront
constexpr int kTileW = 16;   // output columns
constexpr int kMaxKB = 8;    // 32-byte K blocks
constexpr int kMaxPatchDwords = 8;  // per thread: the input patch holds at most 256 * 8 dwords

struct __attribute__((packed, aligned(1))) Unaligned4 {
    uint32_t v;
};
struct __attribute__((packed, aligned(4))) Aligned4x2 {
    v2i v;
};

// Weight repacking: w [OC][C][KH][KW] -> operand order.  Per block of 64 output channels, per
// K block kb, per 32-channel half i, lane l holds the 16 bytes  oc = i*32 + l%32,
// k = kb*32 + (l/32)*16 + 0..15  with  k = (c*KH + kh)*KWP + kw.
__global__ __launch_bounds__(256) void pack_weights_stem_kernel(
        const char* __restrict__ w, int64_t s_oc, int64_t s_c, int64_t s_kh, int64_t s_kw, int OC, int C, int KH, int KW, int KWP,
        int KB, int8_t* __restrict__ wd, int64_t total) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int b = (int)(idx & 15);
    const int l = (int)((idx >> 4) & 63);
    const int i = (int)((idx >> 10) & 1);
    const int64_t rest = idx >> 11;
    const int kb = (int)(rest % KB);
    const int ocblk = (int)(rest / KB);
    const int oc = ocblk * 64 + i * 32 + (l & 31);
    const int k = kb * 32 + (l >> 5) * 16 + b;
    const int g = k / KWP, kw = k % KWP;
    const int c = g / KH, kh = g % KH;
    int8_t v = 0;
    if (oc < OC && c < C && kw < KW) v = *reinterpret_cast<const int8_t*>(w + oc * s_oc + c * s_c + kh * s_kh + kw * s_kw);
    wd[idx] = v;
}

// n / d for n < 2^31 with the multiplier and shift of magic_divisor() (conv_mfma.h)
__device__ __forceinline__ uint32_t magic_div(uint32_t n, uint32_t mul, uint32_t shift) {
    return (__umulhi(n, mul) + n) >> shift;
}

// n / d for n < 2048 and d < 64 with m = ceil(2^20 / d)
__device__ __forceinline__ int small_div(int n, uint32_t m) {
    return (int)(((uint32_t)n * m) >> 20);
}

template <int KWP, bool kRne>
__global__ __launch_bounds__(256) void conv_stem_kernel(ConvStemArgs a) {
    constexpr int GPL = 16 / KWP;  // groups per lane and K block
    extern __shared__ __attribute__((aligned(16))) char lds[];
    // LDS: weights [KB][2][64][16] | staging [4 waves][32 px][64 oc] | constants | patch
    char* const s_w = lds;
    char* const s_stage = s_w + a.KB * 2048;
    float* const s_scale = reinterpret_cast<float*>(s_stage + 4 * 2048);
    int32_t* const s_add = reinterpret_cast<int32_t*>(s_scale + 64);
    float* const s_fbias = reinterpret_cast<float*>(s_add + 64);
    char* const s_patch = reinterpret_cast<char*>(s_fbias + 64);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int oc0 = blockIdx.y * 64;
    const int PH = (kTileH - 1) * a.sh + a.KH;            // patch rows per channel
    const int PP = ((kTileW - 1) * a.sw + KWP + 3) & ~3;  // patch row pitch, bytes
    const int patch_dwords = a.C * PH * (PP >> 2);

    // weights of this block of output channels, already in operand order
    {
        const v4i* src = reinterpret_cast<const v4i*>(a.wd + (int64_t)blockIdx.y * a.KB * 2048);
        for (int q = tid; q < a.KB * 128; q += 256) reinterpret_cast<v4i*>(s_w)[q] = src[q];
    }
    if (tid < 64) {
        const int oc = oc0 + tid;
        float sc = 0.f, fb = 0.f;
        int32_t add = 0;
        if (oc < a.OC) {
            add = a.corr_mult * a.wsum[oc];
            const float wsc = a.w_scale_len > 1 ? a.w_scale[oc] : a.w_scale[0];
            sc = a.rq.x_scale * wsc;
            if (a.bias) {
                if (a.rq.bias_mode == kBiasOnnxInt32) add += a.bias[oc];
                if (a.rq.bias_mode == kBiasReferenceFloat) fb = (float)a.bias[oc];
            }
        }
        s_scale[tid] = sc;
        s_add[tid] = add;
        s_fbias[tid] = fb;
    }

    // the patch dwords this thread fills: the same places for every tile
    int pd_row[kMaxPatchDwords] = {}, pd_col[kMaxPatchDwords] = {}, pd_off[kMaxPatchDwords] = {};
#pragma unroll
    for (int j = 0; j < kMaxPatchDwords; ++j) {
        const int d = tid + 256 * j;
        if (d >= patch_dwords) break;
        const int row = small_div(d, a.m_ppw), cw = d - row * (PP >> 2);
        const int c = small_div(row, a.m_ph), pr = row - c * PH;
        pd_row[j] = pr;
        pd_col[j] = cw * 4;
        pd_off[j] = c * (int)a.x_c_stride + pr * (int)a.x_h_stride + cw * 4;
    }

    // LDS offsets of this lane's K groups, relative to the patch: group row + pixel position
    const int p = lane & 31;
    const int orow = 2 * wave + (p >> 4), ocol = p & 15;
    const int kq = lane >> 5;
    int offs[kMaxKB][GPL];
    {
        const int G = a.C * a.KH;
        const int loff = orow * a.sh * PP + ocol * a.sw;
#pragma unroll
        for (int kb = 0; kb < kMaxKB; ++kb)
#pragma unroll
            for (int j = 0; j < GPL; ++j) {
                int g = kb * (32 / KWP) + kq * GPL + j;
                g = g < G ? g : G - 1;  // padding groups have zero weights; read something valid
                const int c = small_div(g, a.m_kh), kh = g - c * a.KH;
                offs[kb][j] = (c * PH + kh) * PP + loff;
            }
    }
    const uint32_t phase = (uint32_t)(ocol * a.sw) & 3u;  // the pitch and the group rows are multiples of 4
    const uint32_t flip = a.x_unsigned ? 0x80808080u : 0u;
    const uint32_t fill = (uint32_t)(a.x_zp & 0xff) * 0x01010101u;
    char* const my_stage = s_stage + wave * 2048;
    auto staged = [&](int pxl, int ocl) -> char* {
        return my_stage + pxl * 64 + ((((ocl >> 4) ^ (pxl >> 1)) & 3) << 4) + (ocl & 15);
    };

    const int tiles_per_image = a.tiles_h * a.tiles_w;
    const int npd = (patch_dwords + 255) >> 8;  // patch dwords per thread, rounded up
    // The patch of a tile is fetched into registers one tile ahead, so that the memory latency
    // runs under the previous tile's MFMAs and requantization.
    uint32_t pv[kMaxPatchDwords];
    auto fetch_patch = [&](int t) {
        const int n = (int)magic_div((uint32_t)t, a.tpi_mul, a.tpi_shift);
        const int r = t - n * tiles_per_image;
        const int th = (int)magic_div((uint32_t)r, a.tw_mul, a.tw_shift), tw = r - th * a.tiles_w;
        const int ih0 = th * kTileH * a.sh - a.ph, iw0 = tw * kTileW * a.sw - a.pw;
        const char* xn = a.x + (int64_t)n * a.x_n_stride + (int64_t)ih0 * a.x_h_stride + iw0;
#pragma unroll
        for (int j = 0; j < kMaxPatchDwords; ++j) {
            if (j >= npd) break;
            const int ih = ih0 + pd_row[j], iw = iw0 + pd_col[j];
            uint32_t v = fill;
            if (tid + 256 * j < patch_dwords && (unsigned)ih < (unsigned)a.H) {
                const char* src = xn + pd_off[j];
                if (iw >= 0 && iw + 3 < a.W) {
                    v = reinterpret_cast<const Unaligned4*>(src)->v;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if ((unsigned)(iw + e) < (unsigned)a.W)
                            v = (v & ~(0xffu << (8 * e))) | ((uint32_t)(uint8_t)src[e] << (8 * e));
                }
            }
            pv[j] = v;
        }
    };
    // The device deals work-groups out to its 8 XCDs in turn: the work-groups of XCD x (blockIdx.x % 8 == x; the grid's
    // x extent is a multiple of 8) share the tiles [x * chunk, (x + 1) * chunk), so that the input rows neighbouring tiles
    // have in common (15 of a tile's 21 rows for a 7x7 filter with stride 2) are found in that XCD's own L2.
    const int t_step = (int)(gridDim.x >> 3);
    const int chunk = (a.tiles + 7) >> 3;
    const int t_first = (int)(blockIdx.x & 7u) * chunk + (int)(blockIdx.x >> 3);
    const int t_end = min(((int)(blockIdx.x & 7u) + 1) * chunk, a.tiles);
    if (t_first < t_end) fetch_patch(t_first);
    for (int t = t_first; t < t_end; t += t_step) {
        const int n = (int)magic_div((uint32_t)t, a.tpi_mul, a.tpi_shift);
        const int r = t - n * tiles_per_image;
        const int th = (int)magic_div((uint32_t)r, a.tw_mul, a.tw_shift), tw = r - th * a.tiles_w;
        const int oh0 = th * kTileH, ow0 = tw * kTileW;

        __syncthreads();  // the previous tile's patch has been consumed (first pass: constants written)
#pragma unroll
        for (int j = 0; j < kMaxPatchDwords; ++j) {
            if (j >= npd) break;
            if (tid + 256 * j < patch_dwords) reinterpret_cast<uint32_t*>(s_patch)[tid + 256 * j] = pv[j];
        }
        __syncthreads();
        if (t + t_step < t_end) fetch_patch(t + t_step);

        // lane holds, per 32x32 MFMA tile: pixel column p, output-channel rows (v/4)*8 + (lane>>5)*4 + v%4
        v16i acc[2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const v4i ad = *reinterpret_cast<const v4i*>(&s_add[i * 32 + g * 8 + kq * 4]);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[i][g * 4 + e] = ad[e];
            }
#pragma unroll
        for (int kb = 0; kb < kMaxKB; ++kb) {
            if (kb >= a.KB) break;
            // the lane's window starts at any byte: read the aligned dwords around it and shift
            v4i fb;
            if (KWP == 8) {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const char* src = s_patch + (offs[kb][j] & ~3);
                    const v2i d01 = reinterpret_cast<const Aligned4x2*>(src)->v;
                    const int d2 = *reinterpret_cast<const int*>(src + 8);
                    fb[2 * j] = (int)__builtin_amdgcn_alignbyte((uint32_t)d01[1], (uint32_t)d01[0], phase);
                    fb[2 * j + 1] = (int)__builtin_amdgcn_alignbyte((uint32_t)d2, (uint32_t)d01[1], phase);
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const v2i d01 = reinterpret_cast<const Aligned4x2*>(s_patch + (offs[kb][j % GPL] & ~3))->v;
                    fb[j] = (int)__builtin_amdgcn_alignbyte((uint32_t)d01[1], (uint32_t)d01[0], phase);
                }
            }
            fb ^= (int)flip;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const v4i fa = *reinterpret_cast<const v4i*>(s_w + ((kb * 2 + i) * 64 + lane) * 16);
                acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb, acc[i], 0, 0, 0);
            }
        }

        // requantize into the wave's staging rows
        // kPath 0: any 8-bit type and rounding; 1: uint8 in the reference's rounding through
        // floor_sat_u8x4; 2: the same with a lower bound above 0 (a folded Relu)
        auto requantize_tile = [&](auto float_bias_tag, auto path_tag) {
            constexpr bool kFloatBias = decltype(float_bias_tag)::value;
            constexpr int kPath = decltype(path_tag)::value;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                if (oc0 + i * 32 >= a.OC) break;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int ocl = i * 32 + g * 8 + kq * 4;
                    const v4f sc = *reinterpret_cast<const v4f*>(&s_scale[ocl]);
                    v4f fbs = {0.f, 0.f, 0.f, 0.f};
                    if (kFloatBias) fbs = *reinterpret_cast<const v4f*>(&s_fbias[ocl]);
                    int32_t code[4];
                    float pre[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float v = (float)acc[i][g * 4 + e] * sc[e];
                        if (kFloatBias) v = v + fbs[e];
                        if (kPath == 0) code[e] = quantize_value_folded<kRne>(v, a.rq.q, a.inv_y_scale, a.lo_folded);
                        else pre[e] = quantize_prefloor_u8<kPath == 2, kPath != 3>(v, a.rq.q, a.inv_y_scale, a.lo_folded);
                    }
                    *reinterpret_cast<uint32_t*>(staged(p, ocl)) =
                            kPath == 0 ? pack4(code[0], code[1], code[2], code[3]) : floor_sat_u8x4(pre[0], pre[1], pre[2], pre[3]);
                }
            }
        };
        {
            using P0 = std::integral_constant<int, 0>;
            using P1 = std::integral_constant<int, 1>;
            using P2 = std::integral_constant<int, 2>;
            using P3 = std::integral_constant<int, 3>;  // as 1 with a zero point of 0
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
        // the staging rows are private to the wave: its own LDS operations complete in order
#pragma unroll
        for (int rr = 0; rr < 2; ++rr) {
            const int q = lane + 64 * rr;
            const int pxl = q >> 2, ch = q & 3;
            const int oh = oh0 + 2 * wave + (pxl >> 4), ow = ow0 + (pxl & 15);
            const int oc = oc0 + ch * 16;
            if (oh >= a.OH || ow >= a.OW || oc >= a.OC) continue;
            const char* src = staged(pxl, ch * 16);
            const v4i val = *reinterpret_cast<const v4i*>(src);
            char* dst = a.y + (((int64_t)n * a.OH + oh) * a.OW + ow) * a.y_px_stride + oc;
            if (a.y_vec_ok && oc + 16 <= a.OC) {
                *reinterpret_cast<v4i*>(dst) = val;
            } else {
#pragma nounroll
                for (int e = 0; e < 16 && oc + e < a.OC; ++e) dst[e] = src[e];
            }
        }
    }
}

}  // namespace

int stem_k_blocks(int C, int KH, int KW) {
    const int kwp = KW <= 4 ? 4 : 8;
    return (C * KH * kwp + 31) / 32;
}

size_t stem_patch_bytes(int C, int KH, int KW, int sh, int sw) {
    const int kwp = KW <= 4 ? 4 : 8;
    const int PH = (kTileH - 1) * sh + KH;
    const int PP = ((kTileW - 1) * sw + kwp + 3) & ~3;
    return (size_t)C * PH * PP;
}

bool stem_shape_fits(int C, int KH, int KW) {
    return KW <= 8 && C * KH <= 32 && stem_k_blocks(C, KH, KW) <= kMaxKB;
}

bool stem_patch_fits(int C, int KH, int KW, int sh, int sw) {
    const int kwp = KW <= 4 ? 4 : 8;
    // the small_div ranges: rows per channel and dwords per row below 64
    return stem_patch_bytes(C, KH, KW, sh, sw) <= (size_t)256 * kMaxPatchDwords * 4 && (kTileH - 1) * sh + KH < 64 &&
           (kTileW - 1) * sw + kwp < 252;
}

int pack_weights_stem(const chx_hip_tensor& w, int OCpad64, int8_t* wd, hipStream_t s) {
    const int C = (int)w.shape[1], KH = (int)w.shape[2], KW = (int)w.shape[3];
    const int KB = stem_k_blocks(C, KH, KW);
    const int64_t total = (int64_t)(OCpad64 / 64) * KB * 2048;
    pack_weights_stem_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(
            static_cast<const char*>(w.data), w.strides[0], w.strides[1], w.strides[2], w.strides[3], (int)w.shape[0], C, KH, KW,
            KW <= 4 ? 4 : 8, KB, wd, total);
    return launch_check("pack_weights_stem_kernel");
}

int launch_conv_stem(ConvStemArgs a, bool rne, hipStream_t s) {
    a.tiles_h = (a.OH + kTileH - 1) / kTileH;
    a.tiles_w = (a.OW + kTileW - 1) / kTileW;
    const int64_t tiles = (int64_t)a.N * a.tiles_h * a.tiles_w;
    CHX_REQUIRE(tiles < (int64_t(1) << 30), "QLinearConv: too many output tiles for the planar-input kernel");
    a.tiles = (int32_t)tiles;
    magic_divisor((uint32_t)(a.tiles_h * a.tiles_w), &a.tpi_mul, &a.tpi_shift);
    magic_divisor((uint32_t)a.tiles_w, &a.tw_mul, &a.tw_shift);
    a.KB = stem_k_blocks(a.C, a.KH, a.KW);
    {
        const int kwp = a.KW <= 4 ? 4 : 8;
        const uint32_t ppw = (uint32_t)((((kTileW - 1) * a.sw + kwp + 3) & ~3) >> 2), ph_rows = (uint32_t)((kTileH - 1) * a.sh + a.KH);
        a.m_ppw = ((1u << 20) + ppw - 1) / ppw;
        a.m_ph = ((1u << 20) + ph_rows - 1) / ph_rows;
        a.m_kh = ((1u << 20) + (uint32_t)a.KH - 1) / (uint32_t)a.KH;
    }
    // 16 bytes of slack: the aligned reads of the last window reach one dword past it
    const size_t lds = (size_t)a.KB * 2048 + 4 * 2048 + 3 * 64 * 4 + stem_patch_bytes(a.C, a.KH, a.KW, a.sh, a.sw) + 16;
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        cus = 256;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) cus = prop.multiProcessorCount;
    }
    // as many work-groups as the device holds at once, each walking over tiles with the weights resident
    int per_cu = 0;
    const void* fn = a.KW <= 4 ? reinterpret_cast<const void*>(&conv_stem_kernel<4, false>)
                               : reinterpret_cast<const void*>(&conv_stem_kernel<8, false>);
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, 256, lds) != hipSuccess || per_cu < 1) per_cu = 2;
    const int oc_blocks = (a.OC + 63) / 64;
    int per_block = cus * per_cu / oc_blocks;
    if (per_block < 1) per_block = 1;
    // (a multiple of 8 work-groups along x: see the kernel's tile order)
    const int along_x = ((a.tiles < per_block ? a.tiles : per_block) + 7) / 8 * 8;
    const dim3 grid((unsigned)along_x, (unsigned)oc_blocks);
    const bool kwp4 = a.KW <= 4;
    if (kwp4) {
        if (rne) conv_stem_kernel<4, true><<<grid, 256, lds, s>>>(a);
        else conv_stem_kernel<4, false><<<grid, 256, lds, s>>>(a);
    } else {
        if (rne) conv_stem_kernel<8, true><<<grid, 256, lds, s>>>(a);
        else conv_stem_kernel<8, false><<<grid, 256, lds, s>>>(a);
    }
    return launch_check("conv_stem_kernel");
}

}  // namespace chx
