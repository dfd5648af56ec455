// Entry points of the integer contractions: QLinearConv, ConvInteger, MatMulInteger,
// QLinearMatMul.  Validation and shape rules follow the reference's RunImpl bodies
// (runtime/ops/quantize.cc:62-146) and GroupedConv (runtime/chainerx_util.cc:313-340);
// the arithmetic is in the kernels.
#include <climits>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "contract.h"
#include "conv_mfma.h"
#include "depthwise.h"

namespace chx {
namespace {

struct ConvShape {
    int32_t N, C, H, W, OC, Cg, KH, KW, OH, OW;
};

int conv_shape(
        const chx_hip_tensor& x, const chx_hip_tensor& w, const chx_hip_conv_params& p, const chx_hip_tensor& y,
        const char* op, ConvShape* cs) {
    CHX_REQUIRE(x.ndim == 4 && w.ndim == 4 && y.ndim == 4, "%s: x, w and y must be 4-D (2-D convolution only)", op);
    CHX_REQUIRE(is_q8(x.dtype), "%s: x must be uint8 or int8, got %s", op, dtype_name(x.dtype));
    CHX_REQUIRE(is_q8(w.dtype), "%s: w must be uint8 or int8, got %s", op, dtype_name(w.dtype));
    CHX_REQUIRE(p.group >= 1 && p.stride_h >= 1 && p.stride_w >= 1, "%s: group and strides must be positive", op);
    CHX_REQUIRE(p.pad_h_begin >= 0 && p.pad_w_begin >= 0 && p.pad_h_end >= 0 && p.pad_w_end >= 0,
                "%s: negative padding is not supported", op);
    for (int i = 0; i < 4; ++i)
        CHX_REQUIRE(x.shape[i] <= INT32_MAX && w.shape[i] <= INT32_MAX, "%s: extent too large", op);
    cs->N = (int32_t)x.shape[0];
    cs->C = (int32_t)x.shape[1];
    cs->H = (int32_t)x.shape[2];
    cs->W = (int32_t)x.shape[3];
    cs->OC = (int32_t)w.shape[0];
    cs->Cg = (int32_t)w.shape[1];
    cs->KH = (int32_t)w.shape[2];
    cs->KW = (int32_t)w.shape[3];
    CHX_REQUIRE(cs->C == cs->Cg * p.group, "%s: x has %d channels but w expects %d x group %d", op, cs->C, cs->Cg, p.group);
    CHX_REQUIRE(cs->OC % p.group == 0, "%s: %d output channels do not divide into %d groups", op, cs->OC, p.group);
    const int64_t eh = (int64_t)cs->H + p.pad_h_begin + p.pad_h_end - cs->KH;
    const int64_t ew = (int64_t)cs->W + p.pad_w_begin + p.pad_w_end - cs->KW;
    CHX_REQUIRE(eh >= 0 && ew >= 0, "%s: kernel %dx%d larger than the padded input", op, cs->KH, cs->KW);
    cs->OH = (int32_t)(eh / p.stride_h + 1);
    cs->OW = (int32_t)(ew / p.stride_w + 1);
    CHX_REQUIRE(y.shape[0] == cs->N && y.shape[1] == cs->OC && y.shape[2] == cs->OH && y.shape[3] == cs->OW,
                "%s: y is [%lld,%lld,%lld,%lld], expected [%d,%d,%d,%d]", op, (long long)y.shape[0], (long long)y.shape[1],
                (long long)y.shape[2], (long long)y.shape[3], cs->N, cs->OC, cs->OH, cs->OW);
    return CHX_HIP_OK;
}

// A 0-d or 1-d parameter array with `expect_one_or` elements.
int param_vector(const chx_hip_tensor& t, int64_t per_channel, const char* what, int64_t* len, int64_t* stride) {
    CHX_REQUIRE(t.ndim <= 1, "%s must be 0-d or 1-d", what);
    *len = numel(t);
    CHX_REQUIRE(*len == 1 || *len == per_channel, "%s has %lld elements, expected 1 or %lld", what, (long long)*len,
                (long long)per_channel);
    *stride = t.ndim == 1 ? t.strides[0] : 0;
    return CHX_HIP_OK;
}

void fill_conv_args(
        const chx_hip_tensor& x, const chx_hip_tensor& w, const chx_hip_conv_params& p, const chx_hip_tensor& y,
        const ConvShape& cs, ConvDirectArgs* a) {
    memset(a, 0, sizeof(*a));
    a->x = static_cast<const char*>(x.data);
    a->w = static_cast<const char*>(w.data);
    a->y = static_cast<char*>(y.data);
    for (int i = 0; i < 4; ++i) {
        a->xs[i] = x.strides[i];
        a->ws[i] = w.strides[i];
        a->ys[i] = y.strides[i];
    }
    a->N = cs.N; a->C = cs.C; a->H = cs.H; a->W = cs.W;
    a->OC = cs.OC; a->Cg = cs.Cg; a->KH = cs.KH; a->KW = cs.KW; a->OH = cs.OH; a->OW = cs.OW;
    a->sh = p.stride_h; a->sw = p.stride_w; a->ph = p.pad_h_begin; a->pw = p.pad_w_begin; a->group = p.group;
    a->x_signed = x.dtype == CHX_HIP_INT8;
    a->w_signed = w.dtype == CHX_HIP_INT8;
    a->total = (int64_t)cs.N * cs.OC * cs.OH * cs.OW;
    a->D = a->KD = a->OD = a->sd = 1;  // no third spatial axis
}

int fill_requant(
        float x_scale, float y_scale, int32_t y_zp, const chx_hip_tensor& y, const chx_hip_tensor* bias, int64_t bias_len,
        uint32_t flags, const char* op, RequantParams* rq, const int32_t** bias_ptr) {
    CHX_REQUIRE(is_q8(y.dtype), "%s: y must be uint8 or int8, got %s", op, dtype_name(y.dtype));
    const bool i8 = y.dtype == CHX_HIP_INT8;
    CHX_REQUIRE(y_zp >= (i8 ? -128 : 0) && y_zp <= (i8 ? 127 : 255), "%s: zero point %d outside the range of %s", op,
                y_zp, dtype_name(y.dtype));
    rq->q = make_quant_params(y_scale, y_zp, i8);
    rq->x_scale = x_scale;
    rq->relu_floor = (flags & CHX_HIP_FUSE_RELU) ? y_zp : INT32_MIN;
    rq->bias_mode = kBiasNone;
    *bias_ptr = nullptr;
    if (bias) {
        CHX_PROPAGATE(check_tensor(bias, "bias"));
        CHX_REQUIRE(bias->dtype == CHX_HIP_INT32, "%s: bias must be int32, got %s", op, dtype_name(bias->dtype));
        CHX_REQUIRE(bias->ndim == 1 && bias->shape[0] == bias_len && is_contiguous(*bias),
                    "%s: bias must be a contiguous [%lld] vector", op, (long long)bias_len);
        rq->bias_mode = (flags & CHX_HIP_BIAS_ONNX_INT32) ? kBiasOnnxInt32 : kBiasReferenceFloat;
        *bias_ptr = static_cast<const int32_t*>(bias->data);
    }
    return CHX_HIP_OK;
}

struct MatMulShape {
    int64_t batch, M, K, N;
    int64_t a_batch, b_batch, y_batch;
};

// NumpyMatMul, runtime/chainerx_util.cc:210-230: 2-D Dot, or N-D with equal leading dims
// flattened into a batch.  Leading dims must be contiguous among themselves.
int matmul_shape(const chx_hip_tensor& a, const chx_hip_tensor& b, const chx_hip_tensor& y, const char* op, MatMulShape* ms) {
    CHX_REQUIRE(a.ndim >= 2 && b.ndim == a.ndim && y.ndim == a.ndim, "%s: a, b and y must have the same ndim >= 2", op);
    const int nd = a.ndim;
    ms->M = a.shape[nd - 2];
    ms->K = a.shape[nd - 1];
    ms->N = b.shape[nd - 1];
    CHX_REQUIRE(b.shape[nd - 2] == ms->K, "%s: inner dimensions differ (%lld vs %lld)", op, (long long)ms->K,
                (long long)b.shape[nd - 2]);
    CHX_REQUIRE(y.shape[nd - 2] == ms->M && y.shape[nd - 1] == ms->N, "%s: y has the wrong matrix shape", op);
    ms->batch = 1;
    for (int i = 0; i < nd - 2; ++i) {
        CHX_REQUIRE(a.shape[i] == b.shape[i] && a.shape[i] == y.shape[i], "%s: leading dimensions differ", op);
        ms->batch *= a.shape[i];
    }
    auto batch_stride = [&](const chx_hip_tensor& t, int64_t* out) -> int {
        // leading axes must collapse into one
        *out = 0;
        int64_t expect = -1;
        for (int i = nd - 3; i >= 0; --i) {
            if (t.shape[i] == 1) continue;
            if (expect < 0) {
                *out = t.strides[i];
                expect = t.strides[i] * t.shape[i];
            } else {
                CHX_REQUIRE(t.strides[i] == expect, "%s: leading dimensions are not collapsible", op);
                expect *= t.shape[i];
            }
        }
        return CHX_HIP_OK;
    };
    CHX_PROPAGATE(batch_stride(a, &ms->a_batch));
    CHX_PROPAGATE(batch_stride(b, &ms->b_batch));
    CHX_PROPAGATE(batch_stride(y, &ms->y_batch));
    return CHX_HIP_OK;
}

void fill_matmul_args(
        const chx_hip_tensor& a, const chx_hip_tensor& b, const chx_hip_tensor& y, const MatMulShape& ms, MatMulDirectArgs* m) {
    memset(m, 0, sizeof(*m));
    const int nd = a.ndim;
    m->a = static_cast<const char*>(a.data);
    m->b = static_cast<const char*>(b.data);
    m->y = static_cast<char*>(y.data);
    m->a_batch = ms.a_batch; m->a_row = a.strides[nd - 2]; m->a_col = a.strides[nd - 1];
    m->b_batch = ms.b_batch; m->b_row = b.strides[nd - 2]; m->b_col = b.strides[nd - 1];
    m->y_batch = ms.y_batch; m->y_row = y.strides[nd - 2]; m->y_col = y.strides[nd - 1];
    m->M = ms.M; m->K = ms.K; m->N = ms.N;
    m->total = ms.batch * ms.M * ms.N;
    m->a_signed = a.dtype == CHX_HIP_INT8;
    m->b_signed = b.dtype == CHX_HIP_INT8;
}


// ---- MFMA path -------------------------------------------------------------------------------

inline int round_up(int v, int m) {
    return (v + m - 1) / m * m;
}

// Packed weights for the MFMA kernel (see conv_mfma.hip).
struct PackedWeights {
    int8_t* wp = nullptr;
    int32_t* wsum = nullptr;
    int32_t* padsum = nullptr;  // ConvMfmaArgs::padsum (inside wsum's allocation), null for dense packing and for more than 32 taps
    int C64 = 0, OCpad = 0, KP = 0;
    int BK = 64;         // K bytes per kernel step; the packed layout depends on it
    bool dense = false;  // taps packed densely; activations go through an explicit im2col
    int8_t* wd = nullptr;  // dense only: the same weights in the order of the planar-input kernel (inside wp's allocation)
};

// Dense packing pays when per-tap padding to 64 channels would at least double the K extent.
bool prefer_dense(int C, int KH, int KW) {
    return KH * KW > 1 && round_up(C, 64) * KH * KW >= 2 * round_up(C * KH * KW, 64);
}

size_t packed_bytes(int OC, int C, int KH, int KW, PackedWeights* pw) {
    pw->OCpad = round_up(OC, 128);
    pw->dense = prefer_dense(C, KH, KW);
    if (pw->dense) {
        pw->KP = round_up(C * KH * KW, 64);
        pw->C64 = pw->KP;
    } else {
        pw->C64 = round_up(C, 64);
        pw->KP = KH * KW * pw->C64;
    }
    // whole cache lines per pixel and step when the channels allow it
    pw->BK = (!pw->dense && pw->C64 % 128 == 0) ? 128 : 64;
    return (size_t)pw->OCpad * pw->KP;
}

// The weights qualify for the MFMA kernel: one group, int8, accumulator cannot overflow.
bool weights_fit_mfma(const chx_hip_tensor& w, int group) {
    if (group != 1 || w.dtype != CHX_HIP_INT8) return false;
    if (w.shape[1] > (1 << 20) || w.shape[2] * w.shape[3] > 64) return false;  // one mask bit per filter tap
    PackedWeights pw;
    packed_bytes(1, (int)w.shape[1], (int)w.shape[2], (int)w.shape[3], &pw);
    return (int64_t)pw.KP * 128 * 128 < (int64_t(1) << 31) && w.shape[0] < (1 << 24);
}

// How a convolution is launched, beyond what its operands decide.  The defaults are what a host wants; the
// environment variables are overrides for tuning and for tests (which reach every launch configuration through them),
// read when a plan is created or a one-shot entry point is called, never on the path of a plan's runs.
//   CHX_HIP_TILE=<oc>,<px>[,<work-groups per compute unit>[,<wavefronts: 4 or 8>]]  forces a launch configuration
//   CHX_HIP_AUTOTUNE=0          keeps the heuristic tile choice instead of timing the configurations
//   CHX_HIP_NO_STEM=1           keeps few-channel first layers off the planar-input kernel
//   CHX_HIP_AFFINE_RESIDUAL=0   keeps fused residual sums on the operation-by-operation arithmetic
struct LaunchOptions {
    bool forced_tile = false;
    int tile_oc = 0, tile_px = 0, max_wgs_per_cu = 0, waves = 4;
    bool autotune = true;
    bool stem_kernel = true;
    bool affine_residual = true;
};

LaunchOptions read_launch_options() {
    LaunchOptions o;
    if (const char* env = getenv("CHX_HIP_TILE")) {
        int toc = 0, tpx = 0, cap = 0, wv = 4;
        const int got = sscanf(env, "%d,%d,%d,%d", &toc, &tpx, &cap, &wv);
        if (got >= 2 && cap >= 0) {
            o.forced_tile = true;
            o.tile_oc = toc;
            o.tile_px = tpx;
            o.max_wgs_per_cu = got >= 3 ? cap : 0;
            o.waves = wv;
            o.autotune = false;
        }
    }
    if (const char* e = getenv("CHX_HIP_AUTOTUNE")) o.autotune = o.autotune && e[0] != '0';
    o.stem_kernel = getenv("CHX_HIP_NO_STEM") == nullptr;
    if (const char* e = getenv("CHX_HIP_AFFINE_RESIDUAL")) o.affine_residual = e[0] != '0';
    return o;
}

// Tile shape: the largest tile that still gives every compute unit a work-group.
void pick_tile(const LaunchOptions& opt, int OC, int64_t M, int bk, int* tile_oc, int* tile_px, int* max_wgs_per_cu, int* waves) {
    *waves = 4;
    if (opt.forced_tile) {
        const int toc = opt.tile_oc, tpx = opt.tile_px, wv = opt.waves;
        const bool four = wv == 4 && (toc == 64 || toc == 128) && (tpx == 64 || tpx == 128);
        const bool eight = wv == 8 && ((toc == 128 && tpx == 128) || (bk == 128 && ((toc == 128 && tpx == 256) || (toc == 64 && tpx == 128))));
        if (four || eight) {
            *tile_oc = toc;
            *tile_px = tpx;
            *max_wgs_per_cu = opt.max_wgs_per_cu;
            *waves = wv;
            return;
        }
    }
    static const int cand[4][2] = {{128, 128}, {64, 128}, {128, 64}, {64, 64}};
    const int64_t want = 256;
    for (int i = 0; i < 4; ++i) {
        int toc = cand[i][0], tpx = cand[i][1];
        if (OC <= 64 && toc > 64) continue;
        const int64_t blocks = (int64_t)((OC + toc - 1) / toc) * ((M + tpx - 1) / tpx);
        *tile_oc = toc;
        *tile_px = tpx;
        if (blocks >= want) return;
    }
}

// Launch configurations measured for the input shapes a plan has seen: the first eager call on
// a new shape times every tile shape and occupancy cap on the call's own operands (every
// configuration writes the same bytes) and later calls reuse the fastest.
struct TunedConfig {
    int64_t M;
    int32_t H, W, OH, OW;
    int tile_oc, tile_px, max_wgs_per_cu;
    int waves;      // wavefronts per work-group: 4 or 8
    bool with_res;  // measured with a fused residual sum (an entry of its own: the epilogue differs)
    int32_t oc_split = 0;  // measured as two convolutions in one launch, split here (restricts the tiles)
};
struct TuneCache {
    std::vector<TunedConfig> entries;
};

// Times every launch configuration on the call's operands and keeps the fastest in *best.
int tune_conv_mfma(const ConvMfmaArgs& a, bool xu, bool out_int32, bool rne, hipStream_t s, TunedConfig* best) {
    // tile (output channels x pixels), wavefronts; the eight-wavefront kernels take the compute unit alone
    static const int tiles[7][3] = {{128, 128, 4}, {64, 128, 4}, {128, 64, 4}, {64, 64, 4}, {128, 128, 8}, {128, 256, 8}, {64, 128, 8}};
    static const int caps[3] = {0, 2, 1};
    hipEvent_t e0, e1;
    CHX_HIP_CALL(hipEventCreate(&e0));
    CHX_HIP_CALL(hipEventCreate(&e1));
    float best_ms = -1.f;
    int rc = CHX_HIP_OK;
    for (int t = 0; t < 7 && rc == CHX_HIP_OK; ++t) {
        if (a.OC <= 64 && tiles[t][0] > 64) continue;
        if (a.oc_split % tiles[t][0] != 0) continue;  // two outputs: a tile belongs to one of them whole
        if (tiles[t][2] == 8 && (tiles[t][0] == 64 || tiles[t][1] == 256) && a.bk != 128) continue;
        for (int c = 0; c < (tiles[t][2] == 8 ? 1 : 3) && rc == CHX_HIP_OK; ++c) {
            const int reps = 3;
            rc = launch_conv_mfma(a, tiles[t][0], tiles[t][1], caps[c], tiles[t][2], xu, out_int32, rne, s);  // warm
            if (rc != CHX_HIP_OK) break;
            if (hipEventRecord(e0, s) != hipSuccess) rc = CHX_HIP_ERUNTIME;
            for (int r = 0; r < reps && rc == CHX_HIP_OK; ++r)
                rc = launch_conv_mfma(a, tiles[t][0], tiles[t][1], caps[c], tiles[t][2], xu, out_int32, rne, s);
            if (rc != CHX_HIP_OK) break;
            float ms = 0.f;
            if (hipEventRecord(e1, s) != hipSuccess || hipEventSynchronize(e1) != hipSuccess ||
                hipEventElapsedTime(&ms, e0, e1) != hipSuccess) {
                rc = CHX_HIP_ERUNTIME;
                break;
            }
            if (best_ms < 0.f || ms < best_ms) {
                best_ms = ms;
                best->tile_oc = tiles[t][0];
                best->tile_px = tiles[t][1];
                best->max_wgs_per_cu = caps[c];
                best->waves = tiles[t][2];
            }
        }
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc != CHX_HIP_OK) CHX_FAIL(rc, "timing the convolution launch configurations failed: %s", chx_hip_last_error());
    return CHX_HIP_OK;
}

struct XLayout {
    const char* ptr;
    int64_t n_stride, h_stride, w_stride;
    bool direct;  // usable as is
};

// channels-last view with 16-byte aligned pixels whose pitch covers round_up(C, 16) bytes
bool x_is_mfma_ready(const chx_hip_tensor& x) {
    const int64_t C = x.shape[1];
    if (C != 1 && x.strides[1] != 1) return false;
    const int64_t c16 = (C + 15) / 16 * 16;
    if (!aligned(x.data, 16)) return false;
    for (int ax : {0, 2, 3}) {
        if (x.shape[ax] == 1) continue;
        if (x.strides[ax] % 16 != 0 || x.strides[ax] < c16) return false;
    }
    // reading c16 bytes of the last pixel must stay inside the allocation: guaranteed when every
    // pixel pitch covers c16 bytes, which the loop above checked for all axes of extent > 1
    if (x.shape[3] == 1 && x.shape[2] == 1 && x.shape[0] == 1) return C == c16;
    return true;
}

// pixel-major output: (n, oh, ow) collapse to one index with a single stride, channels unit stride
bool y_is_pixel_major(const chx_hip_tensor& y, int64_t* px_stride) {
    const int64_t es = dtype_size(y.dtype);
    if (y.shape[1] != 1 && y.strides[1] != es) return false;
    int64_t stride = -1, expect = -1;
    for (int ax : {3, 2, 0}) {
        if (y.shape[ax] == 1) continue;
        if (stride < 0) {
            stride = y.strides[ax];
            expect = stride * y.shape[ax];
        } else {
            if (y.strides[ax] != expect) return false;
            expect *= y.shape[ax];
        }
    }
    if (stride < 0) stride = y.shape[1] * es;
    if (stride < y.shape[1] * es) return false;
    *px_stride = stride;
    return true;
}

// [lowest, highest + 1) byte address any element of t occupies
void byte_range(const chx_hip_tensor& t, uintptr_t* lo, uintptr_t* hi) {
    int64_t below = 0, above = dtype_size(t.dtype);
    for (int i = 0; i < t.ndim; ++i) {
        if (t.shape[i] <= 1) continue;
        const int64_t span = (t.shape[i] - 1) * t.strides[i];
        if (span < 0) below += span;
        else above += span;
    }
    *lo = reinterpret_cast<uintptr_t>(t.data) + below;
    *hi = reinterpret_cast<uintptr_t>(t.data) + above;
}

bool byte_ranges_overlap(const chx_hip_tensor& a, const chx_hip_tensor& b) {
    if (numel(a) == 0 || numel(b) == 0) return false;
    uintptr_t alo, ahi, blo, bhi;
    byte_range(a, &alo, &ahi);
    byte_range(b, &blo, &bhi);
    return alo < bhi && blo < ahi;
}

// Scratch buffers that outlive a call: a plan keeps its transposition / im2col space so that
// repeated runs allocate nothing (and can be captured into a HIP graph).  Grow-only.
struct ScratchCache {
    void* ptr[2] = {nullptr, nullptr};
    size_t size[2] = {0, 0};
    bool pinned = false;  // a recorded run holds these addresses: the buffers must not move
};

struct ConvCall {
    TuneCache* tune;      // null: heuristic tile choice
    ScratchCache* cache;  // null: stream-ordered scratch for this call only
    const chx_hip_tensor* x;
    chx_hip_tensor* y;
    const chx_hip_conv_params* p;
    ConvShape cs;
    int32_t x_zp;
    bool out_int32;
    bool rne;
    const float* w_scale;
    int32_t w_scale_len;
    const int32_t* bias;
    RequantParams rq;
    const ResidualAdd* res = nullptr;  // a residual sum fused behind the requantization
    LaunchOptions opt;                 // the plan's, or read for this one-shot call
    // two convolutions of x in one launch (ConvMfmaArgs::oc_split): the second one's output and requantization
    const chx_hip_tensor* y2 = nullptr;
    int32_t oc_split = 0;
    RequantParams rq2;
    // CHX_HIP_STORE_MINUS_128 for y / y2: the stored byte is the uint8 code minus 128
    bool y_minus_128 = false, y2_minus_128 = false;
};

// Runs the MFMA kernel on packed weights.  x may be channels-last (used in place) or
// NCHW-contiguous (transposed into scratch first); y may be pixel-major (written in place) or
// NCHW-contiguous 8-bit (written to scratch, then transposed).  Returns EUNSUPPORTED when the
// operand layouts fit neither, so that the caller can fall back to the direct kernel.
int acquire_scratch(ScratchCache* cache, int slot, size_t bytes, hipStream_t s, void** out) {
    if (!cache) return scratch_alloc(out, bytes, s);
    if (cache->size[slot] < bytes) {
        if (cache->pinned)
            CHX_FAIL(CHX_HIP_EPINNED,
                     "this convolution plan is pinned by a recorded run and would have to move its scratch memory (%zu bytes needed, %zu held): "
                     "run larger inputs before recording, or after the recording has been destroyed", bytes, cache->size[slot]);
        // the old buffer may still be in use by work queued on the stream
        CHX_HIP_CALL(hipStreamSynchronize(s));
        if (cache->ptr[slot]) CHX_HIP_CALL(hipFree(cache->ptr[slot]));
        cache->ptr[slot] = nullptr;
        cache->size[slot] = 0;
        CHX_HIP_CALL(hipMalloc(&cache->ptr[slot], bytes));
        cache->size[slot] = bytes;
    }
    *out = cache->ptr[slot];
    return CHX_HIP_OK;
}

void release_scratch(ScratchCache* cache, void* p, hipStream_t s) {
    if (!cache) scratch_free(p, s);
}

int run_conv_mfma(const ConvCall& c, const PackedWeights& pw, hipStream_t s) {
    const chx_hip_tensor& x = *c.x;
    chx_hip_tensor& y = *c.y;
    const ConvShape& cs = c.cs;
    const int C16 = round_up(cs.C, 16);
    void* x_scratch = nullptr;
    void* y_scratch = nullptr;
    ConvMfmaArgs a;
    memset(&a, 0, sizeof(a));
    int KH = cs.KH, KW = cs.KW, H = cs.H, W = cs.W, sh = c.p->stride_h, sw = c.p->stride_w, ph = c.p->pad_h_begin,
        pw_ = c.p->pad_w_begin, C16eff = C16;
    // few channels read from planar rows: the direct kernel, no expanded matrix
    const bool stem = pw.dense && pw.wd && !c.out_int32 && x.strides[3] == 1 &&
                      stem_patch_fits(cs.C, cs.KH, cs.KW, sh, sw) && ph < 64 && pw_ < 64 &&
                      (int64_t)cs.C * (x.strides[1] < 0 ? -x.strides[1] : x.strides[1]) < (int64_t(1) << 30) &&
                      x.strides[2] > 0 && (int64_t)cs.H * x.strides[2] < (int64_t(1) << 30) && c.opt.stem_kernel;
    if (stem && c.res) CHX_FAIL(CHX_HIP_EUNSUPPORTED, "the planar-input kernel has no fused residual sum");
    if (stem) {
        // x is used in place
    } else if (pw.dense) {
        // explicit im2col: [M][Kd] bytes, then a 1x1 convolution over Kd channels and M pixels in a row
        const int64_t M = (int64_t)cs.N * cs.OH * cs.OW;
        CHX_REQUIRE(M <= INT32_MAX, "QLinearConv: too many output pixels for the im2col path");
        CHX_PROPAGATE(acquire_scratch(c.cache, 0, (size_t)M * pw.KP, s, &x_scratch));
        Im2colArgs ia;
        memset(&ia, 0, sizeof(ia));
        ia.x = static_cast<const char*>(x.data);
        for (int i = 0; i < 4; ++i) ia.xs[i] = x.strides[i];
        ia.C = cs.C; ia.H = cs.H; ia.W = cs.W; ia.OH = cs.OH; ia.OW = cs.OW; ia.KH = cs.KH; ia.KW = cs.KW;
        ia.sh = sh; ia.sw = sw; ia.ph = ph; ia.pw = pw_;
        ia.Kd = pw.KP;
        ia.fill = c.x_zp;
        ia.M = M;
        ia.col = static_cast<char*>(x_scratch);
        const int rc = launch_im2col_dense(ia, s);
        if (rc != CHX_HIP_OK) {
            release_scratch(c.cache, x_scratch, s);
            return rc;
        }
        a.x = static_cast<const char*>(x_scratch);
        a.x_w_stride = pw.KP;
        a.x_h_stride = 0;
        a.x_n_stride = 0;
        KH = KW = 1; H = 1; W = (int)M; sh = sw = 1; ph = pw_ = 0;
        C16eff = pw.KP;
    } else if (x_is_mfma_ready(x)) {
        a.x = static_cast<const char*>(x.data);
        a.x_n_stride = x.strides[0];
        a.x_h_stride = x.strides[2];
        a.x_w_stride = x.strides[3];
    } else if (is_contiguous(x)) {
        const int64_t HW = (int64_t)cs.H * cs.W;
        CHX_PROPAGATE(acquire_scratch(c.cache, 0, (size_t)cs.N * HW * C16, s, &x_scratch));
        CHX_PROPAGATE(launch_nchw_to_nhwc_u8(static_cast<const char*>(x.data), static_cast<char*>(x_scratch), cs.N, cs.C,
                                             HW, C16, s));
        a.x = static_cast<const char*>(x_scratch);
        a.x_w_stride = C16;
        a.x_h_stride = (int64_t)cs.W * C16;
        a.x_n_stride = HW * C16;
    } else {
        CHX_FAIL(CHX_HIP_EUNSUPPORTED, "x layout is neither channels-last nor NCHW-contiguous");
    }
    const int64_t es = c.out_int32 ? 4 : 1;
    int64_t y_px = 0;
    bool y_post = false;
    if (y_is_pixel_major(y, &y_px)) {
        a.y = static_cast<char*>(y.data);
        a.y_px_stride = y_px;
    } else if (is_contiguous(y) && !c.out_int32 && !c.res) {
        const int64_t OHW = (int64_t)cs.OH * cs.OW;
        const int pitch = round_up(cs.OC, 16);
        const int rc_y = acquire_scratch(c.cache, 1, (size_t)cs.N * OHW * pitch, s, &y_scratch);
        if (rc_y != CHX_HIP_OK) {
            release_scratch(c.cache, x_scratch, s);
            return rc_y;
        }
        a.y = static_cast<char*>(y_scratch);
        a.y_px_stride = pitch;
        y_post = true;
    } else {
        release_scratch(c.cache, x_scratch, s);
        CHX_FAIL(CHX_HIP_EUNSUPPORTED, "y layout is neither pixel-major nor NCHW-contiguous 8-bit");
    }
    a.y_vec_ok = aligned(a.y, 16) && (a.y_px_stride % 16 == 0) ? 1 : 0;
    (void)es;
    if (c.y_minus_128 || c.y2_minus_128) {
        if (stem || y_post || c.out_int32) {
            release_scratch(c.cache, x_scratch, s);
            release_scratch(c.cache, y_scratch, s);
            CHX_FAIL(CHX_HIP_EUNSUPPORTED, "QLinearConv: codes minus 128 are stored by the matrix-core kernel into channels-last results only");
        }
        a.y_flip = c.y_minus_128 ? 0x80808080u : 0u;
    }
    if (c.y2) {
        int64_t y2_px = 0;
        if (stem || pw.dense || x_scratch || y_post || c.out_int32 || c.res || !y_is_pixel_major(*c.y2, &y2_px)) {
            release_scratch(c.cache, x_scratch, s);
            release_scratch(c.cache, y_scratch, s);
            CHX_FAIL(CHX_HIP_EUNSUPPORTED, "QLinearConv pair: needs channels-last x, y1 and y2 and at least 16 input channels");
        }
        a.oc_split = c.oc_split;
        a.y2 = static_cast<char*>(c.y2->data);
        a.y2_px_stride = y2_px;
        a.y2_vec_ok = aligned(a.y2, 16) && (y2_px % 16 == 0) ? 1 : 0;
        a.y2_flip = c.y2_minus_128 ? 0x80808080u : 0u;
        a.q2 = c.rq2.q;
        a.inv_y_scale2 = 1.0f / c.rq2.q.scale;
        a.lo_folded2 = fold_relu_floor(c.rq2.q, c.rq2.relu_floor, c.rne);
    }
    if (stem) {
        ConvStemArgs sa;
        memset(&sa, 0, sizeof(sa));
        sa.x = static_cast<const char*>(x.data);
        sa.x_n_stride = x.strides[0]; sa.x_c_stride = x.strides[1]; sa.x_h_stride = x.strides[2];
        sa.N = cs.N; sa.C = cs.C; sa.H = cs.H; sa.W = cs.W; sa.OH = cs.OH; sa.OW = cs.OW; sa.KH = cs.KH; sa.KW = cs.KW;
        sa.sh = sh; sa.sw = sw; sa.ph = ph; sa.pw = pw_;
        sa.OC = cs.OC;
        sa.wd = pw.wd;
        sa.wsum = pw.wsum;
        sa.x_zp = c.x_zp;
        sa.x_unsigned = x.dtype == CHX_HIP_UINT8 ? 1 : 0;
        sa.corr_mult = sa.x_unsigned ? 128 - c.x_zp : -c.x_zp;
        sa.y = a.y; sa.y_px_stride = a.y_px_stride; sa.y_vec_ok = a.y_vec_ok;
        sa.w_scale = c.w_scale; sa.w_scale_len = c.w_scale_len; sa.bias = c.bias;
        sa.rq = c.rq;
        sa.inv_y_scale = 1.0f / c.rq.q.scale;
        sa.lo_folded = fold_relu_floor(c.rq.q, c.rq.relu_floor, c.rne);
        int rc = launch_conv_stem(sa, c.rne, s);
        if (rc == CHX_HIP_OK && y_post) {
            rc = launch_nhwc_to_nchw_u8(static_cast<const char*>(y_scratch), static_cast<char*>(y.data), cs.N, cs.OC,
                                        (int64_t)cs.OH * cs.OW, (int)a.y_px_stride, s);
        }
        release_scratch(c.cache, y_scratch, s);
        return rc;
    }
    a.C16 = C16eff;
    {
        // bytes from x to the end of the last pixel's C16 channels (the strides of the three cases above are positive)
        const int64_t n_img = pw.dense ? 1 : cs.N, h_img = pw.dense ? 1 : H, w_img = pw.dense ? (int64_t)cs.N * cs.OH * cs.OW : W;
        const int64_t span = (n_img - 1) * a.x_n_stride + (h_img - 1) * a.x_h_stride + (w_img - 1) * a.x_w_stride + C16eff;
        if (span >= (int64_t(1) << 31) - (int64_t(1) << 24)) {
            release_scratch(c.cache, x_scratch, s);
            release_scratch(c.cache, y_scratch, s);
            CHX_FAIL(CHX_HIP_EUNSUPPORTED, "QLinearConv: the activations span 2 GB or more, which the MFMA kernel does not address");
        }
        a.x_bytes = (uint32_t)span;
    }
    a.C64 = pw.C64;
    a.H = H; a.W = W; a.KH = KH; a.KW = KW;
    a.OH = pw.dense ? 1 : cs.OH;
    a.OW = pw.dense ? (int)((int64_t)cs.N * cs.OH * cs.OW) : cs.OW;
    a.sh = sh; a.sw = sw; a.ph = ph; a.pw = pw_;
    a.M = (int64_t)cs.N * cs.OH * cs.OW;
    a.OC = cs.OC;
    a.KP = pw.KP;
    a.bk = pw.BK;
    a.nk = pw.KP / pw.BK;
    a.wp = pw.wp;
    a.wsum = pw.wsum;
    a.padsum = pw.padsum;
    a.padsum_stride = pw.OCpad;
    a.x_zp = c.x_zp;
    const bool xu = x.dtype == CHX_HIP_UINT8;
    a.corr_mult = xu ? 128 - c.x_zp : -c.x_zp;
    a.w_scale = c.w_scale;
    a.w_scale_len = c.w_scale_len;
    a.bias = c.bias;
    a.rq = c.rq;
    a.inv_y_scale = c.out_int32 ? 0.f : 1.0f / c.rq.q.scale;
    a.lo_folded = fold_relu_floor(c.rq.q, c.rq.relu_floor, c.rne);
    if (c.res) a.res = *c.res;
    CHX_REQUIRE(a.M < (int64_t(1) << 31), "QLinearConv: too many output pixels for the MFMA kernel");
    int toc = 64, tpx = 64, cap = 0, waves = 4;
    pick_tile(c.opt, cs.OC, a.M, a.bk, &toc, &tpx, &cap, &waves);
    if (a.oc_split % toc != 0) toc = 64, waves = 4, tpx = tpx > 128 ? 128 : tpx;  // (the split is a multiple of 64)
    int rc = CHX_HIP_OK;
    const TunedConfig* tuned = nullptr;
    if (c.tune) {
        for (const TunedConfig& t : c.tune->entries)
            if (t.M == a.M && t.H == a.H && t.W == a.W && t.OH == a.OH && t.OW == a.OW && t.with_res == (c.res != nullptr) && t.oc_split == a.oc_split) tuned = &t;
        if (!tuned && c.opt.autotune && !stream_is_capturing(s)) {
            TunedConfig best = {a.M, a.H, a.W, a.OH, a.OW, toc, tpx, 0, waves, c.res != nullptr, a.oc_split};
            rc = tune_conv_mfma(a, xu, c.out_int32, c.rne, s, &best);
            if (rc == CHX_HIP_OK) {
                c.tune->entries.push_back(best);
                tuned = &c.tune->entries.back();
            }
        }
    }
    if (tuned) {
        toc = tuned->tile_oc;
        tpx = tuned->tile_px;
        cap = tuned->max_wgs_per_cu;
        waves = tuned->waves;
    }
    if (rc == CHX_HIP_OK) rc = launch_conv_mfma(a, toc, tpx, cap, waves, xu, c.out_int32, c.rne, s);
    if (rc == CHX_HIP_OK && y_post) {
        rc = launch_nhwc_to_nchw_u8(static_cast<const char*>(y_scratch), static_cast<char*>(y.data), cs.N, cs.OC,
                                    (int64_t)cs.OH * cs.OW, (int)a.y_px_stride, s);
    }
    release_scratch(c.cache, x_scratch, s);
    release_scratch(c.cache, y_scratch, s);
    return rc;
}

// Reads a small parameter vector back to the host (synchronizes the stream).
int read_back(const chx_hip_tensor& t, std::vector<uint8_t>* out, hipStream_t s) {
    const int64_t n = numel(t);
    out->resize((size_t)n);
    if (n == 0) return CHX_HIP_OK;
    if (t.ndim == 0 || t.strides[0] == 1 || n == 1) {
        CHX_HIP_CALL(hipMemcpyAsync(out->data(), t.data, (size_t)n, hipMemcpyDeviceToHost, s));
    } else {
        CHX_HIP_CALL(hipMemcpy2DAsync(out->data(), 1, t.data, (size_t)t.strides[0], 1, (size_t)n, hipMemcpyDeviceToHost, s));
    }
    CHX_HIP_CALL(hipStreamSynchronize(s));
    return CHX_HIP_OK;
}

bool all_zero(const std::vector<uint8_t>& v) {
    for (uint8_t b : v)
        if (b) return false;
    return true;
}

}  // namespace
}  // namespace chx

using namespace chx;


namespace chx {
namespace {

// Allocates and fills packed weights.  With `persistent` the buffers come from hipMalloc and
// live until release_packed(); otherwise they are stream-ordered scratch.
int make_packed(const chx_hip_tensor& w, bool persistent, hipStream_t s, PackedWeights* pw) {
    const size_t mfma_bytes = packed_bytes((int)w.shape[0], (int)w.shape[1], (int)w.shape[2], (int)w.shape[3], pw);
    const bool stem = pw->dense && stem_shape_fits((int)w.shape[1], (int)w.shape[2], (int)w.shape[3]);
    const size_t stem_bytes =
            stem ? (size_t)(pw->OCpad / 64) * stem_k_blocks((int)w.shape[1], (int)w.shape[2], (int)w.shape[3]) * 2048 : 0;
    const size_t bytes = mfma_bytes + stem_bytes;
    // the per-channel sums, and behind them the sixteen classes of border sums
    // (between 2 and 32 taps: the kernel's tap masks hold 32, and a single tap that can lie outside is rare enough for
    // the flat-address padding)
    const bool border_sums = !pw->dense && w.shape[2] * w.shape[3] <= 32 && w.shape[2] * w.shape[3] > 1;
    const size_t sums_bytes = sizeof(int32_t) * pw->OCpad * (border_sums ? 17 : 1);
    void* p0 = nullptr;
    void* p1 = nullptr;
    if (persistent) {
        CHX_HIP_CALL(hipMalloc(&p0, bytes));
        if (hipMalloc(&p1, sums_bytes) != hipSuccess) {
            (void)hipFree(p0);
            CHX_FAIL(CHX_HIP_ERUNTIME, "hipMalloc failed for the per-channel weight sums");
        }
    } else {
        CHX_PROPAGATE(scratch_alloc(&p0, bytes, s));
        if (scratch_alloc(&p1, sums_bytes, s) != CHX_HIP_OK) {
            scratch_free(p0, s);
            return CHX_HIP_ERUNTIME;
        }
    }
    pw->wp = static_cast<int8_t*>(p0);
    pw->wsum = static_cast<int32_t*>(p1);
    pw->padsum = border_sums ? pw->wsum + pw->OCpad : nullptr;
    pw->wd = stem ? pw->wp + mfma_bytes : nullptr;
    if (stem) CHX_PROPAGATE(pack_weights_stem(w, pw->OCpad, pw->wd, s));
    if (pw->dense) return pack_weights_dense(w, pw->KP, pw->BK, pw->OCpad, pw->wp, pw->wsum, s);
    return pack_weights(w, pw->C64, pw->BK, pw->OCpad, pw->wp, pw->wsum, pw->padsum, s);
}

void release_packed(PackedWeights* pw, bool persistent, hipStream_t s) {
    if (persistent) {
        if (pw->wp) (void)hipFree(pw->wp);
        if (pw->wsum) (void)hipFree(pw->wsum);
    } else {
        scratch_free(pw->wp, s);
        scratch_free(pw->wsum, s);
    }
    pw->wp = nullptr;
    pw->wsum = nullptr;
    pw->padsum = nullptr;
    pw->wd = nullptr;
}

// Depthwise 3x3 on int8 weights with zero weight zero points: packed filter rows and per-channel sums.
struct DepthwiseState {
    int C = 0;
    void* block = nullptr;  // one allocation: rows | wsum
    int32_t* rows = nullptr;
    int32_t* wsum = nullptr;
};

bool weights_fit_depthwise(const chx_hip_tensor& w, int group) {
    return w.dtype == CHX_HIP_INT8 && group > 1 && w.shape[0] == group && w.shape[1] == 1 && w.shape[2] == 3 &&
           w.shape[3] == 3 && group % 16 == 0;
}

int make_depthwise(const chx_hip_tensor& w, bool persistent, hipStream_t s, DepthwiseState* st) {
    const int C = (int)w.shape[0];
    const size_t rows_bytes = (size_t)(C / 4) * 12 * sizeof(int32_t);
    const size_t total = rows_bytes + (size_t)C * 4;
    void* p = nullptr;
    if (persistent) CHX_HIP_CALL(hipMalloc(&p, total));
    else CHX_PROPAGATE(scratch_alloc(&p, total, s));
    st->C = C;
    st->block = p;
    char* b = static_cast<char*>(p);
    st->rows = reinterpret_cast<int32_t*>(b);
    st->wsum = reinterpret_cast<int32_t*>(b + rows_bytes);
    return pack_depthwise(w, st->rows, st->wsum, s);
}

void release_depthwise(DepthwiseState* st, bool persistent, hipStream_t s) {
    if (!st->block) return;
    if (persistent) (void)hipFree(st->block);
    else scratch_free(st->block, s);
    st->block = nullptr;
}

// channels-last 8-bit tensor whose pixels are 16-byte aligned vectors of C bytes
bool is_depthwise_layout(const chx_hip_tensor& t) {
    if (!is_q8(t.dtype) || t.strides[1] != 1 || !aligned(t.data, 16)) return false;
    for (int ax : {0, 2, 3})
        if (t.shape[ax] != 1 && (t.strides[ax] % 16 != 0 || t.strides[ax] < t.shape[1])) return false;
    return true;
}

struct QConvChecked {
    ConvShape cs;
    ConvDirectArgs direct;
};

// Validation shared by the one-shot call and the plan: everything QLinearConvOp::RunImpl CHECKs.
int check_qconv(
        const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, const chx_hip_tensor* w,
        const chx_hip_tensor* w_scale, const chx_hip_tensor* w_zero_point, float y_scale, int32_t y_zero_point,
        const chx_hip_tensor* bias, const chx_hip_conv_params* params, uint32_t flags, chx_hip_tensor* y, QConvChecked* out) {
    CHX_PROPAGATE(check_tensor(x, "QLinearConv x"));
    CHX_PROPAGATE(check_tensor(w, "QLinearConv w"));
    CHX_PROPAGATE(check_tensor(w_scale, "QLinearConv w_scale"));
    CHX_PROPAGATE(check_tensor(w_zero_point, "QLinearConv w_zero_point"));
    CHX_PROPAGATE(check_tensor(y, "QLinearConv y"));
    CHX_REQUIRE(params != nullptr, "QLinearConv: null params");
    ConvShape& cs = out->cs;
    CHX_PROPAGATE(conv_shape(*x, *w, *params, *y, "QLinearConv", &cs));
    CHX_REQUIRE(w_scale->dtype == CHX_HIP_FLOAT32, "QLinearConv: w_scale must be float32");
    CHX_REQUIRE(w_zero_point->dtype == w->dtype, "QLinearConv: w_zero_point must have the dtype of w");
    // CHECK_EQ(w_scale.GetTotalSize(), w_zero_point.GetTotalSize()), runtime/ops/quantize.cc:76-77
    int64_t slen, sstride, zlen, zstride;
    CHX_PROPAGATE(param_vector(*w_scale, cs.OC, "QLinearConv w_scale", &slen, &sstride));
    CHX_PROPAGATE(param_vector(*w_zero_point, cs.OC, "QLinearConv w_zero_point", &zlen, &zstride));
    CHX_REQUIRE(slen == zlen && w_scale->ndim == w_zero_point->ndim,
                "QLinearConv: w_scale and w_zero_point must have the same shape");
    CHX_REQUIRE(slen == 1 || sstride == 4, "QLinearConv: w_scale must be contiguous");
    ConvDirectArgs& a = out->direct;
    fill_conv_args(*x, *w, *params, *y, cs, &a);
    a.x_zp = x_zero_point;
    a.w_zp = static_cast<const char*>(w_zero_point->data);
    a.w_zp_len = (int32_t)zlen;
    a.w_zp_stride = zstride;
    a.requant = 1;
    a.w_scale = static_cast<const float*>(w_scale->data);
    a.w_scale_len = (int32_t)slen;
    CHX_PROPAGATE(fill_requant(x_scale, y_scale, y_zero_point, *y, bias, cs.OC, flags, "QLinearConv", &a.rq, &a.bias));
    return CHX_HIP_OK;
}

ConvCall conv_call_from(const QConvChecked& q, const chx_hip_tensor* x, chx_hip_tensor* y, const chx_hip_conv_params* p,
                        bool rne, const LaunchOptions& opt) {
    ConvCall c;
    c.opt = opt;
    c.cache = nullptr;
    c.tune = nullptr;
    c.x = x;
    c.y = y;
    c.p = p;
    c.cs = q.cs;
    c.x_zp = q.direct.x_zp;
    c.out_int32 = false;
    c.rne = rne;
    c.w_scale = q.direct.w_scale;
    c.w_scale_len = q.direct.w_scale_len;
    c.bias = q.direct.bias;
    c.rq = q.direct.rq;
    return c;
}

// Runs the depthwise kernel; EUNSUPPORTED when the operand layouts are not channels-last.
int run_depthwise(const ConvCall& c, const DepthwiseState& st, hipStream_t s) {
    const chx_hip_tensor& x = *c.x;
    const chx_hip_tensor& y = *c.y;
    if (!is_depthwise_layout(x) || !is_depthwise_layout(y))
        CHX_FAIL(CHX_HIP_EUNSUPPORTED, "depthwise kernel needs channels-last 8-bit operands with 16-byte aligned pixels");
    if (x.strides[3] * x.shape[3] >= (int64_t(1) << 31) || y.strides[3] * y.shape[3] >= (int64_t(1) << 31))
        CHX_FAIL(CHX_HIP_EUNSUPPORTED, "depthwise kernel: an input or output row spans 2 GiB or more");
    const bool xs = x.dtype == CHX_HIP_INT8;
    const int32_t zp_u = xs ? c.x_zp + 128 : c.x_zp;
    DepthwiseArgs a;
    memset(&a, 0, sizeof(a));
    a.x = static_cast<const char*>(x.data);
    a.x_n_stride = x.strides[0];
    a.x_h_stride = x.strides[2];
    a.x_w_stride = x.strides[3];
    a.y = static_cast<char*>(y.data);
    a.y_n_stride = y.strides[0];
    a.y_h_stride = y.strides[2];
    a.y_w_stride = y.strides[3];
    a.N = c.cs.N; a.C = c.cs.C; a.H = c.cs.H; a.W = c.cs.W; a.OH = c.cs.OH; a.OW = c.cs.OW;
    a.sh = c.p->stride_h; a.sw = c.p->stride_w; a.ph = c.p->pad_h_begin; a.pw = c.p->pad_w_begin;
    a.x_signed = xs ? 1 : 0;
    a.x_zp_u = zp_u;
    a.rows = st.rows;
    a.wsum = st.wsum;
    a.w_scale = c.w_scale;
    a.w_scale_len = c.w_scale_len;
    a.x_scale = c.rq.x_scale;
    a.bias = c.rq.bias_mode == kBiasNone ? nullptr : c.bias;
    a.float_bias = c.rq.bias_mode == kBiasReferenceFloat ? 1 : 0;
    a.q = c.rq.q;
    a.inv_y_scale = 1.0f / c.rq.q.scale;
    a.lo_folded = fold_relu_floor(c.rq.q, c.rq.relu_floor, c.rne);
    a.y_flip = c.y_minus_128 ? 0x80808080u : 0u;  // (c.y is then the uint8 view of the caller's int8 array)
    return launch_depthwise3x3(a, c.rne, s);
}

}  // namespace
}  // namespace chx

struct chx_hip_qconv_plan {
    chx_hip_tensor w, w_scale, w_zero_point, bias;
    bool has_bias;
    chx_hip_conv_params params;
    bool mfma;
    bool depthwise;
    chx::DepthwiseState dw;
    chx::PackedWeights pw;
    chx::ScratchCache scratch;  // makes run() unsafe to call concurrently on one plan
    chx::TuneCache tune;
    // the residual sums fused behind this convolution so far (run_add): each one's parameters, and whether constants
    // were found with which its two-multiply-add form is exact (find_affine_residual); kept so that the search runs
    // once per set of parameters, also for a caller that alternates between a few of them.  Oldest dropped first.
    struct SearchedResidual {
        chx::ResidualAdd key, found;
    };
    static constexpr size_t kMaxSearchedResiduals = 8;
    std::vector<SearchedResidual> searched;
    chx::LaunchOptions opt;  // read once, when the plan is created
    // recorded runs (HIP graphs) that hold addresses of this plan's packed weights and scratch memory
    int pins = 0;
    bool destroy_when_unpinned = false;
};

extern "C" int chx_hip_qlinear_conv(
        const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, const chx_hip_tensor* w,
        const chx_hip_tensor* w_scale, const chx_hip_tensor* w_zero_point, float y_scale, int32_t y_zero_point,
        const chx_hip_tensor* bias, const chx_hip_conv_params* params, uint32_t flags, chx_hip_tensor* y, void* stream) {
    QConvChecked q;
    CHX_PROPAGATE(check_qconv(x, x_scale, x_zero_point, w, w_scale, w_zero_point, y_scale, y_zero_point, bias, params,
                              flags, y, &q));
    hipStream_t s = as_stream(stream);
    const bool rne = (flags & CHX_HIP_ROUND_ONNX_RNE) != 0;
    if (weights_fit_mfma(*w, params->group)) {
        std::vector<uint8_t> zp;
        CHX_PROPAGATE(read_back(*w_zero_point, &zp, s));
        if (all_zero(zp)) {
            PackedWeights pw;
            CHX_PROPAGATE(make_packed(*w, false, s, &pw));
            const int rc = run_conv_mfma(conv_call_from(q, x, y, params, rne, read_launch_options()), pw, s);
            release_packed(&pw, false, s);
            if (rc != CHX_HIP_EUNSUPPORTED) return rc;
        }
    }
    if (weights_fit_depthwise(*w, params->group)) {
        std::vector<uint8_t> zp;
        CHX_PROPAGATE(read_back(*w_zero_point, &zp, s));
        if (all_zero(zp)) {
            DepthwiseState st;
            CHX_PROPAGATE(make_depthwise(*w, false, s, &st));
            const int rc = run_depthwise(conv_call_from(q, x, y, params, rne, read_launch_options()), st, s);
            release_depthwise(&st, false, s);
            if (rc != CHX_HIP_EUNSUPPORTED) return rc;
        }
    }
    return launch_conv_direct(q.direct, rne, s);
}

namespace chx {
namespace {

// Rank-generic convolutions (ComplementStride / ComplementPad and GroupedConv are rank-generic in the reference,
// runtime/chainerx_util.cc:180-200,313-340).  One spatial axis is a 2-D convolution over images one pixel high and
// takes every kernel the 2-D entry points have; three spatial axes run on the direct kernel, whose outermost spatial
// axis is described here beside the 4-D views (n, c, h, w) that the 2-D checks and argument blocks are made from.
struct ConvNdViews {
    chx_hip_tensor x, w, y;
    chx_hip_conv_params p;
};

chx_hip_tensor drop_axis(const chx_hip_tensor& t, int axis) {
    chx_hip_tensor r = t;
    r.ndim = t.ndim - 1;
    for (int i = axis; i < r.ndim; ++i) {
        r.shape[i] = t.shape[i + 1];
        r.strides[i] = t.strides[i + 1];
    }
    return r;
}

chx_hip_tensor insert_unit_axis(const chx_hip_tensor& t, int axis) {
    chx_hip_tensor r = t;
    r.ndim = t.ndim + 1;
    for (int i = r.ndim - 1; i > axis; --i) {
        r.shape[i] = t.shape[i - 1];
        r.strides[i] = t.strides[i - 1];
    }
    r.shape[axis] = 1;
    r.strides[axis] = t.shape[axis] * t.strides[axis];  // any value serves an axis of extent 1; this one keeps the view dense
    return r;
}

int conv_nd_views(const chx_hip_tensor* x, const chx_hip_tensor* w, const chx_hip_tensor* y, const chx_hip_conv_nd_params* p, const char* op,
                  ConvNdViews* v) {
    CHX_PROPAGATE(check_tensor(x, op));
    CHX_PROPAGATE(check_tensor(w, op));
    CHX_PROPAGATE(check_tensor(y, op));
    CHX_REQUIRE(p != nullptr, "%s: null params", op);
    CHX_REQUIRE(p->n_spatial >= 1 && p->n_spatial <= 3, "%s: %d spatial axes (1, 2 or 3 are computed)", op, p->n_spatial);
    const int nd = p->n_spatial + 2;
    CHX_REQUIRE(x->ndim == nd && w->ndim == nd && y->ndim == nd, "%s: x, w and y must have %d axes for %d spatial ones", op, nd, p->n_spatial);
    const int lead = 3 - p->n_spatial;  // entries of the 2-D parameter block that stay at their neutral values
    int32_t st[3] = {1, 1, 1}, pb[3] = {0, 0, 0}, pe[3] = {0, 0, 0};
    for (int i = 0; i < p->n_spatial; ++i) {
        st[lead + i] = p->stride[i];
        pb[lead + i] = p->pad_begin[i];
        pe[lead + i] = p->pad_end[i];
    }
    v->p.stride_h = st[1]; v->p.stride_w = st[2];
    v->p.pad_h_begin = pb[1]; v->p.pad_w_begin = pb[2];
    v->p.pad_h_end = pe[1]; v->p.pad_w_end = pe[2];
    v->p.group = p->group;
    if (p->n_spatial == 1) {
        v->x = insert_unit_axis(*x, 2);
        v->w = insert_unit_axis(*w, 2);
        v->y = insert_unit_axis(*y, 2);
    } else if (p->n_spatial == 2) {
        v->x = *x; v->w = *w; v->y = *y;
    } else {
        v->x = drop_axis(*x, 2);
        v->w = drop_axis(*w, 2);
        v->y = drop_axis(*y, 2);
    }
    return CHX_HIP_OK;
}

// the outermost spatial axis of a 3-D convolution into the argument block of the direct kernel
int add_depth_axis(const chx_hip_tensor& x, const chx_hip_tensor& w, const chx_hip_tensor& y, const chx_hip_conv_nd_params& p, const char* op,
                   ConvDirectArgs* a) {
    CHX_REQUIRE(p.stride[0] >= 1 && p.pad_begin[0] >= 0 && p.pad_end[0] >= 0, "%s: strides must be positive and pads non-negative", op);
    CHX_REQUIRE(x.shape[2] <= INT32_MAX && w.shape[2] <= INT32_MAX, "%s: extent too large", op);
    const int64_t ed = x.shape[2] + p.pad_begin[0] + p.pad_end[0] - w.shape[2];
    CHX_REQUIRE(ed >= 0, "%s: kernel deeper than the padded input", op);
    const int64_t od = ed / p.stride[0] + 1;
    CHX_REQUIRE(y.shape[2] == od, "%s: y has depth %lld, expected %lld", op, (long long)y.shape[2], (long long)od);
    a->D = (int32_t)x.shape[2];
    a->KD = (int32_t)w.shape[2];
    a->OD = (int32_t)od;
    a->sd = p.stride[0];
    a->pd = p.pad_begin[0];
    a->xsd = x.strides[2];
    a->wsd = w.strides[2];
    a->ysd = y.strides[2];
    a->total *= od;
    return CHX_HIP_OK;
}

}  // namespace
}  // namespace chx

extern "C" int chx_hip_qlinear_conv_nd(
        const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, const chx_hip_tensor* w, const chx_hip_tensor* w_scale,
        const chx_hip_tensor* w_zero_point, float y_scale, int32_t y_zero_point, const chx_hip_tensor* bias,
        const chx_hip_conv_nd_params* params, uint32_t flags, chx_hip_tensor* y, void* stream) {
    ConvNdViews v;
    CHX_PROPAGATE(conv_nd_views(x, w, y, params, "QLinearConv", &v));
    if (params->n_spatial < 3) {
        const int rc = chx_hip_qlinear_conv(&v.x, x_scale, x_zero_point, &v.w, w_scale, w_zero_point, y_scale, y_zero_point, bias, &v.p, flags, &v.y, stream);
        return rc;
    }
    QConvChecked q;
    CHX_PROPAGATE(check_qconv(&v.x, x_scale, x_zero_point, &v.w, w_scale, w_zero_point, y_scale, y_zero_point, bias, &v.p, flags, &v.y, &q));
    CHX_PROPAGATE(add_depth_axis(*x, *w, *y, *params, "QLinearConv", &q.direct));
    return launch_conv_direct(q.direct, (flags & CHX_HIP_ROUND_ONNX_RNE) != 0, as_stream(stream));
}

extern "C" int chx_hip_conv_integer_nd(
        const chx_hip_tensor* x, const chx_hip_tensor* w, int32_t x_zero_point, const chx_hip_tensor* w_zero_point,
        const chx_hip_conv_nd_params* params, chx_hip_tensor* y, void* stream) {
    ConvNdViews v;
    CHX_PROPAGATE(conv_nd_views(x, w, y, params, "ConvInteger", &v));
    if (params->n_spatial < 3) return chx_hip_conv_integer(&v.x, &v.w, x_zero_point, w_zero_point, &v.p, &v.y, stream);
    CHX_REQUIRE(y->dtype == CHX_HIP_INT32, "ConvInteger: y must be int32, got %s", dtype_name(y->dtype));
    ConvShape cs;
    CHX_PROPAGATE(conv_shape(v.x, v.w, v.p, v.y, "ConvInteger", &cs));
    ConvDirectArgs a;
    fill_conv_args(v.x, v.w, v.p, v.y, cs, &a);
    a.x_zp = x_zero_point;
    if (w_zero_point) {
        CHX_PROPAGATE(check_tensor(w_zero_point, "ConvInteger w_zero_point"));
        CHX_REQUIRE(w_zero_point->dtype == w->dtype, "ConvInteger: w_zero_point must have the dtype of w");
        int64_t len, stride;
        CHX_PROPAGATE(param_vector(*w_zero_point, cs.OC, "ConvInteger w_zero_point", &len, &stride));
        a.w_zp = static_cast<const char*>(w_zero_point->data);
        a.w_zp_len = (int32_t)len;
        a.w_zp_stride = stride;
    }
    CHX_PROPAGATE(add_depth_axis(*x, *w, *y, *params, "ConvInteger", &a));
    return launch_conv_direct(a, false, as_stream(stream));
}

extern "C" int chx_hip_qconv_plan_create(
        const chx_hip_tensor* w, const chx_hip_tensor* w_scale, const chx_hip_tensor* w_zero_point,
        const chx_hip_tensor* bias, const chx_hip_conv_params* params, void* stream, chx_hip_qconv_plan** plan) {
    CHX_REQUIRE(plan != nullptr, "QLinearConv plan: null output");
    *plan = nullptr;
    CHX_PROPAGATE(check_tensor(w, "QLinearConv w"));
    CHX_PROPAGATE(check_tensor(w_scale, "QLinearConv w_scale"));
    CHX_PROPAGATE(check_tensor(w_zero_point, "QLinearConv w_zero_point"));
    CHX_REQUIRE(params != nullptr, "QLinearConv plan: null params");
    CHX_REQUIRE(w->ndim == 4 && is_q8(w->dtype), "QLinearConv plan: w must be a 4-D uint8/int8 tensor");
    if (bias) CHX_PROPAGATE(check_tensor(bias, "QLinearConv bias"));
    hipStream_t s = as_stream(stream);
    chx_hip_qconv_plan* p = new chx_hip_qconv_plan();
    p->w = *w;
    p->w_scale = *w_scale;
    p->w_zero_point = *w_zero_point;
    p->has_bias = bias != nullptr;
    if (bias) p->bias = *bias;
    p->params = *params;
    p->mfma = false;
    p->depthwise = false;
    p->opt = chx::read_launch_options();
    if (weights_fit_depthwise(*w, params->group) && w_zero_point->dtype == w->dtype && w_zero_point->ndim <= 1) {
        std::vector<uint8_t> zp;
        int rc = read_back(*w_zero_point, &zp, s);
        if (rc == CHX_HIP_OK && all_zero(zp)) {
            rc = make_depthwise(*w, true, s, &p->dw);
            if (rc == CHX_HIP_OK && hipStreamSynchronize(s) != hipSuccess) rc = CHX_HIP_ERUNTIME;
            if (rc == CHX_HIP_OK) p->depthwise = true;
        }
        if (rc != CHX_HIP_OK) {
            release_depthwise(&p->dw, true, s);
            delete p;
            return rc;
        }
    }
    if (weights_fit_mfma(*w, params->group) && w_zero_point->dtype == w->dtype && w_zero_point->ndim <= 1) {
        std::vector<uint8_t> zp;
        int rc = read_back(*w_zero_point, &zp, s);
        if (rc == CHX_HIP_OK && all_zero(zp)) {
            rc = make_packed(*w, true, s, &p->pw);
            if (rc == CHX_HIP_OK) {
                hipError_t e = hipStreamSynchronize(s);
                if (e != hipSuccess) {
                    set_error("hipStreamSynchronize failed: %s", hipGetErrorString(e));
                    rc = CHX_HIP_ERUNTIME;
                }
            }
            if (rc == CHX_HIP_OK) p->mfma = true;
        }
        if (rc != CHX_HIP_OK) {
            release_packed(&p->pw, true, s);
            delete p;
            return rc;
        }
    }
    *plan = p;
    return CHX_HIP_OK;
}

namespace chx {
namespace {
// CHX_HIP_STORE_MINUS_128: the array is int8, its quantization is that of the uint8 array it stands for.  *view is what
// the checks and the requantization parameters are derived from.
int result_view(const chx_hip_tensor* y, uint32_t flags, const char* op, chx_hip_tensor* view, bool* minus_128) {
    CHX_PROPAGATE(check_tensor(y, op));
    *view = *y;
    *minus_128 = (flags & CHX_HIP_STORE_MINUS_128) != 0;
    if (*minus_128) {
        CHX_REQUIRE(y->dtype == CHX_HIP_INT8, "%s: codes minus 128 are stored into an int8 array, got %s", op, dtype_name(y->dtype));
        view->dtype = CHX_HIP_UINT8;
    }
    return CHX_HIP_OK;
}
}  // namespace
}  // namespace chx

extern "C" int chx_hip_qconv_plan_run(
        const chx_hip_qconv_plan* plan, const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, float y_scale,
        int32_t y_zero_point, uint32_t flags, chx_hip_tensor* y, void* stream) {
    CHX_REQUIRE(plan != nullptr, "QLinearConv plan: null plan");
    chx_hip_tensor yv;
    bool minus_128 = false;
    CHX_PROPAGATE(result_view(y, flags, "QLinearConv y", &yv, &minus_128));
    QConvChecked q;
    CHX_PROPAGATE(check_qconv(x, x_scale, x_zero_point, &plan->w, &plan->w_scale, &plan->w_zero_point, y_scale,
                              y_zero_point, plan->has_bias ? &plan->bias : nullptr, &plan->params, flags, &yv, &q));
    hipStream_t s = as_stream(stream);
    const bool rne = (flags & CHX_HIP_ROUND_ONNX_RNE) != 0;
    if (plan->mfma) {
        ConvCall call = conv_call_from(q, x, &yv, &plan->params, rne, plan->opt);
        call.cache = const_cast<ScratchCache*>(&plan->scratch);
        call.tune = const_cast<TuneCache*>(&plan->tune);
        call.y_minus_128 = minus_128;
        const int rc = run_conv_mfma(call, plan->pw, s);
        if (rc != CHX_HIP_EUNSUPPORTED || minus_128) return rc;
    }
    if (plan->depthwise) {
        ConvCall call = conv_call_from(q, x, &yv, &plan->params, rne, plan->opt);
        call.y_minus_128 = minus_128;
        const int rc = run_depthwise(call, plan->dw, s);
        if (rc != CHX_HIP_EUNSUPPORTED || minus_128) return rc;
    }
    if (minus_128) CHX_FAIL(CHX_HIP_EUNSUPPORTED, "QLinearConv: codes minus 128 are stored by the matrix-core and the depthwise kernel only");
    return launch_conv_direct(q.direct, rne, s);
}

extern "C" int chx_hip_qconv_plan_run_pair(
        const chx_hip_qconv_plan* plan, const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, int32_t split,
        float y1_scale, int32_t y1_zero_point, uint32_t flags1, chx_hip_tensor* y1, float y2_scale, int32_t y2_zero_point,
        uint32_t flags2, chx_hip_tensor* y2, void* stream) {
    CHX_REQUIRE(plan != nullptr, "QLinearConv pair: null plan");
    chx_hip_tensor y1v, y2v;
    bool y1_minus_128 = false, y2_minus_128 = false;
    CHX_PROPAGATE(result_view(y1, flags1, "QLinearConv pair y1", &y1v, &y1_minus_128));
    CHX_PROPAGATE(result_view(y2, flags2, "QLinearConv pair y2", &y2v, &y2_minus_128));
    CHX_REQUIRE(y1->ndim == 4 && y2->ndim == 4, "QLinearConv pair: y1 and y2 must be 4-D");
    const int64_t OC = plan->w.shape[0];
    CHX_REQUIRE(split > 0 && split < OC && y1->shape[1] == split && y2->shape[1] == OC - split,
                "QLinearConv pair: y1 and y2 must hold the first %d and the other %lld of the plan's %lld output channels", split,
                (long long)(OC - split), (long long)OC);
    for (int ax : {0, 2, 3}) CHX_REQUIRE(y1->shape[ax] == y2->shape[ax], "QLinearConv pair: y1 and y2 differ in batch or image size");
    const uint32_t shared = CHX_HIP_BIAS_ONNX_INT32 | CHX_HIP_ROUND_ONNX_RNE;
    CHX_REQUIRE((flags1 & shared) == (flags2 & shared), "QLinearConv pair: the two halves must agree on the bias and rounding flags");
    CHX_PROPAGATE(check_tensor(x, "QLinearConv pair x"));
    CHX_REQUIRE(!byte_ranges_overlap(*y1, *x) && !byte_ranges_overlap(*y2, *x) && !byte_ranges_overlap(*y1, *y2),
                "QLinearConv pair: x, y1 and y2 must not overlap in memory");
    if (split % 64 != 0) CHX_FAIL(CHX_HIP_EUNSUPPORTED, "QLinearConv pair: the first convolution must have a multiple of 64 output channels");
    if (!plan->mfma) CHX_FAIL(CHX_HIP_EUNSUPPORTED, "QLinearConv pair: these weights do not run on the matrix-core kernel");
    // shapes and parameters as for one convolution with all output channels, laid out like y1
    chx_hip_tensor y_all = y1v;
    y_all.shape[1] = OC;
    QConvChecked q;
    CHX_PROPAGATE(check_qconv(x, x_scale, x_zero_point, &plan->w, &plan->w_scale, &plan->w_zero_point, y1_scale, y1_zero_point,
                              plan->has_bias ? &plan->bias : nullptr, &plan->params, flags1, &y_all, &q));
    RequantParams rq2;
    const int32_t* bias2 = nullptr;
    CHX_PROPAGATE(fill_requant(x_scale, y2_scale, y2_zero_point, y2v, plan->has_bias ? &plan->bias : nullptr, OC, flags2,
                               "QLinearConv pair", &rq2, &bias2));
    hipStream_t s = as_stream(stream);
    ConvCall call = conv_call_from(q, x, &y1v, &plan->params, (flags1 & CHX_HIP_ROUND_ONNX_RNE) != 0, plan->opt);
    call.cache = const_cast<ScratchCache*>(&plan->scratch);
    call.tune = const_cast<TuneCache*>(&plan->tune);
    call.y2 = &y2v;
    call.y_minus_128 = y1_minus_128;
    call.y2_minus_128 = y2_minus_128;
    call.oc_split = split;
    call.rq2 = rq2;
    return run_conv_mfma(call, plan->pw, s);
}

extern "C" int chx_hip_qconv_plan_run_add(
        const chx_hip_qconv_plan* plan, const chx_hip_tensor* x, float x_scale, int32_t x_zero_point, float y_scale,
        int32_t y_zero_point, int32_t y_dtype, uint32_t flags, const chx_hip_tensor* r, float r_scale, int32_t r_zero_point,
        float out_scale, int32_t out_zero_point, int32_t relu, chx_hip_tensor* out, void* stream) {
    CHX_REQUIRE(plan != nullptr, "QLinearConv+Add: null plan");
    CHX_PROPAGATE(check_tensor(r, "QLinearConv+Add r"));
    // (with CHX_HIP_STORE_MINUS_128 `out` is an int8 array that holds the codes of a uint8 sum minus 128)
    chx_hip_tensor outv;
    bool out_minus_128 = false;
    CHX_PROPAGATE(result_view(out, flags, "QLinearConv+Add out", &outv, &out_minus_128));
    const int32_t out_dtype = outv.dtype;
    CHX_REQUIRE(is_q8(y_dtype) && is_q8(r->dtype) && is_q8(out_dtype), "QLinearConv+Add: y, r and out must be uint8 or int8");
    CHX_REQUIRE(r->ndim == 4 && out->ndim == 4, "QLinearConv+Add: r and out must be 4-D");
    for (int i = 0; i < 4; ++i)
        CHX_REQUIRE(r->shape[i] == out->shape[i], "QLinearConv+Add: r and out differ in shape (no broadcasting)");
    auto in_range = [](int32_t zp, int32_t dt) { return dt == CHX_HIP_INT8 ? zp >= -128 && zp <= 127 : zp >= 0 && zp <= 255; };
    CHX_REQUIRE(in_range(r_zero_point, r->dtype) && in_range(out_zero_point, out_dtype),
                "QLinearConv+Add: zero point out of the range of its type");
    if (!(out_scale >= 0x1p-60f && out_scale <= 0x1p60f))
        CHX_FAIL(CHX_HIP_EUNSUPPORTED, "QLinearConv+Add: out_scale outside [2^-60, 2^60]");
    // `out` is written while x and r are still being read (and, when the launch configurations are timed,
    // several times over)
    CHX_PROPAGATE(check_tensor(x, "QLinearConv+Add x"));
    CHX_REQUIRE(!byte_ranges_overlap(*out, *x) && !byte_ranges_overlap(*out, *r), "QLinearConv+Add: out overlaps x or r in memory");
    // the convolution's own result has the layout of `out` and the type y_dtype
    chx_hip_tensor y = *out;
    y.dtype = y_dtype;
    QConvChecked q;
    CHX_PROPAGATE(check_qconv(x, x_scale, x_zero_point, &plan->w, &plan->w_scale, &plan->w_zero_point, y_scale,
                              y_zero_point, plan->has_bias ? &plan->bias : nullptr, &plan->params, flags, &y, &q));
    if (!plan->mfma) CHX_FAIL(CHX_HIP_EUNSUPPORTED, "QLinearConv+Add: these weights do not run on the matrix-core kernel");
    int64_t r_px = 0, o_px = 0;
    if (!y_is_pixel_major(*r, &r_px) || !y_is_pixel_major(*out, &o_px))
        CHX_FAIL(CHX_HIP_EUNSUPPORTED, "QLinearConv+Add: r and out must be channels-last");
    ResidualAdd res;
    memset(&res, 0, sizeof(res));
    res.r = static_cast<const char*>(r->data);
    res.r_px_stride = r_px;
    res.r_vec_ok = aligned(r->data, 16) && r_px % 16 == 0 ? 1 : 0;
    res.c_flip = y_dtype == CHX_HIP_INT8 ? 0x80808080u : 0u;
    res.r_flip = r->dtype == CHX_HIP_INT8 ? 0x80808080u : 0u;
    res.c_zpf = (float)(y_zero_point + (y_dtype == CHX_HIP_INT8 ? 128 : 0));
    res.c_scale = y_scale;
    res.r_zpf = (float)(r_zero_point + (r->dtype == CHX_HIP_INT8 ? 128 : 0));
    res.r_scale = r_scale;
    res.relu = relu ? 1 : 0;
    res.out = make_quant_params(out_scale, out_zero_point, out_dtype == CHX_HIP_INT8);
    res.inv_out_scale = 1.0f / out_scale;
    res.big = 0x1p40f * out_scale;
    // |DQ(y) + DQ(r)| <= 511 * (|y_scale| + |r_scale|): when that is far below `big`, limiting is the identity
    const double reach = 511.0 * (fabs((double)y_scale) + fabs((double)r_scale));
    res.guard = (reach == reach && reach < 0.25 * (double)res.big) ? 0 : 1;
    // (r's zero point in the unsigned range: a uint8 r with zero point 0, or the same codes stored minus 128 as int8)
    res.lean = out_dtype == CHX_HIP_UINT8 && res.r_zpf == 0.f && out_zero_point == 0 ? 1 : 0;
    hipStream_t s = as_stream(stream);
    // The cheaper form of the sum, where the search over its constants has shown it exact for these parameters.  The
    // search runs on the first call with new parameters (it synchronizes the stream and allocates, so not while the
    // stream is being captured: such a call computes the sum operation by operation).  CHX_HIP_AFFINE_RESIDUAL=0
    // keeps the operation-by-operation arithmetic everywhere.
    {
        chx_hip_qconv_plan* mp = const_cast<chx_hip_qconv_plan*>(plan);
        ResidualAdd key;
        memcpy(&key, &res, sizeof(key));  // byte copies: the comparison below is one of bytes, padding included
        key.r = nullptr;
        key.r_px_stride = 0;
        key.r_vec_ok = 0;
        const bool wanted = plan->opt.affine_residual;
        const ResidualAdd* known = nullptr;
        for (const chx_hip_qconv_plan::SearchedResidual& e : mp->searched)
            if (memcmp(&key, &e.key, sizeof(key)) == 0) known = &e.found;
        if (wanted && known) {
            res.affine = known->affine;
            res.kc = known->kc;
            res.kr = known->kr;
            res.k0 = known->k0;
            res.floor_pre = known->floor_pre;
        } else if (wanted && !stream_is_capturing(s)) {
            int32_t* counts = nullptr;
            CHX_HIP_CALL(hipMalloc(reinterpret_cast<void**>(&counts), kAffineCandidates * sizeof(int32_t)));
            ResidualAdd found;
            memcpy(&found, &key, sizeof(found));
            const int rc = find_affine_residual(&found, counts, s);
            (void)hipFree(counts);
            CHX_PROPAGATE(rc);
            if (mp->searched.size() == chx_hip_qconv_plan::kMaxSearchedResiduals) mp->searched.erase(mp->searched.begin());
            mp->searched.emplace_back();
            memcpy(&mp->searched.back().key, &key, sizeof(key));
            memcpy(&mp->searched.back().found, &found, sizeof(found));
            res.affine = found.affine;
            res.kc = found.kc;
            res.kr = found.kr;
            res.k0 = found.k0;
            res.floor_pre = found.floor_pre;
        }
    }
    ConvCall call = conv_call_from(q, x, &y, &plan->params, (flags & CHX_HIP_ROUND_ONNX_RNE) != 0, plan->opt);
    call.cache = const_cast<ScratchCache*>(&plan->scratch);
    call.tune = const_cast<TuneCache*>(&plan->tune);
    call.res = &res;
    call.y_minus_128 = out_minus_128;
    return run_conv_mfma(call, plan->pw, s);
}

extern "C" int chx_hip_qconv_plan_describe(const chx_hip_qconv_plan* plan, char* buf, size_t buf_size) {
    CHX_REQUIRE(plan != nullptr && buf != nullptr && buf_size > 0, "QLinearConv plan: null argument");
    std::string text;
    for (const TunedConfig& t : plan->tune.entries) {
        char line[160];
        snprintf(line, sizeof(line), "M=%lld %dx%d res=%d tile=%dx%d wgs_per_cu=%d waves=%d\n", (long long)t.M, t.OH, t.OW, t.with_res ? 1 : 0,
                 t.tile_oc, t.tile_px, t.max_wgs_per_cu, t.waves);
        text += line;
    }
    if (!plan->searched.empty()) text += plan->searched.back().found.affine ? "residual=affine\n" : "residual=exact\n";
    strncpy(buf, text.c_str(), buf_size - 1);
    buf[buf_size - 1] = 0;
    return CHX_HIP_OK;
}

extern "C" int chx_hip_qconv_plan_pin(chx_hip_qconv_plan* plan, int32_t delta) {
    CHX_REQUIRE(plan != nullptr && (delta == 1 || delta == -1), "QLinearConv plan pin: a plan and +1 or -1");
    CHX_REQUIRE(plan->pins + delta >= 0, "QLinearConv plan pin: released more often than pinned");
    plan->pins += delta;
    plan->scratch.pinned = plan->pins > 0;
    if (plan->pins == 0 && plan->destroy_when_unpinned) {
        plan->destroy_when_unpinned = false;
        chx_hip_qconv_plan_destroy(plan);
    }
    return CHX_HIP_OK;
}

extern "C" void chx_hip_qconv_plan_destroy(chx_hip_qconv_plan* plan) {
    if (!plan) return;
    if (plan->pins > 0) {
        // a recorded run still launches kernels on this plan's memory: it goes when the last pin does
        plan->destroy_when_unpinned = true;
        return;
    }
    chx::release_packed(&plan->pw, true, nullptr);
    chx::release_depthwise(&plan->dw, true, nullptr);
    for (int i = 0; i < 2; ++i)
        if (plan->scratch.ptr[i]) (void)hipFree(plan->scratch.ptr[i]);
    delete plan;
}

extern "C" int chx_hip_conv_integer(
        const chx_hip_tensor* x, const chx_hip_tensor* w, int32_t x_zero_point, const chx_hip_tensor* w_zero_point,
        const chx_hip_conv_params* params, chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(x, "ConvInteger x"));
    CHX_PROPAGATE(check_tensor(w, "ConvInteger w"));
    CHX_PROPAGATE(check_tensor(y, "ConvInteger y"));
    CHX_REQUIRE(params != nullptr, "ConvInteger: null params");
    CHX_REQUIRE(y->dtype == CHX_HIP_INT32, "ConvInteger: y must be int32, got %s", dtype_name(y->dtype));
    ConvShape cs;
    CHX_PROPAGATE(conv_shape(*x, *w, *params, *y, "ConvInteger", &cs));
    ConvDirectArgs a;
    fill_conv_args(*x, *w, *params, *y, cs, &a);
    a.x_zp = x_zero_point;
    if (w_zero_point) {
        CHX_PROPAGATE(check_tensor(w_zero_point, "ConvInteger w_zero_point"));
        CHX_REQUIRE(w_zero_point->dtype == w->dtype, "ConvInteger: w_zero_point must have the dtype of w");
        int64_t len, stride;
        CHX_PROPAGATE(param_vector(*w_zero_point, cs.OC, "ConvInteger w_zero_point", &len, &stride));
        a.w_zp = static_cast<const char*>(w_zero_point->data);
        a.w_zp_len = (int32_t)len;
        a.w_zp_stride = stride;
    }
    hipStream_t s = as_stream(stream);
    // (a recorded run takes the kernel without scratch memory: the weights of this entry point are packed per call)
    if (weights_fit_mfma(*w, params->group) && !stream_is_capturing(s)) {
        bool zero = true;
        if (w_zero_point) {
            std::vector<uint8_t> zp;
            CHX_PROPAGATE(read_back(*w_zero_point, &zp, s));
            zero = all_zero(zp);
        }
        if (zero) {
            ConvCall c;
            memset(&c, 0, sizeof(c));
            c.opt = read_launch_options();
            c.x = x;
            c.y = y;
            c.p = params;
            c.cs = cs;
            c.x_zp = x_zero_point;
            c.out_int32 = true;
            PackedWeights pw;
            CHX_PROPAGATE(make_packed(*w, false, s, &pw));
            const int rc = run_conv_mfma(c, pw, s);
            release_packed(&pw, false, s);
            if (rc != CHX_HIP_EUNSUPPORTED) return rc;
        }
    }
    return launch_conv_direct(a, false, s);
}

namespace chx {
namespace {

// A 2-D matrix product as a 1x1 convolution over M "pixels": a [M,K] is a channels-last
// activation row per pixel, b [K,N] the weights of N output channels.
int matmul_via_mfma(
        const chx_hip_tensor& a, const chx_hip_tensor& b, chx_hip_tensor& y, const MatMulShape& ms, int32_t a_zp,
        bool out_int32, bool rne, float b_scale, const int32_t* bias, const RequantParams& rq, hipStream_t s) {
    const int nd = a.ndim;
    if (ms.batch != 1 || b.dtype != CHX_HIP_INT8 || ms.M > INT32_MAX || ms.K > (1 << 20) || ms.N >= (1 << 24))
        return CHX_HIP_EUNSUPPORTED;
    if (stream_is_capturing(s)) return CHX_HIP_EUNSUPPORTED;  // b is packed into scratch memory per call: not inside a recorded run
    chx_hip_tensor x4, w4, y4;
    memset(&x4, 0, sizeof(x4));
    memset(&w4, 0, sizeof(w4));
    memset(&y4, 0, sizeof(y4));
    x4.data = a.data; x4.dtype = a.dtype; x4.ndim = 4;
    x4.shape[0] = 1; x4.shape[1] = ms.K; x4.shape[2] = 1; x4.shape[3] = ms.M;
    x4.strides[0] = 0; x4.strides[1] = a.strides[nd - 1]; x4.strides[2] = 0; x4.strides[3] = a.strides[nd - 2];
    w4.data = b.data; w4.dtype = b.dtype; w4.ndim = 4;
    w4.shape[0] = ms.N; w4.shape[1] = ms.K; w4.shape[2] = 1; w4.shape[3] = 1;
    w4.strides[0] = b.strides[nd - 1]; w4.strides[1] = b.strides[nd - 2]; w4.strides[2] = 0; w4.strides[3] = 0;
    y4.data = y.data; y4.dtype = y.dtype; y4.ndim = 4;
    y4.shape[0] = 1; y4.shape[1] = ms.N; y4.shape[2] = 1; y4.shape[3] = ms.M;
    y4.strides[0] = 0; y4.strides[1] = y.strides[nd - 1]; y4.strides[2] = 0; y4.strides[3] = y.strides[nd - 2];
    if (!weights_fit_mfma(w4, 1) || !x_is_mfma_ready(x4)) return CHX_HIP_EUNSUPPORTED;
    int64_t px;
    if (!y_is_pixel_major(y4, &px)) return CHX_HIP_EUNSUPPORTED;
    chx_hip_conv_params p = {1, 1, 0, 0, 0, 0, 1};
    ConvCall c;
    memset(&c, 0, sizeof(c));
    c.opt = read_launch_options();
    c.x = &x4;
    c.y = &y4;
    c.p = &p;
    c.cs.N = 1; c.cs.C = (int32_t)ms.K; c.cs.H = 1; c.cs.W = (int32_t)ms.M;
    c.cs.OC = (int32_t)ms.N; c.cs.Cg = (int32_t)ms.K; c.cs.KH = 1; c.cs.KW = 1; c.cs.OH = 1; c.cs.OW = (int32_t)ms.M;
    c.x_zp = a_zp;
    c.out_int32 = out_int32;
    c.rne = rne;
    static const float kOne = 0.f;
    (void)kOne;
    c.w_scale = nullptr;
    c.w_scale_len = 1;
    c.bias = bias;
    c.rq = rq;
    PackedWeights pw;
    CHX_PROPAGATE(make_packed(w4, false, s, &pw));
    // the per-tensor b_scale is a host value; the kernel reads scales from device memory
    void* scale_dev = nullptr;
    int rc = CHX_HIP_OK;
    if (!out_int32) {
        rc = scratch_alloc(&scale_dev, sizeof(float), s);
        if (rc == CHX_HIP_OK && hipMemcpyAsync(scale_dev, &b_scale, sizeof(float), hipMemcpyHostToDevice, s) != hipSuccess) {
            set_error("hipMemcpyAsync of the weight scale failed");
            rc = CHX_HIP_ERUNTIME;
        }
        c.w_scale = static_cast<const float*>(scale_dev);
    }
    if (rc == CHX_HIP_OK) rc = run_conv_mfma(c, pw, s);
    scratch_free(scale_dev, s);
    release_packed(&pw, false, s);
    return rc;
}

// Scalar zero point held in a device array of one element (or absent): host value, via a
// synchronizing read.  Returns false when the array is a per-axis vector.
int scalar_zero_point(const chx_hip_tensor* zp, hipStream_t s, bool* is_scalar, int32_t* value) {
    *is_scalar = true;
    *value = 0;
    if (!zp) return CHX_HIP_OK;
    if (numel(*zp) != 1) {
        *is_scalar = false;
        return CHX_HIP_OK;
    }
    std::vector<uint8_t> v;
    CHX_PROPAGATE(read_back(*zp, &v, s));
    *value = zp->dtype == CHX_HIP_INT8 ? (int32_t)(int8_t)v[0] : (int32_t)v[0];
    return CHX_HIP_OK;
}

}  // namespace
}  // namespace chx

extern "C" int chx_hip_matmul_integer(
        const chx_hip_tensor* a, const chx_hip_tensor* b, const chx_hip_tensor* a_zero_point,
        const chx_hip_tensor* b_zero_point, chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(a, "MatMulInteger a"));
    CHX_PROPAGATE(check_tensor(b, "MatMulInteger b"));
    CHX_PROPAGATE(check_tensor(y, "MatMulInteger y"));
    CHX_REQUIRE(is_q8(a->dtype) && is_q8(b->dtype), "MatMulInteger: a and b must be uint8 or int8");
    CHX_REQUIRE(y->dtype == CHX_HIP_INT32, "MatMulInteger: y must be int32, got %s", dtype_name(y->dtype));
    MatMulShape ms;
    CHX_PROPAGATE(matmul_shape(*a, *b, *y, "MatMulInteger", &ms));
    MatMulDirectArgs m;
    fill_matmul_args(*a, *b, *y, ms, &m);
    if (a_zero_point) {
        CHX_PROPAGATE(check_tensor(a_zero_point, "MatMulInteger a_zero_point"));
        CHX_REQUIRE(is_q8(a_zero_point->dtype), "MatMulInteger: a_zero_point must be uint8 or int8");
        int64_t len, stride;
        CHX_PROPAGATE(param_vector(*a_zero_point, ms.K, "MatMulInteger a_zero_point", &len, &stride));  // CHECK_GE(1, ndim)
        m.a_zp = static_cast<const char*>(a_zero_point->data);
        m.a_zp_len = (int32_t)len;
        m.a_zp_stride = stride;
        m.a_zp_signed = a_zero_point->dtype == CHX_HIP_INT8;
    }
    if (b_zero_point) {
        CHX_PROPAGATE(check_tensor(b_zero_point, "MatMulInteger b_zero_point"));
        CHX_REQUIRE(is_q8(b_zero_point->dtype), "MatMulInteger: b_zero_point must be uint8 or int8");
        int64_t len, stride;
        CHX_PROPAGATE(param_vector(*b_zero_point, ms.N, "MatMulInteger b_zero_point", &len, &stride));
        m.b_zp = static_cast<const char*>(b_zero_point->data);
        m.b_zp_len = (int32_t)len;
        m.b_zp_stride = stride;
        m.b_zp_signed = b_zero_point->dtype == CHX_HIP_INT8;
    }
    hipStream_t s = as_stream(stream);
    if (ms.batch == 1 && b->dtype == CHX_HIP_INT8 && ms.M * ms.N * ms.K >= (int64_t(1) << 22) && !stream_is_capturing(s)) {
        bool a_scalar, b_scalar;
        int32_t az, bz;
        CHX_PROPAGATE(scalar_zero_point(a_zero_point, s, &a_scalar, &az));
        CHX_PROPAGATE(scalar_zero_point(b_zero_point, s, &b_scalar, &bz));
        if (a_scalar && b_scalar && bz == 0) {
            RequantParams rq;
            memset(&rq, 0, sizeof(rq));
            const int rc = matmul_via_mfma(*a, *b, *y, ms, az, true, false, 0.f, nullptr, rq, s);
            if (rc != CHX_HIP_EUNSUPPORTED) return rc;
        }
    }
    return launch_matmul_direct(m, false, s);
}

extern "C" int chx_hip_qlinear_matmul(
        const chx_hip_tensor* a, float a_scale, int32_t a_zero_point, const chx_hip_tensor* b, float b_scale,
        int32_t b_zero_point, float y_scale, int32_t y_zero_point, const chx_hip_tensor* bias, uint32_t flags,
        chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_tensor(a, "QLinearMatMul a"));
    CHX_PROPAGATE(check_tensor(b, "QLinearMatMul b"));
    CHX_PROPAGATE(check_tensor(y, "QLinearMatMul y"));
    CHX_REQUIRE(is_q8(a->dtype) && is_q8(b->dtype), "QLinearMatMul: a and b must be uint8 or int8");
    MatMulShape ms;
    CHX_PROPAGATE(matmul_shape(*a, *b, *y, "QLinearMatMul", &ms));
    MatMulDirectArgs m;
    fill_matmul_args(*a, *b, *y, ms, &m);
    m.a_zp_imm = a_zero_point;
    m.b_zp_imm = b_zero_point;
    m.requant = 1;
    m.b_scale = b_scale;
    // the extension's bias is always the ONNX kind: int32, added to the accumulator
    CHX_PROPAGATE(fill_requant(a_scale, y_scale, y_zero_point, *y, bias, ms.N, flags | CHX_HIP_BIAS_ONNX_INT32,
                               "QLinearMatMul", &m.rq, &m.bias));
    hipStream_t s = as_stream(stream);
    const bool rne = (flags & CHX_HIP_ROUND_ONNX_RNE) != 0;
    if (b_zero_point == 0) {
        const int rc = matmul_via_mfma(*a, *b, *y, ms, a_zero_point, false, rne, b_scale, m.bias, m.rq, s);
        if (rc != CHX_HIP_EUNSUPPORTED) return rc;
    }
    return launch_matmul_direct(m, rne, s);
}

