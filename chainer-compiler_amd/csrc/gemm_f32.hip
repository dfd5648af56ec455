// float32 matrix product with the epilogue of GemmOp::RunImpl (runtime/ops/math.cc:160-177) and
// LinearOp::RunImpl (runtime/ops/connection.cc:12-15): the float layers that stay around a
// quantized network (a classifier head that was not quantized, the float model being calibrated).
//
//   r[m, n] = sum_k A[m, k] * B[k, n]      float32, k ascending from an accumulator of 0, one rounding
//                                           per multiplication and one per addition (no fused multiply-add)
//   r = r * alpha                           only when alpha != 1
//   y = r + (beta != 1 ? c * beta : c)      only when c is given and beta != 0; c broadcasts over [M, N]
//
// The order of the sum is what fixes the bits of a float product.  ChainerX's Dot is not in the tree, so
// the order here is the plain one of the CPU restatement this kernel is tested against bit for bit.
//
// One work-group computes a 64 x 64 tile with 256 threads (4 x 4 outputs each) from 64 x 16 and 16 x 64
// operand tiles staged in LDS; operands are read through their strides, so transposed operands cost
// nothing extra and are not copied.
#include "chx_internal.h"

namespace chx {
namespace {

struct GemmArgs {
    const char* a;
    const char* b;
    const char* c;
    char* y;
    int64_t a_sm, a_sk, b_sk, b_sn, c_sm, c_sn, y_sm, y_sn;  // byte strides
    int32_t M, N, K;
    float alpha, beta;
    int32_t has_c;
};

constexpr int kTile = 64, kStep = 16;

__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmArgs g) {
    __shared__ float As[kStep][kTile + 4];  // [k][m]
    __shared__ float Bs[kStep][kTile + 4];  // [k][n]
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * kTile, n0 = blockIdx.x * kTile;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < g.K; k0 += kStep) {
        // 64 x 16 elements of each operand, four per thread; whichever of (row, k) is contiguous in
        // memory runs along consecutive lanes
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int idx = tid + e * 256;
            int r, k;
            if (g.a_sk == 4) { k = idx & 15; r = idx >> 4; } else { r = idx & 63; k = idx >> 6; }
            float v = 0.f;
            if (m0 + r < g.M && k0 + k < g.K) v = *reinterpret_cast<const float*>(g.a + (int64_t)(m0 + r) * g.a_sm + (int64_t)(k0 + k) * g.a_sk);
            As[k][r] = v;
            if (g.b_sk == 4) { k = idx & 15; r = idx >> 4; } else { r = idx & 63; k = idx >> 6; }
            v = 0.f;
            if (n0 + r < g.N && k0 + k < g.K) v = *reinterpret_cast<const float*>(g.b + (int64_t)(k0 + k) * g.b_sk + (int64_t)(n0 + r) * g.b_sn);
            Bs[k][r] = v;
        }
        __syncthreads();
        const int kn = min(kStep, g.K - k0);  // the terms past K are not added at all (0 * inf would be NaN)
        for (int k = 0; k < kn; ++k) {
            float av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = As[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) bv[j] = Bs[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float p = av[i] * bv[j];
                    acc[i][j] = acc[i][j] + p;
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= g.M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= g.N) continue;
            float r = acc[i][j];
            if (g.alpha != 1.f) r = r * g.alpha;
            if (g.has_c) {
                float xc = *reinterpret_cast<const float*>(g.c + (int64_t)m * g.c_sm + (int64_t)n * g.c_sn);
                if (g.beta != 1.f) xc = xc * g.beta;
                r = r + xc;
            }
            *reinterpret_cast<float*>(g.y + (int64_t)m * g.y_sm + (int64_t)n * g.y_sn) = r;
        }
    }
}

int run_gemm(const chx_hip_tensor& a, bool trans_a, const chx_hip_tensor& b, bool trans_b, const chx_hip_tensor* c, float alpha,
             float beta, chx_hip_tensor& y, const char* op, hipStream_t s) {
    GemmArgs g;
    const int64_t M = a.shape[trans_a ? 1 : 0], K = a.shape[trans_a ? 0 : 1];
    const int64_t Kb = b.shape[trans_b ? 1 : 0], N = b.shape[trans_b ? 0 : 1];
    CHX_REQUIRE(K == Kb, "%s: the inner extents differ (%lld and %lld)", op, (long long)K, (long long)Kb);
    CHX_REQUIRE(y.ndim == 2 && y.shape[0] == M && y.shape[1] == N, "%s: y must be [%lld, %lld]", op, (long long)M, (long long)N);
    CHX_REQUIRE(M < (int64_t(1) << 31) && N < (int64_t(1) << 31) && K < (int64_t(1) << 31), "%s: an extent of 2^31 or more", op);
    g.a = static_cast<const char*>(a.data);
    g.b = static_cast<const char*>(b.data);
    g.y = static_cast<char*>(y.data);
    g.a_sm = a.strides[trans_a ? 1 : 0];
    g.a_sk = a.strides[trans_a ? 0 : 1];
    g.b_sk = b.strides[trans_b ? 1 : 0];
    g.b_sn = b.strides[trans_b ? 0 : 1];
    g.y_sm = y.strides[0];
    g.y_sn = y.strides[1];
    g.M = (int32_t)M;
    g.N = (int32_t)N;
    g.K = (int32_t)K;
    g.alpha = alpha;
    g.beta = beta;
    g.has_c = 0;
    g.c = nullptr;
    g.c_sm = g.c_sn = 0;
    if (c != nullptr && beta != 0.f) {
        // numpy broadcasting of c against [M, N]: extents are aligned from the right, an extent of 1 repeats
        CHX_REQUIRE(c->ndim <= 2, "%s: c has more than two axes", op);
        const int64_t cm = c->ndim == 2 ? c->shape[0] : 1, cn = c->ndim >= 1 ? c->shape[c->ndim - 1] : 1;
        CHX_REQUIRE((cm == 1 || cm == M) && (cn == 1 || cn == N), "%s: c does not broadcast to [%lld, %lld]", op, (long long)M, (long long)N);
        g.has_c = 1;
        g.c = static_cast<const char*>(c->data);
        g.c_sm = (c->ndim == 2 && cm != 1) ? c->strides[0] : 0;
        g.c_sn = (c->ndim >= 1 && cn != 1) ? c->strides[c->ndim - 1] : 0;
    }
    if (M == 0 || N == 0) return CHX_HIP_OK;
    const dim3 grid((unsigned)((N + kTile - 1) / kTile), (unsigned)((M + kTile - 1) / kTile));
    CHX_REQUIRE(grid.y <= 65535, "%s: more than 65535 row tiles", op);
    gemm_f32_kernel<<<grid, 256, 0, s>>>(g);
    return launch_check("gemm_f32_kernel");
}

int check_f32_matrix(const chx_hip_tensor* t, const char* op, const char* name) {
    CHX_REQUIRE(t != nullptr, "%s: %s is null", op, name);
    std::string what = std::string(op) + " " + name;
    CHX_PROPAGATE(check_tensor(t, what.c_str()));
    CHX_REQUIRE(t->dtype == CHX_HIP_FLOAT32, "%s: %s must be float32, not %s", op, name, dtype_name(t->dtype));
    return CHX_HIP_OK;
}

}  // namespace
}  // namespace chx

using namespace chx;

extern "C" int chx_hip_gemm_f32(
        const chx_hip_tensor* a, const chx_hip_tensor* b, const chx_hip_tensor* c, float alpha, float beta, int32_t trans_a,
        int32_t trans_b, chx_hip_tensor* y, void* stream) {
    CHX_PROPAGATE(check_f32_matrix(a, "Gemm", "a"));
    CHX_PROPAGATE(check_f32_matrix(b, "Gemm", "b"));
    CHX_PROPAGATE(check_f32_matrix(y, "Gemm", "y"));
    if (c != nullptr) CHX_PROPAGATE(check_f32_matrix(c, "Gemm", "c"));
    CHX_REQUIRE(a->ndim == 2 && b->ndim == 2, "Gemm: a and b must be matrices");
    return run_gemm(*a, trans_a != 0, *b, trans_b != 0, c, alpha, beta, *y, "Gemm", as_stream(stream));
}

extern "C" int chx_hip_linear_f32(
        const chx_hip_tensor* x, const chx_hip_tensor* w, const chx_hip_tensor* b, int32_t n_batch_axes, chx_hip_tensor* y,
        void* stream) {
    CHX_PROPAGATE(check_f32_matrix(x, "Linear", "x"));
    CHX_PROPAGATE(check_f32_matrix(w, "Linear", "w"));
    CHX_PROPAGATE(check_f32_matrix(y, "Linear", "y"));
    if (b != nullptr) CHX_PROPAGATE(check_f32_matrix(b, "Linear", "b"));
    CHX_REQUIRE(w->ndim == 2, "Linear: w must be [out, in]");
    CHX_REQUIRE(n_batch_axes >= 1 && n_batch_axes < x->ndim, "Linear: n_batch_axes must be in [1, rank of x)");
    CHX_REQUIRE(b == nullptr || (b->ndim == 1 && b->shape[0] == w->shape[0]), "Linear: b must be [out]");
    // x as a matrix [batch extents multiplied, the rest multiplied]: the axes on either side must collapse
    // into one stride each, as they do for a C-contiguous x
    chx_hip_tensor xm = *x;
    int64_t rows = 1, cols = 1;
    for (int i = 0; i < n_batch_axes; ++i) rows *= x->shape[i];
    for (int i = n_batch_axes; i < x->ndim; ++i) cols *= x->shape[i];
    for (int i = 0; i + 1 < x->ndim; ++i) {
        if (i + 1 == n_batch_axes) continue;  // the boundary between the two groups
        CHX_REQUIRE(x->shape[i + 1] == 1 || x->shape[i] == 1 || x->strides[i] == x->strides[i + 1] * x->shape[i + 1],
                    "Linear: the axes of x on one side of n_batch_axes are not contiguous with each other");
    }
    xm.ndim = 2;
    xm.shape[0] = rows;
    xm.shape[1] = cols;
    xm.strides[0] = x->strides[n_batch_axes - 1];
    xm.strides[1] = x->strides[x->ndim - 1];
    // y likewise: [batch extents..., out] with the batch axes collapsing
    chx_hip_tensor ym = *y;
    CHX_REQUIRE(y->ndim == n_batch_axes + 1, "Linear: y must have the batch axes of x and one more");
    for (int i = 0; i < n_batch_axes; ++i) CHX_REQUIRE(y->shape[i] == x->shape[i], "Linear: y and x differ in a batch extent");
    for (int i = 0; i + 1 < n_batch_axes; ++i)
        CHX_REQUIRE(y->shape[i + 1] == 1 || y->shape[i] == 1 || y->strides[i] == y->strides[i + 1] * y->shape[i + 1],
                    "Linear: the batch axes of y are not contiguous with each other");
    ym.ndim = 2;
    ym.shape[0] = rows;
    ym.shape[1] = y->shape[n_batch_axes];
    ym.strides[0] = y->strides[n_batch_axes - 1];
    ym.strides[1] = y->strides[n_batch_axes];
    return run_gemm(xm, false, *w, true, b, 1.f, 1.f, ym, "Linear", as_stream(stream));
}
