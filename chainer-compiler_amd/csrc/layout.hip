// Byte-tensor layout changes between NCHW-contiguous arrays (what a caller that knows
// nothing about layouts hands over) and the channels-last layout the MFMA kernels use.
// 64x64-byte tiles through LDS; reads and writes are both contiguous along their
// fastest axis.
#include "conv_mfma.h"

namespace chx {
namespace {

constexpr int kTile = 64;

// src [N][C][HW] -> dst [N][HW][pitch]
__global__ __launch_bounds__(256) void nchw_to_nhwc_u8_kernel(
        const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int C, int64_t HW, int pitch) {
    __shared__ uint8_t tile[kTile][kTile + 4];
    const int n = blockIdx.z;
    const int64_t p0 = (int64_t)blockIdx.x * kTile;
    const int c0 = blockIdx.y * kTile;
    const uint8_t* s = src + (int64_t)n * C * HW;
    uint8_t* d = dst + (int64_t)n * HW * pitch;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4
    for (int r = ty; r < kTile; r += 4) {
        const int c = c0 + r;
        const int64_t p = p0 + tx;
        tile[r][tx] = (c < C && p < HW) ? s[(int64_t)c * HW + p] : 0;
    }
    __syncthreads();
    for (int r = ty; r < kTile; r += 4) {
        const int64_t p = p0 + r;
        const int c = c0 + tx;
        if (p < HW && c < pitch) d[p * pitch + c] = tile[tx][r];
    }
}

// src [N][HW][pitch] -> dst [N][C][HW]
__global__ __launch_bounds__(256) void nhwc_to_nchw_u8_kernel(
        const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int C, int64_t HW, int pitch) {
    __shared__ uint8_t tile[kTile][kTile + 4];
    const int n = blockIdx.z;
    const int64_t p0 = (int64_t)blockIdx.x * kTile;
    const int c0 = blockIdx.y * kTile;
    const uint8_t* s = src + (int64_t)n * HW * pitch;
    uint8_t* d = dst + (int64_t)n * C * HW;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int r = ty; r < kTile; r += 4) {
        const int64_t p = p0 + r;
        const int c = c0 + tx;
        tile[r][tx] = (p < HW && c < C) ? s[p * pitch + c] : 0;
    }
    __syncthreads();
    for (int r = ty; r < kTile; r += 4) {
        const int c = c0 + r;
        const int64_t p = p0 + tx;
        if (c < C && p < HW) d[(int64_t)c * HW + p] = tile[tx][r];
    }
}

}  // namespace

int launch_nchw_to_nhwc_u8(const char* src, char* dst, int N, int C, int64_t HW, int pitch, hipStream_t s) {
    if (N == 0 || C == 0 || HW == 0) return CHX_HIP_OK;
    dim3 grid((unsigned)((HW + kTile - 1) / kTile), (unsigned)((pitch + kTile - 1) / kTile), (unsigned)N);
    nchw_to_nhwc_u8_kernel<<<grid, 256, 0, s>>>(
            reinterpret_cast<const uint8_t*>(src), reinterpret_cast<uint8_t*>(dst), C, HW, pitch);
    return launch_check("nchw_to_nhwc_u8_kernel");
}

int launch_nhwc_to_nchw_u8(const char* src, char* dst, int N, int C, int64_t HW, int pitch, hipStream_t s) {
    if (N == 0 || C == 0 || HW == 0) return CHX_HIP_OK;
    dim3 grid((unsigned)((HW + kTile - 1) / kTile), (unsigned)((C + kTile - 1) / kTile), (unsigned)N);
    nhwc_to_nchw_u8_kernel<<<grid, 256, 0, s>>>(
            reinterpret_cast<const uint8_t*>(src), reinterpret_cast<uint8_t*>(dst), C, HW, pitch);
    return launch_check("nhwc_to_nchw_u8_kernel");
}

}  // namespace chx
