// The float32 matrix product of the true 32-bit path: C = A * W^T (+ bias), 64x64 tiles staged
// through LDS, a 4x4 block of outputs per thread. Every output element is summed by one thread
// in ascending k, so a row's result is the same whatever other rows the call holds.
#include "common.h"
#include "microllm_hip.h"

namespace mll {

constexpr int kTile = 64;
constexpr int kDepth = 16;

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ a, const float* __restrict__ w,
                                                       const float* __restrict__ bias, float* __restrict__ c,
                                                       int m, int n, int k) {
    __shared__ float a_tile[kDepth][kTile + 4];
    __shared__ float w_tile[kDepth][kTile + 4];
    const int row0 = blockIdx.y * kTile;
    const int col0 = blockIdx.x * kTile;
    const int tx = threadIdx.x % 16;  // 4 output columns each
    const int ty = threadIdx.x / 16;  // 4 output rows each
    const int load_row = threadIdx.x / 4;        // 0..63
    const int load_k = (threadIdx.x % 4) * 4;    // 0,4,8,12

    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;

    for (int k0 = 0; k0 < k; k0 += kDepth) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int kk = k0 + load_k + e;
            const int ar = row0 + load_row;
            const int wr = col0 + load_row;
            a_tile[load_k + e][load_row] = (ar < m && kk < k) ? a[static_cast<int64_t>(ar) * k + kk] : 0.0f;
            w_tile[load_k + e][load_row] = (wr < n && kk < k) ? w[static_cast<int64_t>(wr) * k + kk] : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < kDepth; ++kk) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = a_tile[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[j] = w_tile[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = row0 + ty * 4 + i;
        if (row >= m) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = col0 + tx * 4 + j;
            if (col < n) c[static_cast<int64_t>(row) * n + col] = acc[i][j] + (bias ? bias[col] : 0.0f);
        }
    }
}

}  // namespace mll

using namespace mll;

extern "C" int mll_gemm_f32(const float* a, const float* w, const float* bias, float* c,
                            int m, int n, int k, hipStream_t stream) {
    MLL_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm_f32: sizes must be positive");
    if (m == 0) return 0;
    const dim3 grid((n + kTile - 1) / kTile, (m + kTile - 1) / kTile);
    MLL_REQUIRE(grid.y <= 65535, "gemm_f32: too many rows for one call");
    gemm_f32_kernel<<<grid, 256, 0, stream>>>(a, w, bias, c, m, n, k);
    return check_launch("gemm_f32");
}
