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

// The same product for at most 16 rows (decoding): a workgroup takes 16 columns of C, so that a weight of a few
// thousand rows fills the GPU where tiles of 64 would leave most of it idle, and one thread one output element.
// Each thread sums in ascending k with the same fused multiply-adds as the tiled kernel: the two give the same
// bits, so a token's result does not depend on how many rows the step had.
constexpr int kSmallColumns = 16;
constexpr int kSmallDepth = 128;

// VECTOR: k is a multiple of 4 and both matrices are 16-byte aligned, so a thread's four consecutive elements are
// one load.
template <bool VECTOR>
__global__ __launch_bounds__(256) void gemm_f32_small_kernel(const float* __restrict__ a, const float* __restrict__ w,
                                                             const float* __restrict__ bias, float* __restrict__ c,
                                                             int m, int n, int k) {
    // Rows of kSmallDepth + 4 floats: 16-byte aligned, so that four consecutive k are one read, and four banks on
    // from row to row, so that the 16 rows (or columns) that a wave reads at one k fall on different banks.
    __shared__ __align__(16) float a_tile[16][kSmallDepth + 4];
    __shared__ __align__(16) float w_tile[kSmallColumns][kSmallDepth + 4];
    const int col0 = blockIdx.x * kSmallColumns;
    const int column = threadIdx.x % kSmallColumns;     // this thread's output: row `row`, column col0 + `column`
    const int row = threadIdx.x / kSmallColumns;
    // What a thread brings in of a chunk of kSmallDepth of k: of row load_row of A and of W, elements
    // load_k .. load_k + 3 and 64 + load_k .. 64 + load_k + 3.
    const int load_row = threadIdx.x / 16;
    const int load_k = (threadIdx.x % 16) * 4;
    const bool a_live = load_row < m, w_live = col0 + load_row < n;
    const float* a_row = a + static_cast<int64_t>(a_live ? load_row : 0) * k;
    const float* w_row = w + static_cast<int64_t>(w_live ? col0 + load_row : 0) * k;
    float4 a_next[2], w_next[2];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int part = 0; part < 2; ++part) {
            const int kk = k0 + 64 * part + load_k;
            if (VECTOR) {
                a_next[part] = (a_live && kk < k) ? *reinterpret_cast<const float4*>(a_row + kk) : make_float4(0.f, 0.f, 0.f, 0.f);
                w_next[part] = (w_live && kk < k) ? *reinterpret_cast<const float4*>(w_row + kk) : make_float4(0.f, 0.f, 0.f, 0.f);
            } else {
                float av[4], wv[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    av[e] = (a_live && kk + e < k) ? a_row[kk + e] : 0.0f;
                    wv[e] = (w_live && kk + e < k) ? w_row[kk + e] : 0.0f;
                }
                a_next[part] = make_float4(av[0], av[1], av[2], av[3]);
                w_next[part] = make_float4(wv[0], wv[1], wv[2], wv[3]);
            }
        }
    };
    float acc = 0.0f;
    fetch(0);
    for (int k0 = 0; k0 < k; k0 += kSmallDepth) {
#pragma unroll
        for (int part = 0; part < 2; ++part) {
            const int at = 64 * part + load_k;
            *reinterpret_cast<float4*>(&a_tile[load_row][at]) = a_next[part];
            *reinterpret_cast<float4*>(&w_tile[load_row][at]) = w_next[part];
        }
        __syncthreads();
        if (k0 + kSmallDepth < k) fetch(k0 + kSmallDepth);      // the next chunk is on its way while this one is summed
        // Four k a read, summed one after the other in ascending k as before: the same bits.
#pragma unroll
        for (int kk = 0; kk < kSmallDepth; kk += 4) {
            const float4 av = *reinterpret_cast<const float4*>(&a_tile[row][kk]);
            const float4 wv = *reinterpret_cast<const float4*>(&w_tile[column][kk]);
            acc = fmaf(av.x, wv.x, acc);
            acc = fmaf(av.y, wv.y, acc);
            acc = fmaf(av.z, wv.z, acc);
            acc = fmaf(av.w, wv.w, acc);
        }
        __syncthreads();
    }
    const int col = col0 + column;
    if (row < m && col < n) c[static_cast<int64_t>(row) * n + col] = acc + (bias ? bias[col] : 0.0f);
}

}  // namespace mll

using namespace mll;

extern "C" int mll_gemm_f32(const float* a, const float* w, const float* bias, float* c,
                            int m, int n, int k, hipStream_t stream) {
    MLL_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm_f32: sizes must be positive");
    if (m == 0) return 0;
    if (m <= 16) {
        const bool vector = k % 4 == 0 && reinterpret_cast<uintptr_t>(a) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
        const int groups = (n + kSmallColumns - 1) / kSmallColumns;
        if (vector) gemm_f32_small_kernel<true><<<groups, 256, 0, stream>>>(a, w, bias, c, m, n, k);
        else gemm_f32_small_kernel<false><<<groups, 256, 0, stream>>>(a, w, bias, c, m, n, k);
        return check_launch("gemm_f32");
    }
    const dim3 grid((n + kTile - 1) / kTile, (m + kTile - 1) / kTile);
    MLL_REQUIRE(grid.y <= 65535, "gemm_f32: too many rows for one call");
    gemm_f32_kernel<<<grid, 256, 0, stream>>>(a, w, bias, c, m, n, k);
    return check_launch("gemm_f32");
}
