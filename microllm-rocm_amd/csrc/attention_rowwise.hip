// Paged attention, one wave per (query token, head): the plain path that every dtype and every
// head size can take, and the float32 path's only attention. Keys are reduced in tiles of 64
// aligned to absolute positions, with a running maximum and sum, so a query's result depends
// on its position and its request's keys only: not on the step's cut, the batch or the pages.
#include "cache_layout.h"
#include "common.h"
#include "microllm_hip.h"

namespace mll {

constexpr int kRowwiseMaxHeadDim = 512;
constexpr int kDimsPerLane = kRowwiseMaxHeadDim / kWave;

template <typename T>
__global__ __launch_bounds__(kWave) void paged_attention_rowwise_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ positions, T* __restrict__ out, float scale, int window,
    int heads, int kv_heads, int head_dim, int page_size) {
    __shared__ float q_shared[kRowwiseMaxHeadDim];
    __shared__ float p_shared[kWave];
    __shared__ int64_t v_shared[kWave];
    const CacheLayout layout(kv_heads, page_size, head_dim);

    const int token = blockIdx.x;
    const int head = blockIdx.y;
    const int lane = threadIdx.x;
    const int kv_head = head / (heads / kv_heads);
    const int seq = seq_of_token[token];
    if (seq < 0) return;      // a row that only pads the step to a fixed shape: its output stays as it is
    const int position = positions[token];
    const int low = window > 0 ? max(0, position - window + 1) : 0;
    const int32_t* table = block_table + static_cast<int64_t>(seq) * table_width;

    const T* q_row = q + (static_cast<int64_t>(token) * heads + head) * head_dim;
    for (int d = lane; d < head_dim; d += kWave) q_shared[d] = to_float(q_row[d]);
    __syncthreads();

    float acc[kDimsPerLane];
#pragma unroll
    for (int i = 0; i < kDimsPerLane; ++i) acc[i] = 0.0f;
    float running_max = -INFINITY;
    float running_sum = 0.0f;

    for (int tile = (low / kWave) * kWave; tile <= position; tile += kWave) {
        const int key = tile + lane;
        const bool visible = key >= low && key <= position;
        float score = -INFINITY;
        int64_t v_column = 0;
        if (visible) {
            const int64_t page = table[key / page_size];
            const int offset = key % page_size;
            const T* k_tile = k_cache + layout.k_tile(page, kv_head, offset / 16);
            v_column = layout.v_tile(page, kv_head, offset / 16) + offset % 16;      // the tile (a multiple of 16) and the place in it
            float dot = 0.0f;
            for (int d = 0; d < head_dim; ++d) dot += q_shared[d] * to_float(k_tile[CacheLayout::k_in_tile(offset % 16, d)]);
            score = dot * scale;
        }
        const float new_max = fmaxf(running_max, wave_max(score));  // every tile holds a visible key
        const float p = visible ? expf(score - new_max) : 0.0f;
        const float rescale = expf(running_max - new_max);          // exp(-inf) = 0 on the first tile
        running_sum = running_sum * rescale + wave_sum(p);
        running_max = new_max;

        __syncthreads();  // the previous tile's readers are done
        p_shared[lane] = p;
        v_shared[lane] = v_column;
        __syncthreads();
        const int first = max(low - tile, 0);
        const int last = min(position - tile, kWave - 1);
#pragma unroll
        for (int i = 0; i < kDimsPerLane; ++i) {
            const int d = lane + i * kWave;
            if (d < head_dim) {
                float value = acc[i] * rescale;
                for (int j = first; j <= last; ++j)
                    value += p_shared[j] * to_float(v_cache[(v_shared[j] & ~int64_t(15)) + layout.v_in_tile(static_cast<int>(v_shared[j] & 15), d)]);
                acc[i] = value;
            }
        }
    }

    T* out_row = out + (static_cast<int64_t>(token) * heads + head) * head_dim;
    const float inverse = 1.0f / running_sum;
#pragma unroll
    for (int i = 0; i < kDimsPerLane; ++i) {
        const int d = lane + i * kWave;
        if (d < head_dim) out_row[d] = from_float<T>(acc[i] * inverse);
    }
}

}  // namespace mll

using namespace mll;

extern "C" int mll_paged_attention_rowwise(const void* q, int dtype, const void* k_cache, const void* v_cache,
                                           const int32_t* block_table, int table_width,
                                           const int32_t* seq_of_token, const int32_t* positions, void* out,
                                           float scale, int window, int n_tokens, int heads, int kv_heads,
                                           int head_dim, int page_size, hipStream_t stream) {
    MLL_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "paged_attention: heads must divide into kv_heads groups");
    MLL_REQUIRE(head_dim > 0 && head_dim <= kRowwiseMaxHeadDim, "paged_attention: head_dim must be in [1, 512]");
    MLL_REQUIRE(page_size > 0 && page_size % 16 == 0 && table_width > 0,
                "paged_attention: page_size must be a multiple of 16 and the table width positive");
    MLL_REQUIRE(heads <= 65535, "paged_attention: more than 65535 heads");
    if (n_tokens == 0) return 0;
    const dim3 grid(n_tokens, heads);
    if (dtype == kF32) {
        paged_attention_rowwise_kernel<float><<<grid, kWave, 0, stream>>>(
            static_cast<const float*>(q), static_cast<const float*>(k_cache), static_cast<const float*>(v_cache),
            block_table, table_width, seq_of_token, positions, static_cast<float*>(out), scale, window,
            heads, kv_heads, head_dim, page_size);
    } else if (dtype == kBF16) {
        paged_attention_rowwise_kernel<bf16><<<grid, kWave, 0, stream>>>(
            static_cast<const bf16*>(q), static_cast<const bf16*>(k_cache), static_cast<const bf16*>(v_cache),
            block_table, table_width, seq_of_token, positions, static_cast<bf16*>(out), scale, window,
            heads, kv_heads, head_dim, page_size);
    } else {
        return fail("paged_attention: unknown dtype");
    }
    return check_launch("paged_attention_rowwise");
}
