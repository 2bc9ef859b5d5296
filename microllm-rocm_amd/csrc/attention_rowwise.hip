// Paged attention, one wave per (query token, head) or per (query token, head, chunk of keys): the plain path
// that every dtype and every head size can take, and the float32 path's only attention.
//
// A query's keys are cut into chunks of 128 at absolute positions. Within a chunk the keys are reduced in tiles
// of 64, also at absolute positions, with a running maximum and sum; the chunks' results are then merged one
// after the other, lowest positions first. Both happen in a fixed order that depends on the query's position
// and its window alone, so a query's result does not depend on the step's cut, the batch or the pages, to the
// last bit. Two ways to run this give the same bits: one wave walks all chunks of its row and merges as it goes
// (steps with many rows: portions of prompts), or one wave per chunk leaves its result in a workspace and a
// second kernel merges them (steps with few rows, whose keys would otherwise be walked by a handful of waves).
// Sums that decide bits are written with explicit fused multiply-adds, so that both kernels round alike.
#include <type_traits>

#include "cache_layout.h"
#include "common.h"
#include "microllm_hip.h"

namespace mll {

constexpr int kRowwiseMaxHeadDim = 512;
constexpr int kRowwiseChunk = 128;      // keys; a multiple of the tiles of 64
// How many query heads of a kv head a wave takes in the float32 kernels: 0 lets the launch choose by how many waves
// the step then still has (rowwise_heads_a_wave); tests and measurements force 1 to 8 with mll_rowwise_heads_a_wave.
static int forced_heads_a_wave = 0;
constexpr int64_t kRowwiseWavesWanted = 4096;      // four a SIMD: fewer leave the loads' latency in the open

__device__ inline void load_eight(const float* from, float (&to)[8]) {
    const float4 low = *reinterpret_cast<const float4*>(from);
    const float4 high = *reinterpret_cast<const float4*>(from + 4);
    to[0] = low.x, to[1] = low.y, to[2] = low.z, to[3] = low.w;
    to[4] = high.x, to[5] = high.y, to[6] = high.z, to[7] = high.w;
}

__device__ inline void load_eight(const bf16* from, float (&to)[8]) {
    union { uint4 raw; bf16 values[8]; } piece;
    piece.raw = *reinterpret_cast<const uint4*>(from);
#pragma unroll
    for (int i = 0; i < 8; ++i) to[i] = to_float(piece.values[i]);
}

// What a row needs to walk its keys.
template <typename T>
struct RowwiseRow {
    const T* k_cache;
    const T* v_cache;
    const int32_t* table;
    int kv_head, head_dim, page_size, lane;
    int low, position;      // the keys the query sees
    float scale;
};

// The keys [first, last] of one chunk (all visible, in one chunk): maximum, sum of exp(score - maximum) and the
// weighted sum of values (dims lane, lane + 64, ...), from zero. q_shared holds the query.
template <typename T, int DIMS>
__device__ inline void attend_chunk(const RowwiseRow<T>& row, const CacheLayout& layout, const float* q_shared,
                                    float* p_shared, int64_t (*v_shared)[kWave], int first, int last, float& chunk_max,
                                    float& chunk_sum, float (&acc)[DIMS]) {
    const int lane = row.lane;
#pragma unroll
    for (int i = 0; i < DIMS; ++i) acc[i] = 0.0f;
    chunk_max = -INFINITY;
    chunk_sum = 0.0f;
    for (int tile = (first / kWave) * kWave; tile <= last; tile += kWave) {
        const int key = tile + lane;
        const bool visible = key >= first && key <= last;
        float score = -INFINITY;
        int64_t v_place = 0, v_place_last = 0;
        if (visible) {
            const int64_t page = row.table[key / row.page_size];
            const int offset = key % row.page_size;
            const T* k_tile = row.k_cache + layout.k_tile(page, row.kv_head, offset / 16) + (offset % 16) * 8;
            // Values lie as [dim / 32][position / 8][dim % 32][position % 8], a last block of 16 dims as
            // [position / 8][16][8] (cache_layout.h): the share of the place that the key's group of 8 positions
            // has, for either kind of block; the dim's share is added below.
            const int64_t v_tile = layout.v_tile(page, row.kv_head, offset / 16);
            v_place = v_tile + ((offset % 16) / 8) * 256;
            v_place_last = v_tile + ((offset % 16) / 8) * 128;
            float dot = 0.0f;
            const int whole = row.head_dim / 8 * 8;
            for (int d = 0; d < whole; d += 8) {      // keys lie as [dim / 8][position][dim % 8]
                float k[8];
                load_eight(k_tile + (d / 8) * 128, k);
#pragma unroll
                for (int i = 0; i < 8; ++i) dot = __fmaf_rn(q_shared[d + i], k[i], dot);
            }
            for (int d = whole; d < row.head_dim; ++d) dot = __fmaf_rn(q_shared[d], to_float(k_tile[(d / 8) * 128 + d % 8]), dot);
            score = __fmul_rn(dot, row.scale);
        }
        const float new_max = fmaxf(chunk_max, wave_max(score));      // every tile holds a visible key
        const float p = visible ? expf(score - new_max) : 0.0f;
        const float rescale = expf(chunk_max - new_max);               // exp(-inf) = 0 on the first tile
        chunk_sum = __fmaf_rn(chunk_sum, rescale, wave_sum(p));
        chunk_max = new_max;

        __syncthreads();      // the previous tile's readers are done
        p_shared[lane] = p;
        v_shared[0][lane] = v_place;
        v_shared[1][lane] = v_place_last;
        __syncthreads();
        const int begin = max(first - tile, 0);
        const int end = min(last - tile, kWave - 1);
#pragma unroll
        for (int i = 0; i < DIMS; ++i) {
            const int d = lane + i * kWave;
            if (d < row.head_dim) {
                const int of_dim = layout.v_in_tile(0, d);
                const int64_t* places = v_shared[layout.v_in_tile(8, d) - of_dim == 256 ? 0 : 1];
                float value = __fmul_rn(acc[i], rescale);
                // Eight positions lie side by side: one read brings a dim's values of a group of 8 keys, of which the
                // visible ones are added in the order of the keys (the others may be stale memory: never multiplied).
                for (int group = begin / 8; group <= end / 8; ++group) {
                    const int from = max(begin, 8 * group), to = min(end, 8 * group + 7);
                    float v[8];
                    load_eight(row.v_cache + places[from] + of_dim, v);
#pragma unroll
                    for (int r = 0; r < 8; ++r)
                        if (8 * group + r >= from && 8 * group + r <= to) value = __fmaf_rn(p_shared[8 * group + r], v[r], value);
                }
                acc[i] = value;
            }
        }
    }
}

// (maximum, sum, values) of the chunks so far, and one more chunk: the same arithmetic wherever chunks are merged.
__device__ inline void merge_scales(float so_far_max, float chunk_max, float& new_max, float& keep, float& add) {
    new_max = fmaxf(so_far_max, chunk_max);
    keep = so_far_max == -INFINITY ? 0.0f : expf(so_far_max - new_max);
    add = expf(chunk_max - new_max);
}

__device__ inline float merged(float so_far, float keep, float chunk, float add) {
    return __fmaf_rn(so_far, keep, __fmul_rn(chunk, add));
}

// DIMS: dims a lane holds (head_dim <= 64 * DIMS). MODE 0: one wave per (token, head) walks all chunks. MODE 1: one wave per (token, head, chunk) writes
// part_o[row][slot][dim] and part_ml[row][slot] = (maximum, sum), slot counting from the row's first chunk.
template <typename T, int MODE, int DIMS>
__global__ __launch_bounds__(kWave) void paged_attention_rowwise_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ positions, T* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, int max_chunks, float scale, int window, int heads, int kv_heads, int head_dim,
    int page_size) {
    __shared__ float q_shared[kRowwiseMaxHeadDim];
    __shared__ float p_shared[kWave];
    __shared__ int64_t v_shared[2][kWave];
    const CacheLayout layout(kv_heads, page_size, head_dim);

    const int token = blockIdx.x;
    const int head = blockIdx.y;
    const int lane = threadIdx.x;
    const int seq = seq_of_token[token];
    if (seq < 0) return;      // a row that only pads the step to a fixed shape: its output stays as it is
    const int position = positions[token];
    const int low = window > 0 ? max(0, position - window + 1) : 0;
    const int first_chunk = low / kRowwiseChunk, last_chunk = position / kRowwiseChunk;
    if (MODE == 1 && first_chunk + static_cast<int>(blockIdx.z) > last_chunk) return;

    RowwiseRow<T> row;
    row.k_cache = k_cache;
    row.v_cache = v_cache;
    row.table = block_table + static_cast<int64_t>(seq) * table_width;
    row.kv_head = head / (heads / kv_heads);
    row.head_dim = head_dim;
    row.page_size = page_size;
    row.lane = lane;
    row.low = low;
    row.position = position;
    row.scale = scale;

    const T* q_row = q + (static_cast<int64_t>(token) * heads + head) * head_dim;
    for (int d = lane; d < head_dim; d += kWave) q_shared[d] = to_float(q_row[d]);
    __syncthreads();

    float acc[DIMS];
    float chunk_max, chunk_sum;
    if (MODE == 1) {
        const int chunk = first_chunk + blockIdx.z;
        attend_chunk(row, layout, q_shared, p_shared, v_shared, max(low, chunk * kRowwiseChunk),
                     min(position, chunk * kRowwiseChunk + kRowwiseChunk - 1), chunk_max, chunk_sum, acc);
        const int64_t slot = (static_cast<int64_t>(token) * heads + head) * max_chunks + blockIdx.z;
#pragma unroll
        for (int i = 0; i < DIMS; ++i) {
            const int d = lane + i * kWave;
            if (d < head_dim) part_o[slot * head_dim + d] = acc[i];
        }
        if (lane == 0) {
            part_ml[slot * 2] = chunk_max;
            part_ml[slot * 2 + 1] = chunk_sum;
        }
        return;
    }

    float total[DIMS];
#pragma unroll
    for (int i = 0; i < DIMS; ++i) total[i] = 0.0f;
    float total_max = -INFINITY, total_sum = 0.0f;
    for (int chunk = first_chunk; chunk <= last_chunk; ++chunk) {
        attend_chunk(row, layout, q_shared, p_shared, v_shared, max(low, chunk * kRowwiseChunk),
                     min(position, chunk * kRowwiseChunk + kRowwiseChunk - 1), chunk_max, chunk_sum, acc);
        float new_max, keep, add;
        merge_scales(total_max, chunk_max, new_max, keep, add);
        total_sum = merged(total_sum, keep, chunk_sum, add);
#pragma unroll
        for (int i = 0; i < DIMS; ++i) total[i] = merged(total[i], keep, acc[i], add);
        total_max = new_max;
    }
    T* out_row = out + (static_cast<int64_t>(token) * heads + head) * head_dim;
    const float inverse = 1.0f / total_sum;
#pragma unroll
    for (int i = 0; i < DIMS; ++i) {
        const int d = lane + i * kWave;
        if (d < head_dim) out_row[d] = from_float<T>(__fmul_rn(total[i], inverse));
    }
}

// MODE 1 for GW query heads of one kv head in one wave: a chunk's keys and values are read once and used for all of
// them (with 7 query heads a kv head the plain kernel reads every key 7 times, and it is those reads that bound it
// when a step has many rows of long requests). Head by head the operations and their order are those of
// attend_chunk: the dot products in ascending dims, the tile's maximum and sum over the wave, the values in the
// order of the keys; only what is independent of the head (addresses, loads) is done once. Writes what MODE 1 writes,
// bit for bit. Head sizes up to 64 * DIMS <= 128.
// MODE as in the kernel for one head a wave: 0 walks all chunks of the row and merges as it goes (out), 1 takes the chunk
// blockIdx.z and leaves its result in the workspace (part_o, part_ml).
template <typename T, int MODE, int DIMS, int GW>
__global__ __launch_bounds__(kWave) void paged_attention_rowwise_heads_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ positions, T* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
    int max_chunks, float scale, int window, int heads, int kv_heads, int head_dim, int page_size) {
    __shared__ float q_shared[GW][64 * DIMS];
    __shared__ float p_shared[GW][kWave];
    __shared__ int64_t v_shared[2][kWave];
    const CacheLayout layout(kv_heads, page_size, head_dim);
    const int token = blockIdx.x;
    const int lane = threadIdx.x;
    const int group = heads / kv_heads;
    const int waves_of_group = (group + GW - 1) / GW;            // the group's last wave may have fewer heads
    const int kv_head = blockIdx.y / waves_of_group;
    const int first_in_group = (blockIdx.y % waves_of_group) * GW;
    const int first_head = kv_head * group + first_in_group;
    const int heads_here = min(GW, group - first_in_group);      // heads past them repeat the last one and write nothing
    const int seq = seq_of_token[token];
    if (seq < 0) return;
    const int position = positions[token];
    const int low = window > 0 ? max(0, position - window + 1) : 0;
    const int first_chunk = low / kRowwiseChunk, last_chunk = position / kRowwiseChunk;
    if (MODE == 1 && first_chunk + static_cast<int>(blockIdx.z) > last_chunk) return;
    const int32_t* table = block_table + static_cast<int64_t>(seq) * table_width;
#pragma unroll
    for (int g = 0; g < GW; ++g) {
        const T* q_row = q + (static_cast<int64_t>(token) * heads + first_head + min(g, heads_here - 1)) * head_dim;
        for (int d = lane; d < head_dim; d += kWave) q_shared[g][d] = to_float(q_row[d]);
    }
    __syncthreads();

    float acc[GW][DIMS], chunk_max[GW], chunk_sum[GW];
    // The keys [first, last] of one chunk, from zero: attend_chunk for every head of the wave.
    auto attend = [&](int first, int last) __attribute__((always_inline)) {
#pragma unroll
    for (int g = 0; g < GW; ++g) {
        chunk_max[g] = -INFINITY;
        chunk_sum[g] = 0.0f;
#pragma unroll
        for (int i = 0; i < DIMS; ++i) acc[g][i] = 0.0f;
    }
    for (int tile = (first / kWave) * kWave; tile <= last; tile += kWave) {
        const int key = tile + lane;
        const bool visible = key >= first && key <= last;
        float dot[GW];
#pragma unroll
        for (int g = 0; g < GW; ++g) dot[g] = 0.0f;
        int64_t v_place = 0, v_place_last = 0;
        if (visible) {
            const int64_t page = table[key / page_size];
            const int offset = key % page_size;
            const T* k_tile = k_cache + layout.k_tile(page, kv_head, offset / 16) + (offset % 16) * 8;
            const int64_t v_tile = layout.v_tile(page, kv_head, offset / 16);
            v_place = v_tile + ((offset % 16) / 8) * 256;
            v_place_last = v_tile + ((offset % 16) / 8) * 128;
            const int whole = head_dim / 8 * 8;
#pragma unroll 4
            for (int d = 0; d < whole; d += 8) {
                float k[8];
                load_eight(k_tile + (d / 8) * 128, k);
#pragma unroll
                for (int g = 0; g < GW; ++g)
#pragma unroll
                    for (int i = 0; i < 8; ++i) dot[g] = __fmaf_rn(q_shared[g][d + i], k[i], dot[g]);
            }
            for (int d = whole; d < head_dim; ++d) {
                const float k = to_float(k_tile[(d / 8) * 128 + d % 8]);
#pragma unroll
                for (int g = 0; g < GW; ++g) dot[g] = __fmaf_rn(q_shared[g][d], k, dot[g]);
            }
        }
        float rescale[GW];
        __syncthreads();      // the previous tile's readers are done
#pragma unroll
        for (int g = 0; g < GW; ++g) {
            const float score = visible ? __fmul_rn(dot[g], scale) : -INFINITY;
            const float new_max = fmaxf(chunk_max[g], wave_max(score));
            const float p = visible ? expf(score - new_max) : 0.0f;
            rescale[g] = expf(chunk_max[g] - new_max);
            chunk_sum[g] = __fmaf_rn(chunk_sum[g], rescale[g], wave_sum(p));
            chunk_max[g] = new_max;
            p_shared[g][lane] = p;
        }
        v_shared[0][lane] = v_place;
        v_shared[1][lane] = v_place_last;
        __syncthreads();
        const int begin = max(first - tile, 0);
        const int end = min(last - tile, kWave - 1);
#pragma unroll
        for (int i = 0; i < DIMS; ++i) {
            const int d = lane + i * kWave;
            if (d < head_dim) {
                const int of_dim = layout.v_in_tile(0, d);
                const int64_t* places = v_shared[layout.v_in_tile(8, d) - of_dim == 256 ? 0 : 1];
                float value[GW];
#pragma unroll
                for (int g = 0; g < GW; ++g) value[g] = __fmul_rn(acc[g][i], rescale[g]);
                for (int eight = begin / 8; eight <= end / 8; ++eight) {
                    const int from = max(begin, 8 * eight), to = min(end, 8 * eight + 7);
                    float v[8];
                    load_eight(v_cache + places[from] + of_dim, v);
#pragma unroll
                    for (int g = 0; g < GW; ++g)
#pragma unroll
                        for (int r = 0; r < 8; ++r)
                            if (8 * eight + r >= from && 8 * eight + r <= to) value[g] = __fmaf_rn(p_shared[g][8 * eight + r], v[r], value[g]);
                }
#pragma unroll
                for (int g = 0; g < GW; ++g) acc[g][i] = value[g];
            }
        }
    }
    };

    if (MODE == 1) {
        const int chunk = first_chunk + blockIdx.z;
        attend(max(low, chunk * kRowwiseChunk), min(position, chunk * kRowwiseChunk + kRowwiseChunk - 1));
#pragma unroll
        for (int g = 0; g < GW; ++g) {
            if (g >= heads_here) break;
            const int64_t slot = (static_cast<int64_t>(token) * heads + first_head + g) * max_chunks + blockIdx.z;
#pragma unroll
            for (int i = 0; i < DIMS; ++i) {
                const int d = lane + i * kWave;
                if (d < head_dim) part_o[slot * head_dim + d] = acc[g][i];
            }
            if (lane == 0) {
                part_ml[slot * 2] = chunk_max[g];
                part_ml[slot * 2 + 1] = chunk_sum[g];
            }
        }
        return;
    }
    float total[GW][DIMS], total_max[GW], total_sum[GW];
#pragma unroll
    for (int g = 0; g < GW; ++g) {
        total_max[g] = -INFINITY;
        total_sum[g] = 0.0f;
#pragma unroll
        for (int i = 0; i < DIMS; ++i) total[g][i] = 0.0f;
    }
    for (int chunk = first_chunk; chunk <= last_chunk; ++chunk) {
        attend(max(low, chunk * kRowwiseChunk), min(position, chunk * kRowwiseChunk + kRowwiseChunk - 1));
#pragma unroll
        for (int g = 0; g < GW; ++g) {
            float new_max, keep, add;
            merge_scales(total_max[g], chunk_max[g], new_max, keep, add);
            total_sum[g] = merged(total_sum[g], keep, chunk_sum[g], add);
#pragma unroll
            for (int i = 0; i < DIMS; ++i) total[g][i] = merged(total[g][i], keep, acc[g][i], add);
            total_max[g] = new_max;
        }
    }
#pragma unroll
    for (int g = 0; g < GW; ++g) {
        if (g >= heads_here) break;
        T* out_row = out + (static_cast<int64_t>(token) * heads + first_head + g) * head_dim;
        const float inverse = 1.0f / total_sum[g];
#pragma unroll
        for (int i = 0; i < DIMS; ++i) {
            const int d = lane + i * kWave;
            if (d < head_dim) out_row[d] = from_float<T>(__fmul_rn(total[g][i], inverse));
        }
    }
}

// How many query heads of a kv head one wave of the kernel above takes in a step of `rows` (token, kv head, chunk)
// items: as many as leave the GPU its waves, of the counts that fill the group's waves evenly (7 heads: 7, or 4
// and 3, or 2, 2, 2 and 1; not 5 and 2). One: the kernel for one head a wave.
static int rowwise_heads_a_wave(int group, int64_t rows) {
    const int most = group < 8 ? group : 8;
    if (forced_heads_a_wave > 0) return forced_heads_a_wave < most ? forced_heads_a_wave : most;
    for (int count = most; count >= 2; --count) {
        const int waves = (group + count - 1) / count;
        if (waves * count - group > 1) continue;      // the group's last wave would have much less than the others
        if (rows * waves >= kRowwiseWavesWanted) return count;
    }
    return 1;
}

// Merges what MODE 1 left, in the order and with the arithmetic of MODE 0. One wave per (token, head).
template <typename T, int DIMS>
__global__ __launch_bounds__(kWave) void paged_attention_rowwise_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ positions, T* __restrict__ out, int max_chunks, int window, int heads, int head_dim) {
    const int token = blockIdx.x;
    const int head = blockIdx.y;
    const int lane = threadIdx.x;
    if (seq_of_token[token] < 0) return;
    const int position = positions[token];
    const int low = window > 0 ? max(0, position - window + 1) : 0;
    const int chunks = position / kRowwiseChunk - low / kRowwiseChunk + 1;
    const int64_t first_slot = (static_cast<int64_t>(token) * heads + head) * max_chunks;
    float total[DIMS];
#pragma unroll
    for (int i = 0; i < DIMS; ++i) total[i] = 0.0f;
    float total_max = -INFINITY, total_sum = 0.0f;
    // Eight chunks' results are asked for at once and then merged one after the other: the loads of a chunk do not
    // wait for the merge of the chunk before.
    constexpr int kAtOnce = 8;
    for (int base = 0; base < chunks; base += kAtOnce) {
        float chunk_max[kAtOnce], chunk_sum[kAtOnce], chunk_o[kAtOnce][DIMS];
#pragma unroll
        for (int u = 0; u < kAtOnce; ++u) {
            const int64_t slot = first_slot + min(base + u, chunks - 1);
            chunk_max[u] = part_ml[slot * 2];
            chunk_sum[u] = part_ml[slot * 2 + 1];
#pragma unroll
            for (int i = 0; i < DIMS; ++i) {
                const int d = lane + i * kWave;
                chunk_o[u][i] = d < head_dim ? part_o[slot * head_dim + d] : 0.0f;
            }
        }
#pragma unroll
        for (int u = 0; u < kAtOnce; ++u) {
            if (base + u >= chunks) break;
            float new_max, keep, add;
            merge_scales(total_max, chunk_max[u], new_max, keep, add);
            total_sum = merged(total_sum, keep, chunk_sum[u], add);
#pragma unroll
            for (int i = 0; i < DIMS; ++i) total[i] = merged(total[i], keep, chunk_o[u][i], add);
            total_max = new_max;
        }
    }
    T* out_row = out + (static_cast<int64_t>(token) * heads + head) * head_dim;
    const float inverse = 1.0f / total_sum;
#pragma unroll
    for (int i = 0; i < DIMS; ++i) {
        const int d = lane + i * kWave;
        if (d < head_dim) out_row[d] = from_float<T>(__fmul_rn(total[i], inverse));
    }
}

template <typename T, int DIMS>
static int launch_rowwise_dims(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_table,
                          int table_width, const int32_t* seq_of_token, const int32_t* positions, void* out,
                          float* part_o, float* part_ml, int max_chunks, int usual_chunks, float scale, int window, int n_tokens,
                          int heads, int kv_heads, int head_dim, int page_size, hipStream_t stream) {
    const int group = heads / kv_heads;
    const int64_t rows = static_cast<int64_t>(n_tokens) * kv_heads * (max_chunks > 0 ? (usual_chunks > 0 ? usual_chunks : max_chunks) : 1);
    const int gw = (std::is_same<T, float>::value && DIMS <= 2) ? rowwise_heads_a_wave(group, rows) : 1;
    const bool several_heads = gw >= 2;
    const int group_waves = kv_heads * ((group + gw - 1) / gw);
#define MLL_ROWWISE_HEADS(MODE, GW)                                                                                    \
    case GW:                                                                                                           \
        paged_attention_rowwise_heads_kernel<T, MODE, DIMS, GW><<<heads_grid, kWave, 0, stream>>>(                      \
            static_cast<const T*>(q), static_cast<const T*>(k_cache), static_cast<const T*>(v_cache), block_table,    \
            table_width, seq_of_token, positions, static_cast<T*>(out), part_o, part_ml, max_chunks, scale, window,   \
            heads, kv_heads, head_dim, page_size);                                                                     \
        break;
#define MLL_ROWWISE_HEADS_ALL(MODE)                                                                                    \
    switch (gw) {                                                                                                      \
        MLL_ROWWISE_HEADS(MODE, 2) MLL_ROWWISE_HEADS(MODE, 3) MLL_ROWWISE_HEADS(MODE, 4) MLL_ROWWISE_HEADS(MODE, 5)    \
        MLL_ROWWISE_HEADS(MODE, 6) MLL_ROWWISE_HEADS(MODE, 7) MLL_ROWWISE_HEADS(MODE, 8)                               \
        default: break;                                                                                                \
    }
    if (max_chunks == 0) {
        if constexpr (std::is_same<T, float>::value && DIMS <= 2) {
            if (several_heads) {
                const dim3 heads_grid(n_tokens, group_waves);
                MLL_ROWWISE_HEADS_ALL(0)
                return check_launch("paged_attention_rowwise");
            }
        }
        paged_attention_rowwise_kernel<T, 0, DIMS><<<dim3(n_tokens, heads), kWave, 0, stream>>>(
            static_cast<const T*>(q), static_cast<const T*>(k_cache), static_cast<const T*>(v_cache), block_table,
            table_width, seq_of_token, positions, static_cast<T*>(out), nullptr, nullptr, 0, scale, window, heads,
            kv_heads, head_dim, page_size);
        return check_launch("paged_attention_rowwise");
    }
    // Several query heads of a kv head in one wave where the step still has rows enough for the GPU that way
    // (float32, head sizes up to 128: the path of the 32-bit engine).
    bool grouped = false;
    if constexpr (std::is_same<T, float>::value && DIMS <= 2) {
        if (several_heads) {
            grouped = true;
            const dim3 heads_grid(n_tokens, group_waves, max_chunks);
            MLL_ROWWISE_HEADS_ALL(1)
        }
    }
    if (!grouped)
        paged_attention_rowwise_kernel<T, 1, DIMS><<<dim3(n_tokens, heads, max_chunks), kWave, 0, stream>>>(
            static_cast<const T*>(q), static_cast<const T*>(k_cache), static_cast<const T*>(v_cache), block_table,
            table_width, seq_of_token, positions, static_cast<T*>(out), part_o, part_ml, max_chunks, scale, window, heads,
            kv_heads, head_dim, page_size);
    if (const int status = check_launch("paged_attention_rowwise")) return status;
    paged_attention_rowwise_merge_kernel<T, DIMS><<<dim3(n_tokens, heads), kWave, 0, stream>>>(
        part_o, part_ml, seq_of_token, positions, static_cast<T*>(out), max_chunks, window, heads, head_dim);
    return check_launch("paged_attention_rowwise_merge");
#undef MLL_ROWWISE_HEADS_ALL
#undef MLL_ROWWISE_HEADS
}

template <typename T>
static int launch_rowwise(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_table,
                          int table_width, const int32_t* seq_of_token, const int32_t* positions, void* out,
                          float* part_o, float* part_ml, int max_chunks, int usual_chunks, float scale, int window, int n_tokens,
                          int heads, int kv_heads, int head_dim, int page_size, hipStream_t stream) {
#define MLL_ROWWISE_DIMS(D)                                                                                            \
    return launch_rowwise_dims<T, D>(q, k_cache, v_cache, block_table, table_width, seq_of_token, positions, out, part_o, \
                                     part_ml, max_chunks, usual_chunks, scale, window, n_tokens, heads, kv_heads, head_dim, page_size, stream)
    if (head_dim <= kWave) MLL_ROWWISE_DIMS(1);
    if (head_dim <= 2 * kWave) MLL_ROWWISE_DIMS(2);
    if (head_dim <= 4 * kWave) MLL_ROWWISE_DIMS(4);
    MLL_ROWWISE_DIMS(8);
#undef MLL_ROWWISE_DIMS
}

}  // namespace mll

using namespace mll;

extern "C" int mll_paged_attention_rowwise_chunk() { return kRowwiseChunk; }

// Forces how many query heads of a kv head a wave of the float32 kernels takes (1 to 8; more than the group has:
// the group), or with 0 gives the choice back to the launch; returns the value before. Every count gives the same bits.
extern "C" int mll_rowwise_heads_a_wave(int count) {
    const int before = mll::forced_heads_a_wave;
    mll::forced_heads_a_wave = count < 0 ? 0 : count;
    return before;
}

// max_chunks 0: one wave per (token, head). Otherwise one wave per chunk, for rows whose keys span at most
// max_chunks chunks (the caller's promise: a row with more would lose its last ones), with part_o
// [n_tokens * heads * max_chunks * head_dim] and part_ml [n_tokens * heads * max_chunks * 2] floats as workspace.
// usual_chunks (0: max_chunks): how many chunks the step's rows have now, where max_chunks leaves room for later
// steps of the same shape; only how many heads a wave takes follows from it.
extern "C" int mll_paged_attention_rowwise(const void* q, int dtype, const void* k_cache, const void* v_cache,
                                           const int32_t* block_table, int table_width,
                                           const int32_t* seq_of_token, const int32_t* positions, void* out,
                                           float* part_o, float* part_ml, int max_chunks, int usual_chunks, float scale,
                                           int window, int n_tokens, int heads, int kv_heads, int head_dim, int page_size,
                                           hipStream_t stream) {
    MLL_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "paged_attention: heads must divide into kv_heads groups");
    MLL_REQUIRE(head_dim > 0 && head_dim <= kRowwiseMaxHeadDim, "paged_attention: head_dim must be in [1, 512]");
    MLL_REQUIRE(page_size > 0 && page_size % 16 == 0 && table_width > 0,
                "paged_attention: page_size must be a multiple of 16 and the table width positive");
    MLL_REQUIRE(heads <= 65535, "paged_attention: more than 65535 heads");
    MLL_REQUIRE(max_chunks >= 0 && max_chunks <= 65535, "paged_attention: bad number of chunks");
    MLL_REQUIRE(max_chunks == 0 || (part_o && part_ml), "paged_attention: chunks need the partial buffers");
    if (n_tokens == 0) return 0;
    if (dtype == kF32)
        return launch_rowwise<float>(q, k_cache, v_cache, block_table, table_width, seq_of_token, positions, out, part_o,
                                     part_ml, max_chunks, usual_chunks, scale, window, n_tokens, heads, kv_heads, head_dim, page_size, stream);
    if (dtype == kBF16)
        return launch_rowwise<bf16>(q, k_cache, v_cache, block_table, table_width, seq_of_token, positions, out, part_o,
                                    part_ml, max_chunks, usual_chunks, scale, window, n_tokens, heads, kv_heads, head_dim, page_size, stream);
    return fail("paged_attention: unknown dtype");
}
