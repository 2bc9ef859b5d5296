// Paged attention for portions of prompts in bfloat16: MFMA for both products, online softmax in float32.
//
// A workgroup (4 waves) takes 64 consecutive tokens of one request's portion and one query head; a wave
// takes 16 of those tokens. As in the decode kernel, scores are computed transposed, S^T = K . Q^T, with the
// 16 columns now being 16 query positions, and O^T = V^T . P^T follows from registers alone. A wave walks the
// keys of its request from the first one any of its queries can see to its last query's own position, in
// pairs of 16-key tiles read straight from the pages (which are laid out in MFMA order, cache_layout.h);
// only pairs that touch the causal diagonal or the window's edge pay for the mask.
// The list of 64-token tiles (request, first token in the flat list, tokens in the tile) is built on the host.
#include "cache_layout.h"
#include "common.h"
#include "microllm_hip.h"

namespace mll {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kPrefillWaves = 4;
constexpr int kPrefillThreads = kPrefillWaves * kWave;
constexpr int kPrefillTile = 16 * kPrefillWaves;   // tokens per workgroup

union PFrag8 {
    bf16x8 v;
    bf16x4 h[2];
    uint4 raw;
};

template <int HD_TILES>
__global__ __launch_bounds__(kPrefillThreads) void paged_attention_prefill_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ tiles,
    const int32_t* __restrict__ positions, bf16* __restrict__ out, float scale, int window, int heads,
    int kv_heads, int page_size) {
    constexpr int HD = HD_TILES * 16;
    constexpr int K_STEPS = (HD + 31) / 32;
    constexpr int K_CHUNKS = HD / 8;

    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int col = lane % 16;
    const int quad = lane / 16;

    const int seq = tiles[3 * blockIdx.x + 0];
    const int tile_token = tiles[3 * blockIdx.x + 1];
    const int tile_count = tiles[3 * blockIdx.x + 2];
    const int head = blockIdx.y;
    const int kv_head = head / (heads / kv_heads);
    const int first = wave * 16;              // this wave's first token inside the tile
    if (first >= tile_count) return;
    const int valid = min(16, tile_count - first);
    const int token0 = tile_token + first;
    const int position0 = positions[token0];  // tokens of a portion have consecutive positions
    const int my_position = position0 + min(col, valid - 1);   // columns past the end repeat the last token
    const int last_position = position0 + valid - 1;
    const int my_low = window > 0 ? max(0, my_position - window + 1) : 0;
    const int first_low = window > 0 ? max(0, position0 - window + 1) : 0;
    const int last_low = window > 0 ? max(0, last_position - window + 1) : 0;
    const int32_t* table = block_table + static_cast<int64_t>(seq) * table_width;
    const CacheLayout layout(kv_heads, page_size, HD);

    PFrag8 q_frag[K_STEPS];
#pragma unroll
    for (int ks = 0; ks < K_STEPS; ++ks) {
        const int dim = ks * 32 + quad * 8;
        q_frag[ks].raw = make_uint4(0, 0, 0, 0);
        if (dim < HD)
            q_frag[ks].raw = *reinterpret_cast<const uint4*>(
                q + (static_cast<int64_t>(token0 + min(col, valid - 1)) * heads + head) * HD + dim);
    }

    floatx4 o_acc[HD_TILES];
#pragma unroll
    for (int d = 0; d < HD_TILES; ++d) o_acc[d] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    float running_max = -INFINITY, running_sum = 0.0f;

    auto page_of = [&](int tile_key) -> int {
        return (tile_key <= last_position && tile_key + 15 >= first_low) ? table[tile_key / page_size] : -1;
    };
    const int pair_end = last_position / 32 + 1;
    int pair = first_low / 32;
    int next_page[2] = {page_of(pair * 32), page_of(pair * 32 + 16)};
    for (; pair < pair_end; ++pair) {
        const int key0 = pair * 32;
        const int page[2] = {next_page[0], next_page[1]};
        if (pair + 1 < pair_end) {
            next_page[0] = page_of((pair + 1) * 32);
            next_page[1] = page_of((pair + 1) * 32 + 16);
        }
        PFrag8 k_frag[2][K_STEPS];
        PFrag8 v_frag[HD_TILES];
#pragma unroll
        for (int d = 0; d < HD_TILES; ++d) v_frag[d].raw = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int offset = (key0 + 16 * t) % page_size;
            const bf16* k_tile = k_cache + layout.k_tile(max(page[t], 0), kv_head, offset / 16) + col * 8;
            const bf16* v_tile = v_cache + layout.v_tile(max(page[t], 0), kv_head, offset / 16) + (quad * 16 + col) * 4;
#pragma unroll
            for (int ks = 0; ks < K_STEPS; ++ks) {
                const int piece = ks * 4 + quad;
                k_frag[t][ks].raw = make_uint4(0, 0, 0, 0);
                if (page[t] >= 0 && piece < K_CHUNKS)
                    k_frag[t][ks].raw = *reinterpret_cast<const uint4*>(k_tile + piece * 128);
            }
            if (page[t] >= 0) {
#pragma unroll
                for (int d = 0; d < HD_TILES; ++d)
                    v_frag[d].h[t] = *reinterpret_cast<const bf16x4*>(v_tile + d * 256);
            }
        }

        float score[8];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            floatx4 s = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int ks = 0; ks < K_STEPS; ++ks)
                s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k_frag[t][ks].v, q_frag[ks].v, s, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) score[4 * t + i] = s[i] * scale;
        }
        // Pairs every query of the wave sees whole need no mask.
        if (key0 + 31 > position0 || key0 < last_low) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int key = key0 + 16 * (j / 4) + 4 * quad + (j % 4);
                if (key > my_position || key < my_low) score[j] = -INFINITY;
                // Keys no query of the wave can see may be stale memory: keep them out of the product.
                if (key > last_position || key < first_low) {
#pragma unroll
                    for (int d = 0; d < HD_TILES; ++d) v_frag[d].v[j] = static_cast<__bf16>(0.0f);
                }
            }
        }

        float tile_max = score[0];
#pragma unroll
        for (int j = 1; j < 8; ++j) tile_max = fmaxf(tile_max, score[j]);
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, kWave));
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, kWave));
        const float new_max = fmaxf(running_max, tile_max);
        // A query may see nothing of a pair that others see (the window's edge): its maximum stays -inf.
        const float safe_max = new_max == -INFINITY ? 0.0f : new_max;
        const float rescale = __expf(running_max - safe_max);
        PFrag8 p_frag;
        float tile_sum = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float p = __expf(score[j] - safe_max);
            tile_sum += p;
            p_frag.v[j] = static_cast<__bf16>(p);
        }
        tile_sum += __shfl_xor(tile_sum, 16, kWave);
        tile_sum += __shfl_xor(tile_sum, 32, kWave);
        running_sum = running_sum * rescale + tile_sum;
        running_max = new_max;
#pragma unroll
        for (int d = 0; d < HD_TILES; ++d) {
            o_acc[d] *= rescale;
            o_acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_frag[d].v, p_frag.v, o_acc[d], 0, 0, 0);
        }
    }

    if (col < valid) {
        const float inverse = 1.0f / running_sum;
        bf16* out_row = out + (static_cast<int64_t>(token0 + col) * heads + head) * HD;
#pragma unroll
        for (int d = 0; d < HD_TILES; ++d)
#pragma unroll
            for (int i = 0; i < 4; ++i) out_row[d * 16 + quad * 4 + i] = from_float<bf16>(o_acc[d][i] * inverse);
    }
}

template <int HD_TILES>
static int launch_prefill(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_table,
                          int table_width, const int32_t* tiles, int n_tiles, const int32_t* positions, void* out,
                          float scale, int window, int heads, int kv_heads, int page_size, hipStream_t stream) {
    const dim3 grid(n_tiles, heads);
    paged_attention_prefill_kernel<HD_TILES><<<grid, kPrefillThreads, 0, stream>>>(
        static_cast<const bf16*>(q), static_cast<const bf16*>(k_cache), static_cast<const bf16*>(v_cache), block_table,
        table_width, tiles, positions, static_cast<bf16*>(out), scale, window, heads, kv_heads, page_size);
    return check_launch("paged_attention_prefill");
}

}  // namespace mll

using namespace mll;

extern "C" int mll_paged_attention_prefill_tile() { return kPrefillTile; }

extern "C" int mll_paged_attention_prefill(const void* q, const void* k_cache, const void* v_cache,
                                           const int32_t* block_table, int table_width, const int32_t* tiles,
                                           int n_tiles, const int32_t* positions, void* out, float scale, int window,
                                           int heads, int kv_heads, int head_dim, int page_size, hipStream_t stream) {
    MLL_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "paged_attention_prefill: heads must divide into kv_heads groups");
    MLL_REQUIRE(head_dim % 16 == 0 && head_dim >= 16 && head_dim <= 256,
                "paged_attention_prefill: head_dim must be a multiple of 16 in [16, 256]");
    MLL_REQUIRE(page_size > 0 && page_size % 16 == 0, "paged_attention_prefill: page_size must be a multiple of 16");
    MLL_REQUIRE(heads <= 65535, "paged_attention_prefill: more than 65535 heads");
    if (n_tiles == 0) return 0;
#define MLL_PREFILL_CASE(TILES)                                                                                      \
    case TILES:                                                                                                      \
        return launch_prefill<TILES>(q, k_cache, v_cache, block_table, table_width, tiles, n_tiles, positions, out,  \
                                     scale, window, heads, kv_heads, page_size, stream);
    switch (head_dim / 16) {
        MLL_PREFILL_CASE(1) MLL_PREFILL_CASE(2) MLL_PREFILL_CASE(3) MLL_PREFILL_CASE(4) MLL_PREFILL_CASE(5)
        MLL_PREFILL_CASE(6) MLL_PREFILL_CASE(7) MLL_PREFILL_CASE(8) MLL_PREFILL_CASE(9) MLL_PREFILL_CASE(10)
        MLL_PREFILL_CASE(11) MLL_PREFILL_CASE(12) MLL_PREFILL_CASE(13) MLL_PREFILL_CASE(14) MLL_PREFILL_CASE(15)
        MLL_PREFILL_CASE(16)
        default: return fail("paged_attention_prefill: unsupported head_dim");
    }
#undef MLL_PREFILL_CASE
}
