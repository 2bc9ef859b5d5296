// Paged attention for portions of prompts in bfloat16: MFMA for both products, online softmax in float32.
//
// A workgroup (4 waves) takes up to 128 consecutive tokens of one request's portion and one query head; a wave
// takes 32 of them as two blocks of 16 columns. The workgroup walks the keys its tokens can see in blocks of
// 64 (32 for head sizes above 128): the block's key and value tiles are copied from the pages into LDS as they
// lie there (the pages are in MFMA order, cache_layout.h), the next block's being fetched from memory while
// this one is used. As in the decode kernel, scores are computed transposed, S^T = K . Q^T, the 16 columns
// being query positions, and O^T = V^T . P^T follows from registers; every fragment of K and V read from LDS
// serves both column blocks. Only pairs of tiles that touch the causal diagonal or the window's edge pay
// for the mask (they run a second instance of the inner loop's body), and values that no token of the
// workgroup can see are cleared once, on their way into LDS, so that stale memory never meets a zero weight.
// The vector unit, not the MFMA, bounds this kernel: the scale is folded into the exponent's multiply-add and
// the accumulators are rescaled only when some maximum has moved.
// The list of tiles (request, first token in the flat list, tokens) is built on the host.
#include <type_traits>

#include "cache_layout.h"
#include "common.h"
#include "microllm_hip.h"

namespace mll {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kPrefillWaves = 4;
constexpr int kPrefillThreads = kPrefillWaves * kWave;
constexpr int kPrefillWaveTokens = 32;
constexpr int kPrefillTile = kPrefillWaveTokens * kPrefillWaves;   // tokens per workgroup

union PFrag8 {
    bf16x8 v;
    bf16x4 h[2];
    uint4 raw;
};

template <int HD_TILES>
__global__ __launch_bounds__(kPrefillThreads, 2) void paged_attention_prefill_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ tiles,
    const int32_t* __restrict__ positions, bf16* __restrict__ out, float scale, int window, int heads,
    int kv_heads, int page_size) {
    constexpr int HD = HD_TILES * 16;
    constexpr int K_STEPS = (HD + 31) / 32;
    constexpr int K_CHUNKS = HD / 8;
    constexpr int BLOCK_KEYS = HD <= 128 ? 64 : 32;
    constexpr int BLOCK_TILES = BLOCK_KEYS / 16;
    constexpr int TILE_ELEMENTS = HD * 16;                       // of keys and of values alike
    constexpr int TILE_PASSES = (TILE_ELEMENTS * 2 + kPrefillThreads * 16 - 1) / (kPrefillThreads * 16);
    extern __shared__ __align__(16) bf16 lds[];                  // [2 stages][K | V][BLOCK_TILES][TILE_ELEMENTS]
    constexpr int STAGE_ELEMENTS = 2 * BLOCK_TILES * TILE_ELEMENTS;

    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int col = lane % 16;
    const int quad = lane / 16;

    const int seq = tiles[3 * blockIdx.x + 0];
    const int tile_token = tiles[3 * blockIdx.x + 1];
    const int tile_count = tiles[3 * blockIdx.x + 2];
    const int head = blockIdx.y;
    const int kv_head = head / (heads / kv_heads);
    const int32_t* table = block_table + static_cast<int64_t>(seq) * table_width;
    const CacheLayout layout(kv_heads, page_size, HD);
    const float scale_log2 = scale * 1.4426950408889634f;      // scores are kept in units of log 2: p = 2^(s - max)

    // The workgroup's tokens and the keys any of them can see.
    const int tile_position = positions[tile_token];             // tokens of a portion have consecutive positions
    const int group_last = tile_position + tile_count - 1;
    const int group_low = window > 0 ? max(0, tile_position - window + 1) : 0;
    // This wave's tokens.
    const int wave_first = wave * kPrefillWaveTokens;
    const int wave_valid = min(kPrefillWaveTokens, max(0, tile_count - wave_first));
    const int column_blocks = (wave_valid + 15) / 16;
    const int wave_position = tile_position + wave_first;
    const int wave_last = wave_position + wave_valid - 1;
    const int wave_low = window > 0 ? max(0, wave_position - window + 1) : 0;
    const int wave_last_low = window > 0 ? max(0, wave_last - window + 1) : 0;

    PFrag8 q_frag[2][K_STEPS];
    int my_position[2], my_low[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const int valid = min(16, max(0, wave_valid - 16 * c));
        const int index = wave_first + 16 * c + min(col, max(valid - 1, 0));      // columns past the end repeat the last token
        my_position[c] = tile_position + index;
        my_low[c] = window > 0 ? max(0, my_position[c] - window + 1) : 0;
#pragma unroll
        for (int ks = 0; ks < K_STEPS; ++ks) {
            const int dim = ks * 32 + quad * 8;
            q_frag[c][ks].raw = make_uint4(0, 0, 0, 0);
            if (valid > 0 && dim < HD)
                q_frag[c][ks].raw = *reinterpret_cast<const uint4*>(
                    q + (static_cast<int64_t>(tile_token + index) * heads + head) * HD + dim);
        }
    }

    floatx4 o_acc[2][HD_TILES];
    float running_max[2] = {-INFINITY, -INFINITY}, running_sum[2] = {0.0f, 0.0f};
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int d = 0; d < HD_TILES; ++d) o_acc[c][d] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

    // Copy of one block's tiles: thread i moves bytes [16 i, 16 i + 16) of every pass of every tile.
    uint4 staged[BLOCK_TILES][2][TILE_PASSES];
    int staged_block = 0;
    // The page of a tile: pages hold tiles_per_page tiles of 16 positions (often one, mostly a power of two).
    const int tiles_per_page = page_size / 16;
    const int page_shift = (tiles_per_page & (tiles_per_page - 1)) == 0 ? __ffs(tiles_per_page) - 1 : -1;
    auto fetch_tile = [&](int t, int tile_key, bool live) {
        const int tile_index = tile_key / 16;
        const int slot = page_shift >= 0 ? tile_index >> page_shift : tile_index / tiles_per_page;
        const int tile_in_page = tile_index - slot * tiles_per_page;
        const int64_t page = live ? table[slot] : 0;
        const bf16* k_tile = k_cache + layout.k_tile(page, kv_head, tile_in_page);
        const bf16* v_tile = v_cache + layout.v_tile(page, kv_head, tile_in_page);
#pragma unroll
        for (int pass = 0; pass < TILE_PASSES; ++pass) {
            const int element = (pass * kPrefillThreads + threadIdx.x) * 8;
            staged[t][0][pass] = make_uint4(0, 0, 0, 0);
            staged[t][1][pass] = make_uint4(0, 0, 0, 0);
            if (live && element < TILE_ELEMENTS) {
                staged[t][0][pass] = *reinterpret_cast<const uint4*>(k_tile + element);
                staged[t][1][pass] = *reinterpret_cast<const uint4*>(v_tile + element);
            }
        }
    };
    // A block all of whose keys some token of the workgroup can see (most blocks) needs no checks per tile.
    auto inside = [&](int block) { return block * BLOCK_KEYS >= group_low && block * BLOCK_KEYS + BLOCK_KEYS - 1 <= group_last; };
    auto fetch = [&](int block) {
        staged_block = block;
        if (inside(block)) {
#pragma unroll
            for (int t = 0; t < BLOCK_TILES; ++t) fetch_tile(t, block * BLOCK_KEYS + 16 * t, true);
        } else {
#pragma unroll
            for (int t = 0; t < BLOCK_TILES; ++t) {
                const int tile_key = block * BLOCK_KEYS + 16 * t;
                fetch_tile(t, tile_key, tile_key <= group_last && tile_key + 15 >= group_low);
            }
        }
    };
    auto stash = [&](int stage) {
        bf16* base = lds + stage * STAGE_ELEMENTS;
        if (!inside(staged_block)) {
#pragma unroll
            for (int t = 0; t < BLOCK_TILES; ++t) {
                // A tile that straddles an end of what the workgroup's tokens can see holds positions that may be
                // stale memory: their values are cleared here (their scores are masked where they are computed).
                const int tile_key = staged_block * BLOCK_KEYS + 16 * t;
                if (tile_key <= group_last && tile_key + 15 >= group_low && (tile_key + 15 > group_last || tile_key < group_low)) {
#pragma unroll
                    for (int pass = 0; pass < TILE_PASSES; ++pass) {
                        const int element = (pass * kPrefillThreads + threadIdx.x) * 8;   // 2 dims x positions 4 g .. 4 g + 3
                        const int first_key = tile_key + 4 * ((element / 64) % 4);
                        PFrag8 values;
                        values.raw = staged[t][1][pass];
#pragma unroll
                        for (int i = 0; i < 8; ++i)
                            if (first_key + i % 4 > group_last || first_key + i % 4 < group_low) values.v[i] = static_cast<__bf16>(0.0f);
                        staged[t][1][pass] = values.raw;
                    }
                }
            }
        }
#pragma unroll
        for (int t = 0; t < BLOCK_TILES; ++t)
#pragma unroll
            for (int pass = 0; pass < TILE_PASSES; ++pass) {
                const int element = (pass * kPrefillThreads + threadIdx.x) * 8;
                if (element < TILE_ELEMENTS) {
                    *reinterpret_cast<uint4*>(base + t * TILE_ELEMENTS + element) = staged[t][0][pass];
                    *reinterpret_cast<uint4*>(base + (BLOCK_TILES + t) * TILE_ELEMENTS + element) = staged[t][1][pass];
                }
            }
    };

    // One pair of key tiles (32 keys) against the wave's 32 tokens. MASKED: some key of the pair is hidden from
    // some token of the wave (the causal diagonal, the window's edge, the end of the sequence).
    // Scores stay in the product's units; p = 2^((s - max) * scale_log2) is one multiply-add and one exponent.
    auto process_pair = [&](auto masked_tag, const bf16* k_lds, const bf16* v_lds, int pair, int key0) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        PFrag8 k_frag[2][K_STEPS];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int ks = 0; ks < K_STEPS; ++ks) {
                const int piece = ks * 4 + quad;
                k_frag[t][ks].raw = make_uint4(0, 0, 0, 0);
                if (piece < K_CHUNKS)
                    k_frag[t][ks].raw = *reinterpret_cast<const uint4*>(
                        k_lds + (2 * pair + t) * TILE_ELEMENTS + piece * 128 + col * 8);
            }
        PFrag8 p_frag[2];
        float rescale[2];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            if (c >= column_blocks) {
                p_frag[c].raw = make_uint4(0, 0, 0, 0);
                rescale[c] = 1.0f;
                continue;
            }
            float score[8];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                floatx4 s = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int ks = 0; ks < K_STEPS; ++ks)
                    s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k_frag[t][ks].v, q_frag[c][ks].v, s, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; ++i) score[4 * t + i] = s[i];
            }
            if (MASKED) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int key = key0 + 16 * (j / 4) + 4 * quad + (j % 4);
                    if (key > my_position[c] || key < my_low[c]) score[j] = -INFINITY;
                }
            }
            float tile_max = score[0];
#pragma unroll
            for (int j = 1; j < 8; ++j) tile_max = fmaxf(tile_max, score[j]);
            tile_max = max_lanes_16_apart(tile_max);
            const float new_max = fmaxf(running_max[c], tile_max);
            // A query may see nothing of a pair that others see (the window's edge): its maximum stays -inf.
            const float safe_max = (MASKED && new_max == -INFINITY) ? 0.0f : new_max;
            const float offset = -safe_max * scale_log2;
            rescale[c] = __builtin_amdgcn_exp2f(fmaf(running_max[c], scale_log2, offset));
            float tile_sum = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float p = __builtin_amdgcn_exp2f(fmaf(score[j], scale_log2, offset));
                tile_sum += p;
                p_frag[c].v[j] = static_cast<__bf16>(p);
            }
            tile_sum = sum_lanes_16_apart(tile_sum);
            running_sum[c] = running_sum[c] * rescale[c] + tile_sum;
            running_max[c] = new_max;
        }
        // Once the running maxima have settled, no column's sum needs rescaling: one branch for the whole wave.
        if (__any(rescale[0] != 1.0f || rescale[1] != 1.0f)) {
#pragma unroll
            for (int c = 0; c < 2; ++c)
#pragma unroll
                for (int d = 0; d < HD_TILES; ++d) o_acc[c][d] *= rescale[c];
        }
#pragma unroll
        for (int d = 0; d < HD_TILES; ++d) {
            PFrag8 v_frag;
#pragma unroll
            for (int t = 0; t < 2; ++t)
                v_frag.h[t] = *reinterpret_cast<const bf16x4*>(
                    v_lds + (2 * pair + t) * TILE_ELEMENTS + d * 256 + (quad * 16 + col) * 4);
#pragma unroll
            for (int c = 0; c < 2; ++c)
                o_acc[c][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_frag.v, p_frag[c].v, o_acc[c][d], 0, 0, 0);
        }
    };

    const int first_block = group_low / BLOCK_KEYS;
    const int last_block = group_last / BLOCK_KEYS;
    fetch(first_block);
    stash(0);
    __syncthreads();
    for (int block = first_block; block <= last_block; ++block) {
        const int stage = (block - first_block) & 1;
        if (block < last_block) fetch(block + 1);
        const bf16* k_lds = lds + stage * STAGE_ELEMENTS;
        const bf16* v_lds = k_lds + BLOCK_TILES * TILE_ELEMENTS;

        if (wave_valid > 0) {
#pragma unroll
            for (int pair = 0; pair < BLOCK_TILES / 2; ++pair) {
                const int key0 = block * BLOCK_KEYS + 32 * pair;
                if (key0 > wave_last || key0 + 31 < wave_low) continue;   // nothing of this pair is visible to the wave
                if (key0 + 31 > wave_position || key0 < wave_last_low) process_pair(std::true_type{}, k_lds, v_lds, pair, key0);
                else process_pair(std::false_type{}, k_lds, v_lds, pair, key0);
            }
        }
        if (block < last_block) stash(stage ^ 1);
        __syncthreads();
    }

#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const int valid = min(16, max(0, wave_valid - 16 * c));
        if (col < valid) {
            const float inverse = 1.0f / running_sum[c];
            bf16* out_row = out + (static_cast<int64_t>(tile_token + wave_first + 16 * c + col) * heads + head) * HD;
#pragma unroll
            for (int d = 0; d < HD_TILES; ++d) {
                bf16x4 four;
#pragma unroll
                for (int i = 0; i < 4; ++i) four[i] = static_cast<__bf16>(o_acc[c][d][i] * inverse);
                *reinterpret_cast<bf16x4*>(out_row + d * 16 + quad * 4) = four;
            }
        }
    }
}

template <int HD_TILES>
static int launch_prefill(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_table,
                          int table_width, const int32_t* tiles, int n_tiles, const int32_t* positions, void* out,
                          float scale, int window, int heads, int kv_heads, int page_size, hipStream_t stream) {
    constexpr int HD = HD_TILES * 16;
    constexpr int BLOCK_KEYS = HD <= 128 ? 64 : 32;
    const size_t lds_bytes = 2 * 2 * (BLOCK_KEYS / 16) * HD * 16 * sizeof(bf16);   // at most 64 KB
    const dim3 grid(n_tiles, heads);
    paged_attention_prefill_kernel<HD_TILES><<<grid, kPrefillThreads, lds_bytes, stream>>>(
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
