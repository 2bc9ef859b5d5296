// Paged attention for portions of prompts in bfloat16: MFMA for both products, online softmax in float32.
//
// A workgroup (8 waves) takes two tiles of up to 128 consecutive tokens each, of one request's portion and one
// query head. A wave takes two blocks of 16 tokens (16 columns of the MFMA): 16 tokens of the first tile and 16 of
// the second. The host pairs a tile that sees many keys with one that sees few, so that every workgroup walks
// about as many keys and the compute units finish together (under a causal mask the last tile of a prompt has
// as many times the work of the first as there are tiles); both tiles read the same keys from LDS, and every
// wave has work to the end of the longer walk. The second tile may be empty: then waves 0-3 take 32 consecutive
// tokens each.
// The workgroup walks the keys its tokens can see in blocks of 128 (64 for head sizes above 128): the block's key
// and value tiles are copied from the pages straight into LDS as they lie there (the pages are in MFMA order,
// cache_layout.h), the next block's being on its way while this one is used. The two stages are two LDS
// variables, so that the compiler need not wait for a load into one before it reads the other. As in the decode
// kernel, scores are computed transposed, S^T = K . Q^T, the 16 columns being query positions, and
// O^T = V^T . P^T follows from registers; every fragment of K and V read from LDS serves both column blocks.
// Only pairs of key tiles that touch the causal diagonal or the window's edge pay for the mask (they run a second
// instance of the inner loop's body), and values that no token of the workgroup can see are cleared in LDS before
// a block at an end of the walk is used, so that stale memory never meets a zero weight.
// The vector unit and the reads from LDS, not the MFMA, bound this kernel: the scale is folded into the exponent's
// multiply-add and the accumulators are rescaled only when some maximum has moved.
// The list of workgroups (request; first token in the flat list and tokens, for either tile) is built on the host.
#include <type_traits>

#include "cache_layout.h"
#include "common.h"
#include "microllm_hip.h"

namespace mll {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kPrefillWaves = 8;
constexpr int kPrefillThreads = kPrefillWaves * kWave;
constexpr int kPrefillTile = 16 * kPrefillWaves;   // tokens of one tile; a workgroup takes two tiles

union PFrag8 {
    bf16x8 v;
    bf16x4 h[2];
    uint4 raw;
};

template <int HD_TILES>
__global__ __launch_bounds__(kPrefillThreads, 1) void paged_attention_prefill_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ tiles,
    const int32_t* __restrict__ positions, bf16* __restrict__ out, float scale, int window, int heads,
    int kv_heads, int page_size) {
    constexpr int HD = HD_TILES * 16;
    constexpr int K_STEPS = (HD + 31) / 32;
    constexpr int K_CHUNKS = HD / 8;
    constexpr int BLOCK_KEYS = HD <= 128 ? 128 : 64;
    constexpr int BLOCK_TILES = BLOCK_KEYS / 16;
    constexpr int TILE_ELEMENTS = HD * 16;                       // of keys and of values alike
    constexpr int TILE_CHUNKS = TILE_ELEMENTS / 8;               // pieces of 16 bytes
    constexpr int STAGE_ELEMENTS = 2 * BLOCK_TILES * TILE_ELEMENTS;
    // Two stages of [K | V][BLOCK_TILES][TILE_ELEMENTS]. They are two variables, not one array: the compiler then
    // knows that a load into one stage does not write what is read from the other, and lets the two overlap.
    __shared__ __align__(16) bf16 stage_even[STAGE_ELEMENTS];
    __shared__ __align__(16) bf16 stage_odd[STAGE_ELEMENTS];

    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int col = lane % 16;
    const int quad = lane / 16;

    const int32_t* entry = tiles + 5 * blockIdx.x;
    const int seq = entry[0];
    const int head = blockIdx.y;
    const int kv_head = head / (heads / kv_heads);
    const int32_t* table = block_table + static_cast<int64_t>(seq) * table_width;
    const float scale_log2 = scale * 1.4426950408889634f;      // scores are kept in units of log 2: p = 2^(s - max)

    // Either tile's tokens and the keys any of them can see (tokens of a portion have consecutive positions);
    // an empty tile sees nothing: no key lies in its range.
    int range_low[2], range_last[2];
#pragma unroll
    for (int side = 0; side < 2; ++side) {
        const int count = entry[2 + 2 * side];
        const int position = count > 0 ? positions[entry[1 + 2 * side]] : 0;
        range_last[side] = count > 0 ? position + count - 1 : -1;
        range_low[side] = count > 0 ? (window > 0 ? max(0, position - window + 1) : 0) : (1 << 30);
    }
    const int group_low = min(range_low[0], range_low[1]);
    const int group_last = max(range_last[0], range_last[1]);
    auto seen = [&](int key) {      // by some token of the workgroup
        return (key >= range_low[0] && key <= range_last[0]) || (key >= range_low[1] && key <= range_last[1]);
    };
    auto tile_seen = [&](int tile_key) {      // some of its 16 keys
        return (tile_key + 15 >= range_low[0] && tile_key <= range_last[0]) || (tile_key + 15 >= range_low[1] && tile_key <= range_last[1]);
    };
    // A block all of whose keys one tile's tokens can see (most blocks) needs no checks per key tile.
    auto inside = [&](int block) {
        const int first = block * BLOCK_KEYS, last = first + BLOCK_KEYS - 1;
        return (first >= range_low[0] && last <= range_last[0]) || (first >= range_low[1] && last <= range_last[1]);
    };
    // A block of which nothing is seen (between the two tiles' windows) is passed over.
    auto block_seen = [&](int block) {
        const int first = block * BLOCK_KEYS, last = first + BLOCK_KEYS - 1;
        return (last >= range_low[0] && first <= range_last[0]) || (last >= range_low[1] && first <= range_last[1]);
    };

    // This wave's two blocks of 16 columns. With two tiles in the workgroup the first block is 16 tokens of the
    // first tile and the second 16 tokens of the second: every wave then walks the keys of both, and the waves of
    // a compute unit stay busy together to the end of the longer walk. With one tile, waves 0 to 3 take 32
    // consecutive tokens each.
    const bool two_tiles = entry[2] > 0 && entry[4] > 0;
    const int only_side = entry[2] > 0 ? 0 : 1;
    int block_token[2], block_valid[2], block_position[2], block_last[2], block_low[2], block_last_low[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const int side = two_tiles ? c : only_side;
        const int first = 16 * (two_tiles ? wave : 2 * wave + c);          // in the tile
        const int count = entry[2 + 2 * side];
        block_token[c] = entry[1 + 2 * side] + first;
        block_valid[c] = min(16, max(0, count - first));
        block_position[c] = (block_valid[c] > 0 ? positions[entry[1 + 2 * side]] : 0) + first;
        block_last[c] = block_position[c] + block_valid[c] - 1;
        block_low[c] = window > 0 ? max(0, block_position[c] - window + 1) : 0;        // the lowest key its first token sees
        block_last_low[c] = window > 0 ? max(0, block_last[c] - window + 1) : 0;       // and its last token
    }

    PFrag8 q_frag[2][K_STEPS];
    int my_position[2], my_low[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const int valid = block_valid[c];
        const int index = min(col, max(valid - 1, 0));      // columns past the end repeat the last token
        my_position[c] = block_position[c] + index;
        my_low[c] = window > 0 ? max(0, my_position[c] - window + 1) : 0;
#pragma unroll
        for (int ks = 0; ks < K_STEPS; ++ks) {
            const int dim = ks * 32 + quad * 8;
            q_frag[c][ks].raw = make_uint4(0, 0, 0, 0);
            if (valid > 0 && dim < HD)
                q_frag[c][ks].raw = *reinterpret_cast<const uint4*>(
                    q + (static_cast<int64_t>(block_token[c] + index) * heads + head) * HD + dim);
        }
    }

    floatx4 o_acc[2][HD_TILES];
    float running_max[2] = {-INFINITY, -INFINITY}, running_sum[2] = {0.0f, 0.0f};
    float running_offset[2] = {0.0f, 0.0f};      // -(running maximum) in units of log 2; 0 while the maximum is -inf
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int d = 0; d < HD_TILES; ++d) o_acc[c][d] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

    // Copy of one block's tiles, from the pages straight into LDS (no registers in between): a wave moves 64
    // consecutive pieces of 16 bytes of the block's key tiles as they lie in LDS, piece pass * threads + thread,
    // and the pieces of the value tiles at the same places. Where a wave's lanes stay within one tile (head
    // sizes in steps of 32) the tile, its page and its address are the same for the whole wave and are worked
    // out by the scalar unit.
    constexpr bool UNIFORM = TILE_CHUNKS % kWave == 0;
    constexpr int HALF_CHUNKS = BLOCK_TILES * TILE_CHUNKS;
    constexpr int PASSES = (HALF_CHUNKS + kPrefillThreads - 1) / kPrefillThreads;
    // The page of a tile: pages hold tiles_per_page tiles of 16 positions (often one, mostly a power of two).
    const int tiles_per_page = page_size / 16;
    const int page_shift = (tiles_per_page & (tiles_per_page - 1)) == 0 ? __ffs(tiles_per_page) - 1 : -1;
    const int64_t page_elements = static_cast<int64_t>(kv_heads) * tiles_per_page * TILE_ELEMENTS;
    const int head_elements = kv_head * tiles_per_page * TILE_ELEMENTS;
    const int wave_chunk = __builtin_amdgcn_readfirstlane(wave) * kWave;      // the wave's first piece of pass 0
    auto tile_of = [&](int pass) { return (pass * kPrefillThreads + wave_chunk + (UNIFORM ? 0 : lane)) / TILE_CHUNKS; };   // in the block
    auto piece_of = [&](int pass) { return (pass * kPrefillThreads + wave_chunk + (UNIFORM ? 0 : lane)) % TILE_CHUNKS + (UNIFORM ? lane : 0); };
    auto wanted = [&](int block, int pass) {      // whether the tile is brought in: some token sees some of it
        const int tile_key = block * BLOCK_KEYS + 16 * tile_of(pass);
        return tile_of(pass) < BLOCK_TILES && tile_key <= group_last && (inside(block) || tile_seen(tile_key));
    };
    // The pages of a block's tiles are looked up one block ahead of the tiles themselves, so that no load waits
    // for another. The look-up is a load of the vector unit also where the whole wave asks for one entry: those
    // are counted with the loads into LDS and have arrived when these have, whereas a load of the scalar unit
    // would be waited for by the first read from LDS that follows it.
    int pages[PASSES];
    int no_lane = 0;
    asm volatile("v_mov_b32 %0, 0" : "=v"(no_lane));      // zero, but the compiler cannot tell: keeps the address per lane
    auto look_up = [&](int block) {
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            const int tile_index = block * BLOCK_TILES + tile_of(pass);
            pages[pass] = -1;
            if (wanted(block, pass))
                pages[pass] = table[(page_shift >= 0 ? tile_index >> page_shift : tile_index / tiles_per_page) + no_lane];
        }
    };
    auto fetch = [&](int block, bf16* stage) {      // after look_up(block)
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            const int tile_index = block * BLOCK_TILES + tile_of(pass);
            const int tile_in_page = page_shift >= 0 ? tile_index & (tiles_per_page - 1) : tile_index % tiles_per_page;
            const int page = UNIFORM ? __builtin_amdgcn_readfirstlane(pages[pass]) : pages[pass];
            if (page >= 0) {
                const int64_t tile_start = page * page_elements + head_elements + tile_in_page * TILE_ELEMENTS;
                const bf16* key_piece = k_cache + tile_start + piece_of(pass) * 8;
                const bf16* value_piece = v_cache + tile_start + piece_of(pass) * 8;
                bf16* key_place = stage + (pass * kPrefillThreads + wave_chunk) * 8;      // the lane's 16 bytes follow by themselves
                bf16* value_place = key_place + HALF_CHUNKS * 8;
                __builtin_amdgcn_global_load_lds(key_piece, key_place, 16, 0, 0);
                __builtin_amdgcn_global_load_lds(value_piece, value_place, 16, 0, 0);
            }
        }
    };
    // A block at an end of what the workgroup's tokens see, once it lies in LDS: values at positions that no
    // token sees may be stale memory, and the places of tiles that were not brought in hold what was there
    // before. Both are cleared (their scores are masked where they are computed).
    auto clear_unseen = [&](int block, bf16* stage) {
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            if (tile_of(pass) >= BLOCK_TILES) continue;
            uint4* place = reinterpret_cast<uint4*>(stage + HALF_CHUNKS * 8 + (tile_of(pass) * TILE_CHUNKS + piece_of(pass)) * 8);
            PFrag8 values;
            values.raw = make_uint4(0, 0, 0, 0);
            if (wanted(block, pass)) {
                values.raw = *place;
                const int element = piece_of(pass) * 8;      // 2 dims x positions 4 g .. 4 g + 3
                const int first_key = block * BLOCK_KEYS + 16 * tile_of(pass) + 4 * ((element / 64) % 4);
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (!seen(first_key + i % 4)) values.v[i] = static_cast<__bf16>(0.0f);
            }
            *place = values.raw;
        }
    };
    // The wave's loads into LDS have landed (the compiler does not wait for loads that return nothing), and so
    // have everyone's; everyone is done with the stage that is written next.
    auto landed = [&](int block, bf16* stage) {
        wait_for_loads();
        __syncthreads();
        if (block <= group_last / BLOCK_KEYS && !inside(block)) {
            clear_unseen(block, stage);
            __syncthreads();
        }
    };
    auto next_seen = [&](int block) {      // the next block after this one of which something is seen
        ++block;
        while (block * BLOCK_KEYS <= group_last && !block_seen(block)) ++block;
        return block;
    };

    // One pair of key tiles (32 keys) against the wave's two blocks of 16 tokens; see0 / see1: whether the block
    // sees any of the pair. MASKED: some key of the pair is hidden from some token of a block that sees the pair
    // (the causal diagonal, the window's edge, the end of the sequence).
    // Scores stay in the product's units; p = 2^((s - max) * scale_log2) is one multiply-add and one exponent.
    auto process_pair = [&](auto masked_tag, const bf16* k_lds, const bf16* v_lds, int pair, int key0, bool see0, bool see1) {
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
            if (!(c == 0 ? see0 : see1)) {
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
            // Far into a prompt a pair rarely holds a new maximum for any of the wave's tokens: then the four
            // lanes of a token need not compare notes, and nothing is rescaled (the same numbers either way).
            rescale[c] = 1.0f;
            if (__any(tile_max > running_max[c])) {
                tile_max = max_lanes_16_apart(tile_max);
                const float new_max = fmaxf(running_max[c], tile_max);
                // A query may see nothing of a pair that others see (the window's edge): its maximum stays -inf.
                const float safe_max = (MASKED && new_max == -INFINITY) ? 0.0f : new_max;
                running_offset[c] = -safe_max * scale_log2;
                // exactly 1 for a token whose maximum stays (the rounding of maximum * scale would else leave a factor
                // of 1 +- 1e-7, and every sum would be multiplied by it)
                rescale[c] = new_max == running_max[c] ? 1.0f : __builtin_amdgcn_exp2f(fmaf(running_max[c], scale_log2, running_offset[c]));
                running_max[c] = new_max;
            }
            const float offset = running_offset[c];
            float tile_sum = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float p = __builtin_amdgcn_exp2f(fmaf(score[j], scale_log2, offset));
                tile_sum += p;
                p_frag[c].v[j] = static_cast<__bf16>(p);
            }
            tile_sum = sum_lanes_16_apart(tile_sum);
            running_sum[c] = running_sum[c] * rescale[c] + tile_sum;
        }
        // Once the running maxima have settled, no column's sum needs rescaling: one branch for the whole wave.
        if (__any(rescale[0] != 1.0f || rescale[1] != 1.0f)) {
#pragma unroll
            for (int c = 0; c < 2; ++c)
#pragma unroll
                for (int d = 0; d < HD_TILES; ++d) o_acc[c][d] *= rescale[c];
        }
        auto values_times_weights = [&](auto first_tag, auto second_tag) {
#pragma unroll
            for (int d = 0; d < HD_TILES; ++d) {
                PFrag8 v_frag;
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    v_frag.h[t] = *reinterpret_cast<const bf16x4*>(
                        v_lds + (2 * pair + t) * TILE_ELEMENTS + d * 256 + (quad * 16 + col) * 4);
                if (decltype(first_tag)::value)
                    o_acc[0][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_frag.v, p_frag[0].v, o_acc[0][d], 0, 0, 0);
                if (decltype(second_tag)::value)
                    o_acc[1][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_frag.v, p_frag[1].v, o_acc[1][d], 0, 0, 0);
            }
        };
        if (see0 && see1) values_times_weights(std::true_type{}, std::true_type{});
        else if (see0) values_times_weights(std::true_type{}, std::false_type{});
        else values_times_weights(std::false_type{}, std::true_type{});
    };

    const int first_block = group_low / BLOCK_KEYS;
    const int last_block = group_last / BLOCK_KEYS;
    // One block: the next one is sent for, this one is used. Called by turns with the stages exchanged.
    int block = first_block;
    int following = next_seen(first_block);
    auto walk = [&](const bf16* stage, bf16* next_stage) {
        if (following <= last_block) {
            fetch(following, next_stage);
            const int after = next_seen(following);
            if (after <= last_block) look_up(after);
        }
        const bf16* k_lds = stage;
        const bf16* v_lds = stage + HALF_CHUNKS * 8;
#pragma unroll 1
        for (int pair = 0; pair < BLOCK_TILES / 2; ++pair) {
            const int key0 = block * BLOCK_KEYS + 32 * pair;
            bool see[2], hidden = false;
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                see[c] = block_valid[c] > 0 && key0 <= block_last[c] && key0 + 31 >= block_low[c];
                hidden = hidden || (see[c] && (key0 + 31 > block_position[c] || key0 < block_last_low[c]));
            }
            if (!see[0] && !see[1]) continue;      // nothing of this pair is visible to the wave
            if (hidden) process_pair(std::true_type{}, k_lds, v_lds, pair, key0, see[0], see[1]);
            else process_pair(std::false_type{}, k_lds, v_lds, pair, key0, see[0], see[1]);
        }
        landed(following, next_stage);
        block = following;
        following = next_seen(block);
    };
    look_up(first_block);
    fetch(first_block, stage_even);
    if (following <= last_block) look_up(following);
    landed(first_block, stage_even);
    while (block <= last_block) {
        walk(stage_even, stage_odd);
        if (block > last_block) break;
        walk(stage_odd, stage_even);
    }

#pragma unroll
    for (int c = 0; c < 2; ++c) {
        if (col < block_valid[c]) {
            const float inverse = 1.0f / running_sum[c];
            bf16* out_row = out + (static_cast<int64_t>(block_token[c] + col) * heads + head) * HD;
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
    constexpr int BLOCK_KEYS = HD <= 128 ? 128 : 64;
    const dim3 grid(n_tiles, heads);   // n_tiles: workgroups, of two tiles each
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
