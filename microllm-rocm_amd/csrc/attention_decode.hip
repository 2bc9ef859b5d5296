// Paged attention for single query tokens (decoding) in bfloat16: split over the keys, MFMA for both
// products, online softmax in float32, a second kernel that joins the splits.
//
// One workgroup (4 waves) takes one token, one kv head (with up to 16 of its query heads) and one split
// of the visible keys. A wave walks pairs of 16-key tiles. Scores are computed transposed,
// S^T = K . Q^T (v_mfma_f32_16x16x32_bf16: A = 16 keys x 32 dims straight from the page, B = Q^T), so
// that a lane ends up with 8 keys of one head: exactly the B operand of O^T = V^T . P^T, whose A operand
// comes straight from the value pages. Pages are laid out in MFMA order (cache_layout.h), so every load of
// a wave is one contiguous piece. Nothing passes through LDS but the final join of the 4 waves.
#include "cache_layout.h"
#include "common.h"
#include "microllm_hip.h"

namespace mll {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kDecodeWaves = 4;
constexpr int kDecodeThreads = kDecodeWaves * kWave;

typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

// 16 bytes of keys or values. STREAM: read past the caches (nothing is read twice): with a workgroup or more per
// compute unit the pages then come in at 6.4 instead of 5.6 TB/s (64 requests of 4096 positions, 8 of 32000); with
// fewer workgroups it is slower (128 workgroups: 41 -> 64 us), so the launch decides.
template <bool STREAM>
__device__ inline uint4 load_piece(const bf16* from) {
    if (STREAM) {
        const uintx4 piece = __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(from));
        return make_uint4(piece[0], piece[1], piece[2], piece[3]);
    }
    return *reinterpret_cast<const uint4*>(from);
}

union Frag8 {
    bf16x8 v;
    bf16x4 h[2];
    uint4 raw;
};

template <int HD_TILES, bool STREAM>
__global__ __launch_bounds__(kDecodeThreads) void paged_attention_decode_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ token_ids, bf16* __restrict__ out,
    float* __restrict__ part_o, float* __restrict__ part_ml, float scale, int window, int heads, int kv_heads,
    int page_size, int n_splits) {
    constexpr int HD = HD_TILES * 16;
    constexpr int K_STEPS = (HD + 31) / 32;
    constexpr int K_CHUNKS = HD / 8;
    // Join buffer: one slot per wave when it fits, else one slot that the waves enter in turn.
    constexpr bool kParallelJoin = HD_TILES <= 8;
    constexpr int kSlots = kParallelJoin ? kDecodeWaves : 1;
    __shared__ float o_shared[kSlots][16][HD + 4];
    __shared__ float m_shared[kSlots][16];
    __shared__ float l_shared[kSlots][16];

    const int token = token_ids ? token_ids[blockIdx.x] : blockIdx.x;   // a step may give the kernel some of its tokens only
    if (token < 0) return;      // an entry that only pads the list to a fixed length
    const int group = heads / kv_heads;
    const int chunks = (group + 15) / 16;
    const int kv_head = blockIdx.y / chunks;
    const int chunk = blockIdx.y % chunks;
    const int split = blockIdx.z;
    const int head0 = kv_head * group + chunk * 16;
    const int heads_here = min(16, group - chunk * 16);
    const CacheLayout layout(kv_heads, page_size, HD);

    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int col = lane % 16;   // head (B operands, results) or key/dim row (A operands)
    const int quad = lane / 16;  // which 8 of the 32 k-slots this lane supplies

    const int seq = seq_of_token[token];
    const int position = positions[token];
    const int low = window > 0 ? max(0, position - window + 1) : 0;
    const int32_t* table = block_table + static_cast<int64_t>(seq) * table_width;

    const int first_pair = low / 32, last_pair = position / 32;
    const int total_pairs = last_pair - first_pair + 1;
    const int pairs_per_split = (total_pairs + n_splits - 1) / n_splits;
    const int pair_begin = first_pair + split * pairs_per_split;
    const int pair_end = min(pair_begin + pairs_per_split, last_pair + 1);

    // Q^T fragments: head `col`, dims ks * 32 + quad * 8 ... + 7.
    Frag8 q_frag[K_STEPS];
#pragma unroll
    for (int ks = 0; ks < K_STEPS; ++ks) {
        const int dim = ks * 32 + quad * 8;
        q_frag[ks].raw = make_uint4(0, 0, 0, 0);
        if (col < heads_here && dim < HD) {
            q_frag[ks].raw = *reinterpret_cast<const uint4*>(
                q + (static_cast<int64_t>(token) * heads + head0 + col) * HD + dim);
        }
    }

    floatx4 o_acc[HD_TILES];
#pragma unroll
    for (int d = 0; d < HD_TILES; ++d) o_acc[d] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    float running_max = -INFINITY, running_sum = 0.0f;

    // A pair's keys and values, from the pages into registers. A lane's 8 k-slots of the second product are the
    // 8 positions 8 * (quad % 2) .. + 7 of tile quad / 2 of the pair: one load of 16 bytes per 16 dims from the
    // value pages (which hold blocks of 32 dims as [position / 8][dim][position % 8], cache_layout.h). The first product's rows are taken in the order that makes the scores come out so: of its two
    // products, product t gives lane (head, quad) the keys 8 * quad + 4 * t .. + 3 of the pair, so its row
    // 4 * quad' + i (the lane whose `col` that is brings it) is key 8 * quad' + 4 * t + i.
    // Every load is issued, none behind a branch (a tile that no query sees is read from page 0 and masked like a
    // stale one): only of straight-line code does the compiler know how many loads are still on their way, and
    // waits for one pair alone while the next flies.
    auto load_pair = [&](int pair_index, const int (&page)[2], Frag8 (&k_frag)[2][K_STEPS], Frag8 (&v_frag)[HD_TILES]) {
        const int k_side = col / 8, v_side = quad / 2;      // which tile of the pair the lane's row / its k-slots lie in
        const int k_offset = (pair_index * 32 + 16 * k_side) % page_size;
        const int v_offset = (pair_index * 32 + 16 * v_side) % page_size;
        const bf16* k_tile = k_cache + layout.k_tile(max(k_side ? page[1] : page[0], 0), kv_head, k_offset / 16) +
                             (8 * ((col / 4) % 2) + col % 4) * 8;
        const bf16* v_tile = v_cache + layout.v_tile(max(v_side ? page[1] : page[0], 0), kv_head, v_offset / 16);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int ks = 0; ks < K_STEPS; ++ks) {
                const int piece = ks * 4 + quad;
                if (HD % 32 == 0) {
                    k_frag[t][ks].raw = load_piece<STREAM>(k_tile + piece * 128 + t * 32);
                } else {      // the last 32 dims are not all there: nothing may be read past the tile
                    k_frag[t][ks].raw = make_uint4(0, 0, 0, 0);
                    if (piece < K_CHUNKS) k_frag[t][ks].raw = load_piece<STREAM>(k_tile + piece * 128 + t * 32);
                }
            }
        }
#pragma unroll
        for (int d = 0; d < HD_TILES; ++d) {
            constexpr int kLast = HD_TILES - 1;
            const int width = (HD_TILES % 2 == 1 && d == kLast) ? 16 : 32;      // dims of the block of 32 this tile of 16 lies in
            v_frag[d].raw = load_piece<STREAM>(v_tile + (d / 2) * 512 + ((quad % 2) * width + (d % 2) * 16 + col) * 8);
        }
    };
    auto attend_pair = [&](int pair_index, const Frag8 (&k_frag)[2][K_STEPS], Frag8 (&v_frag)[HD_TILES]) {
        const int key0 = pair_index * 32;
        // S^T = K . Q^T: lane holds head `col`, keys 8 * quad + 4 * t + i of the pair from product t.
        float score[8];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            floatx4 s = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int ks = 0; ks < K_STEPS; ++ks)
                s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k_frag[t][ks].v, q_frag[ks].v, s, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = key0 + 8 * quad + 4 * t + i;
                score[4 * t + i] = (key >= low && key <= position) ? s[i] * scale : -INFINITY;
            }
        }
        // A pair that straddles an end of the visible range may hold stale values: they must not reach
        // the product, where 0 * NaN would be NaN.
        if (key0 < low || key0 + 31 > position) {
#pragma unroll
            for (int d = 0; d < HD_TILES; ++d)
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (score[j] == -INFINITY) v_frag[d].v[j] = static_cast<__bf16>(0.0f);
        }

        float tile_max = score[0];
#pragma unroll
        for (int j = 1; j < 8; ++j) tile_max = fmaxf(tile_max, score[j]);
        tile_max = max_lanes_16_apart(tile_max);
        const float new_max = fmaxf(running_max, tile_max);   // finite: every pair holds a visible key
        const float rescale = __expf(running_max - new_max);
        Frag8 p_frag;
        float tile_sum = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float p = __expf(score[j] - new_max);
            tile_sum += p;
            p_frag.v[j] = static_cast<__bf16>(p);
        }
        tile_sum = sum_lanes_16_apart(tile_sum);
        running_sum = running_sum * rescale + tile_sum;
        running_max = new_max;
#pragma unroll
        for (int d = 0; d < HD_TILES; ++d) {
            o_acc[d] *= rescale;
            o_acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_frag[d].v, p_frag.v, o_acc[d], 0, 0, 0);
        }
    };
    // The block table's entry for a tile, read whatever the tile (see load_pair): a tile that no query sees may
    // have none (the table ends) or a released one (-1); load_pair reads page 0 then.
    int no_lane = 0;
    asm volatile("v_mov_b32 %0, 0" : "=v"(no_lane));      // zero, but the compiler cannot tell: the entry stays in a vector
                                                           // register and is not waited for until a round later
    auto page_of = [&](int tile_key) -> int { return table[min(tile_key / page_size, table_width - 1) + no_lane]; };

    // The wave's pairs: pair_begin + wave, then every kDecodeWaves-th. While one pair is attended to the next one's
    // keys and values are on their way into the other set of registers, and the pages of the one after are
    // looked up. After its last pair a wave asks for that pair again (a place that exists) and drops it.
    int pair = pair_begin + wave;
    if (pair < pair_end) {
        const int last = pair + (pair_end - 1 - pair) / kDecodeWaves * kDecodeWaves;      // this wave's last pair
        Frag8 k_first[2][K_STEPS], k_second[2][K_STEPS];
        Frag8 v_first[HD_TILES], v_second[HD_TILES];
        // Loads arrive in the order they were issued: a look-up is issued before the keys and values of the same
        // round, so that waiting for it a round later does not wait for them.
        int page[2] = {page_of(pair * 32), page_of(pair * 32 + 16)};
        int following = min(pair + kDecodeWaves, last);
        int next_page[2] = {page_of(following * 32), page_of(following * 32 + 16)};
        load_pair(pair, page, k_first, v_first);
        while (true) {
            int after = min(following + kDecodeWaves, last);
            page[0] = page_of(after * 32);
            page[1] = page_of(after * 32 + 16);
            load_pair(following, next_page, k_second, v_second);
            attend_pair(pair, k_first, v_first);
            if (pair == last) break;
            pair = following;
            following = after;

            after = min(following + kDecodeWaves, last);
            next_page[0] = page_of(after * 32);
            next_page[1] = page_of(after * 32 + 16);
            load_pair(following, page, k_first, v_first);
            attend_pair(pair, k_second, v_second);
            if (pair == last) break;
            pair = following;
            following = after;
        }
    }

    // Join the 4 waves in LDS: o_shared[slot][head][dim]; lane holds head `col`, dims d*16 + quad*4 + i.
    if (kParallelJoin) {
#pragma unroll
        for (int d = 0; d < HD_TILES; ++d)
#pragma unroll
            for (int i = 0; i < 4; ++i) o_shared[wave][col][d * 16 + quad * 4 + i] = o_acc[d][i];
        if (quad == 0) {
            m_shared[wave][col] = running_max;
            l_shared[wave][col] = running_sum;
        }
        __syncthreads();
    } else {
        for (int w = 0; w < kDecodeWaves; ++w) {
            __syncthreads();
            if (wave != w) continue;
            const float old_max = w == 0 ? -INFINITY : m_shared[0][col];
            const float old_sum = w == 0 ? 0.0f : l_shared[0][col];
            const float new_max = fmaxf(old_max, running_max);
            const float keep = (old_max == -INFINITY) ? 0.0f : __expf(old_max - new_max);
            const float add = (running_max == -INFINITY) ? 0.0f : __expf(running_max - new_max);
#pragma unroll
            for (int d = 0; d < HD_TILES; ++d)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int dim = d * 16 + quad * 4 + i;
                    const float before = w == 0 ? 0.0f : o_shared[0][col][dim];
                    o_shared[0][col][dim] = before * keep + o_acc[d][i] * add;
                }
            if (quad == 0) {
                m_shared[0][col] = new_max;
                l_shared[0][col] = old_sum * keep + running_sum * add;
            }
        }
        __syncthreads();
    }

    for (int index = threadIdx.x; index < heads_here * HD; index += kDecodeThreads) {
        const int h = index / HD, dim = index % HD;
        float top = m_shared[0][h];
#pragma unroll
        for (int w = 1; w < kSlots; ++w) top = fmaxf(top, m_shared[w][h]);
        float total = 0.0f, sum = 0.0f;
#pragma unroll
        for (int w = 0; w < kSlots; ++w) {
            const float m = m_shared[w][h];
            const float weight = (m == -INFINITY) ? 0.0f : __expf(m - top);
            total += weight * o_shared[w][h][dim];
            sum += weight * l_shared[w][h];
        }
        const int64_t row = static_cast<int64_t>(token) * heads + head0 + h;
        const int64_t part_row = static_cast<int64_t>(blockIdx.x) * heads + head0 + h;   // partial results are kept densely
        if (n_splits == 1) {
            out[row * HD + dim] = from_float<bf16>(total / sum);
        } else {
            part_o[(part_row * n_splits + split) * HD + dim] = total;
            if (dim == 0) {
                part_ml[(part_row * n_splits + split) * 2 + 0] = top;
                part_ml[(part_row * n_splits + split) * 2 + 1] = sum;
            }
        }
    }
}

// Joins the splits of one (token, head): out = sum_s w_s O_s / sum_s w_s l_s with w_s = exp(m_s - max m).
__global__ void paged_attention_join_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                            const int32_t* __restrict__ token_ids, bf16* __restrict__ out, int heads,
                                            int head_dim, int n_splits) {
    const int token = token_ids ? token_ids[blockIdx.x / heads] : blockIdx.x / heads;
    if (token < 0) return;      // an entry that only pads the list to a fixed length
    const int64_t row = static_cast<int64_t>(token) * heads + blockIdx.x % heads;
    const int64_t part_row = blockIdx.x;
    // Eight splits at a time: their loads are asked for together, then used in the order of the splits.
    const float2* ml = reinterpret_cast<const float2*>(part_ml) + part_row * n_splits;
    float top = -INFINITY;
    for (int base = 0; base < n_splits; base += 8) {
        float2 pair[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) pair[j] = ml[min(base + j, n_splits - 1)];
#pragma unroll
        for (int j = 0; j < 8; ++j) top = fmaxf(top, pair[j].x);
    }
    for (int dim = threadIdx.x; dim < head_dim; dim += blockDim.x) {
        float total = 0.0f, weight_sum = 0.0f;
        for (int base = 0; base < n_splits; base += 8) {
            float2 pair[8];
            float part[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int split = min(base + j, n_splits - 1);
                pair[j] = ml[split];
                part[j] = part_o[(part_row * n_splits + split) * head_dim + dim];
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                if (base + j >= n_splits || pair[j].x == -INFINITY) continue;   // past the end, or a split without keys
                const float weight = __expf(pair[j].x - top);
                total += weight * part[j];
                weight_sum += weight * pair[j].y;
            }
        }
        out[row * head_dim + dim] = from_float<bf16>(total / weight_sum);
    }
}

template <int HD_TILES>
static int launch_decode(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_table,
                         int table_width, const int32_t* seq_of_token, const int32_t* positions,
                         const int32_t* token_ids, void* out, float* part_o, float* part_ml, float scale, int window,
                         int n_tokens, int heads, int kv_heads, int page_size, int n_splits, hipStream_t stream) {
    const int group = heads / kv_heads;
    const dim3 grid(n_tokens, kv_heads * ((group + 15) / 16), n_splits);
    const bool stream_pages = static_cast<int64_t>(grid.x) * grid.y * grid.z >= 256;      // a workgroup per compute unit or more
#define MLL_DECODE_LAUNCH(STREAM)                                                                                     \
    paged_attention_decode_kernel<HD_TILES, STREAM><<<grid, kDecodeThreads, 0, stream>>>(                             \
        static_cast<const bf16*>(q), static_cast<const bf16*>(k_cache), static_cast<const bf16*>(v_cache), block_table, \
        table_width, seq_of_token, positions, token_ids, static_cast<bf16*>(out), part_o, part_ml, scale, window, heads, \
        kv_heads, page_size, n_splits)
    if (stream_pages) MLL_DECODE_LAUNCH(true); else MLL_DECODE_LAUNCH(false);
#undef MLL_DECODE_LAUNCH
    return check_launch("paged_attention_decode");
}

}  // namespace mll

using namespace mll;

extern "C" int mll_paged_attention_decode(const void* q, const void* k_cache, const void* v_cache,
                                          const int32_t* block_table, int table_width, const int32_t* seq_of_token,
                                          const int32_t* positions, const int32_t* token_ids, void* out, float* part_o,
                                          float* part_ml, float scale, int window, int n_tokens, int heads, int kv_heads,
                                          int head_dim, int page_size, int n_splits, hipStream_t stream) {
    MLL_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "paged_attention_decode: heads must divide into kv_heads groups");
    MLL_REQUIRE(head_dim % 16 == 0 && head_dim >= 16 && head_dim <= 256,
                "paged_attention_decode: head_dim must be a multiple of 16 in [16, 256]");
    MLL_REQUIRE(page_size > 0 && page_size % 16 == 0, "paged_attention_decode: page_size must be a multiple of 16");
    MLL_REQUIRE(n_splits >= 1 && n_splits <= 65535, "paged_attention_decode: bad number of splits");
    MLL_REQUIRE(n_splits == 1 || (part_o && part_ml), "paged_attention_decode: splits need the partial buffers");
    MLL_REQUIRE(kv_heads * ((heads / kv_heads + 15) / 16) <= 65535, "paged_attention_decode: too many heads");
    if (n_tokens == 0) return 0;
    int status = 0;
#define MLL_DECODE_CASE(TILES)                                                                                        \
    case TILES:                                                                                                       \
        status = launch_decode<TILES>(q, k_cache, v_cache, block_table, table_width, seq_of_token, positions,         \
                                      token_ids, out, part_o, part_ml, scale, window, n_tokens, heads, kv_heads,      \
                                      page_size, n_splits, stream);                                                   \
        break;
    switch (head_dim / 16) {
        MLL_DECODE_CASE(1) MLL_DECODE_CASE(2) MLL_DECODE_CASE(3) MLL_DECODE_CASE(4) MLL_DECODE_CASE(5)
        MLL_DECODE_CASE(6) MLL_DECODE_CASE(7) MLL_DECODE_CASE(8) MLL_DECODE_CASE(9) MLL_DECODE_CASE(10)
        MLL_DECODE_CASE(11) MLL_DECODE_CASE(12) MLL_DECODE_CASE(13) MLL_DECODE_CASE(14) MLL_DECODE_CASE(15)
        MLL_DECODE_CASE(16)
        default: return fail("paged_attention_decode: unsupported head_dim");
    }
#undef MLL_DECODE_CASE
    if (status != 0) return status;
    if (n_splits > 1) {
        const int threads = head_dim <= 64 ? 64 : (head_dim <= 128 ? 128 : 256);
        paged_attention_join_kernel<<<n_tokens * heads, threads, 0, stream>>>(part_o, part_ml, token_ids,
                                                                             static_cast<bf16*>(out), heads, head_dim, n_splits);
        return check_launch("paged_attention_join");
    }
    return 0;
}
