// Paged attention for portions of prompts in bfloat16: MFMA for both products, online softmax in float32.
//
// A workgroup (8 waves) takes two tiles of up to 128 consecutive tokens each, of one request's portion and one
// query head: waves 0 to 3 a block of 32 tokens each of the first tile, waves 4 to 7 of the second; the 32 tokens
// are the 32 columns of v_mfma_f32_32x32x16_bf16. Every SIMD thus has a wave of either tile, whose matrix and
// vector work overlap. The host pairs a tile that sees many keys with one that sees few, so that every workgroup
// walks about as many keys and the compute units finish together (under a causal mask the last tile of a prompt
// has as many times the work of the first as there are tiles), and neighbouring tiles under a window, which read
// nearly the same keys. Both tiles read the same keys from LDS. The second tile may be empty.
// The workgroup walks the keys its tokens can see in blocks of 128 (64 for head sizes above 128): the block's key
// and value tiles are copied from the pages straight into LDS as they lie there (the pages are in MFMA order,
// cache_layout.h), the next block's being on its way while this one is used. The two stages are two LDS
// variables, so that the compiler need not wait for a load into one before it reads the other.
// Scores are computed transposed, S^T = K . Q^T: a lane then holds 16 keys of one token (its column), and the other
// half of the wave the other 16, so a token's maximum takes 15 comparisons and one exchange, and its sum is kept in
// two halves that meet once, at the end. O^T = V^T . P^T follows from registers: the rows of the first product are
// the run's keys in such an order (bits 2 and 3 of the row number exchanged) that the lane's scores of a 16-key
// tile are for 8 neighbouring positions, the 16 bytes that one read brings from the value tile for its dim.
// Only steps that touch the causal diagonal or the window's edge pay for the mask (a second
// instance of the loop's body), and values that no token of the workgroup can see are cleared in LDS before a
// block at an end of the walk is used, so that stale memory never meets a zero weight.
// The scale is folded into the exponent's multiply-add and the accumulators are rescaled only when some maximum
// has moved. The list of workgroups (request; first token in the flat list and tokens, for either tile) is built on
// the host.
#include <type_traits>

#include "cache_layout.h"
#include "common.h"
#include "microllm_hip.h"

namespace mll {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kPrefillWaves = 8;
constexpr int kPrefillThreads = kPrefillWaves * kWave;
constexpr int kPrefillTile = 128;     // tokens of one tile: four blocks of 32, a wave each

union PFrag8 {
    bf16x8 v;
    bf16x4 h[2];
    uint4 raw;
};

// op over the two lanes {l, l ^ 32} of a wave, both of which get the result (v_permlane32_swap of gfx950).
template <typename Op>
__device__ inline float reduce_lanes_32_apart(float value, Op op) {
    const unsigned bits = __builtin_bit_cast(unsigned, value);
    const auto halves = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
    const unsigned low = halves[0], high = halves[1];
    return op(__builtin_bit_cast(float, low), __builtin_bit_cast(float, high));
}


template <int HD_TILES>
__global__ __launch_bounds__(kPrefillThreads, 1) void paged_attention_prefill_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ tiles,
    const int32_t* __restrict__ positions, bf16* __restrict__ out, float scale, int window, int heads,
    int kv_heads, int page_size) {
    constexpr int HD = HD_TILES * 16;
    constexpr int K_STEPS = HD_TILES;                            // steps of 16 dims of the first product
    constexpr int D_BLOCKS = (HD + 31) / 32;                     // blocks of 32 dims of the second product's result
    constexpr int BLOCK_KEYS = HD <= 128 ? 128 : 64;
    constexpr int BLOCK_TILES = BLOCK_KEYS / 16;
    constexpr int STEPS = BLOCK_KEYS / 32;                       // steps of 32 keys in a block
    constexpr int TILE_ELEMENTS = HD * 16;                       // of keys and of values alike
    constexpr int TILE_CHUNKS = TILE_ELEMENTS / 8;               // pieces of 16 bytes
    constexpr int STAGE_ELEMENTS = 2 * BLOCK_TILES * TILE_ELEMENTS;
    // Two stages of [K | V][BLOCK_TILES][TILE_ELEMENTS]. They are two variables, not one array: the compiler then
    // knows that a load into one stage does not write what is read from the other, and lets the two overlap.
    __shared__ __align__(16) bf16 stage_even[STAGE_ELEMENTS];
    __shared__ __align__(16) bf16 stage_odd[STAGE_ELEMENTS];

    // Which entry and head this workgroup takes. Workgroups go to the GPU's 8 dies (each with a second-level cache
    // of its own) by turns, in the order of their number; numbered entry-first, every die would read every kv
    // head's keys and values. Instead a die takes the query heads of one kv head (of 8 / kv_heads dies each), the
    // entries still in the list's order (longest first): a long prompt's keys then mostly come from the die's own
    // cache (8192 tokens at 7B sizes: 800 -> 680 us; 16384: 2650 -> 2340). Where the numbers do not divide, the
    // workgroups keep their plain numbering.
    int entry_index = blockIdx.x, head = blockIdx.y;
    {
        constexpr int kDies = 8;
        const int group = heads / kv_heads;
        const int dies_per_kv_head = kv_heads <= kDies && kDies % kv_heads == 0 ? kDies / kv_heads : 0;
        if (dies_per_kv_head > 0 && (gridDim.x * group) % dies_per_kv_head == 0) {
            const int number = blockIdx.x + gridDim.x * blockIdx.y;
            const int die = number % kDies, turn = number / kDies;
            const int item = turn * dies_per_kv_head + die % dies_per_kv_head;      // among the kv head's entries x heads
            entry_index = item / group;
            head = (die / dies_per_kv_head) * group + item % group;
        }
    }
    const int32_t* entry = tiles + 5 * entry_index;
    if (entry[2] <= 0 && entry[4] <= 0) return;      // an entry that only pads the list to a fixed length
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int column = lane % 32;     // token of the block (B operands, results) or key / dim row (A operands)
    const int half = lane / 32;       // which 8 of a step's 16 k-slots this lane supplies
    const int seq = entry[0];
    const int kv_head = head / (heads / kv_heads);
    const int32_t* table = block_table + static_cast<int64_t>(seq) * table_width;
    const float scale_log2 = scale * 1.4426950408889634f;      // scores are kept in units of log 2: p = 2^(s - max)

    // Either tile's tokens and the keys any of them can see (tokens of a portion have consecutive positions);
    // an empty tile sees nothing: no key lies in its range.
    int range_low[2], range_last[2], tile_positions[2];
#pragma unroll
    for (int side = 0; side < 2; ++side) {
        const int count = entry[2 + 2 * side];
        tile_positions[side] = count > 0 ? positions[entry[1 + 2 * side]] : 0;
        range_last[side] = count > 0 ? tile_positions[side] + count - 1 : -1;
        range_low[side] = count > 0 ? (window > 0 ? max(0, tile_positions[side] - window + 1) : 0) : (1 << 30);
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

    // This wave's block of 32 tokens: waves 0 to 3 take the first tile, waves 4 to 7 the second.
    const int side = wave / 4;
    const int count = entry[2 + 2 * side];
    const int first_token = entry[1 + 2 * side];
    const int tile_position = tile_positions[side];
    const int block_first = 32 * (wave % 4);                              // in the tile
    const int block_valid = min(32, max(0, count - block_first));
    const int block_position = tile_position + block_first;
    const int block_last = block_position + block_valid - 1;
    const int block_low = window > 0 ? max(0, block_position - window + 1) : 0;        // the lowest key its first token sees
    const int block_last_low = window > 0 ? max(0, block_last - window + 1) : 0;       // and its last token
    const int index = min(column, max(block_valid - 1, 0));                // columns past the end repeat the last token
    const int my_position = block_position + index;
    const int my_low = window > 0 ? max(0, my_position - window + 1) : 0;

    PFrag8 q_frag[K_STEPS];
#pragma unroll
    for (int ks = 0; ks < K_STEPS; ++ks) {
        q_frag[ks].raw = make_uint4(0, 0, 0, 0);
        if (block_valid > 0)
            q_frag[ks].raw = *reinterpret_cast<const uint4*>(
                q + (static_cast<int64_t>(first_token + block_first + index) * heads + head) * HD + ks * 16 + half * 8);
    }

    floatx16 o_acc[D_BLOCKS];
#pragma unroll
    for (int d = 0; d < D_BLOCKS; ++d)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[d][i] = 0.0f;
    float running_max = -INFINITY;
    float running_sum = 0.0f;         // over this lane's keys only; the two halves of the wave meet at the end
    float running_offset = 0.0f;      // -(running maximum) in units of log 2; 0 while the maximum is -inf

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
    constexpr bool FULL_PASSES = HALF_CHUNKS % kPrefillThreads == 0;      // every pass of every wave lies within the block
    auto wanted = [&](int block, int pass) {      // whether the tile is brought in: some token sees some of it
        const int tile_key = block * BLOCK_KEYS + 16 * tile_of(pass);
        return (FULL_PASSES || tile_of(pass) < BLOCK_TILES) && tile_key <= group_last && (inside(block) || tile_seen(tile_key));
    };
    // Pages mostly hold a power of two of tiles (often one): then the page of a tile is a shift, else a division.
    // The choice is made once per block, not per tile.
    auto page_index = [&](auto shift_tag, int tile_index) {
        return decltype(shift_tag)::value ? tile_index >> page_shift : tile_index / tiles_per_page;
    };
    auto tile_in_its_page = [&](auto shift_tag, int tile_index) {
        return decltype(shift_tag)::value ? tile_index & (tiles_per_page - 1) : tile_index % tiles_per_page;
    };
    // The pages of a block's tiles are looked up one block ahead of the tiles themselves, so that no load waits
    // for another. The look-up is a load of the vector unit also where the whole wave asks for one entry: those
    // are counted with the loads into LDS and have arrived when these have, whereas a load of the scalar unit
    // would be waited for by the first read from LDS that follows it.
    int pages[PASSES];
    int no_lane = 0;
    asm volatile("v_mov_b32 %0, 0" : "=v"(no_lane));      // zero, but the compiler cannot tell: keeps the address per lane
    auto look_up_with = [&](auto shift_tag, int block) __attribute__((always_inline)) {
        const bool whole = FULL_PASSES && inside(block);      // the usual case: every tile of the block, no questions
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            const int tile_index = block * BLOCK_TILES + tile_of(pass);
            pages[pass] = -1;
            if (whole || wanted(block, pass)) pages[pass] = table[page_index(shift_tag, tile_index) + no_lane];
        }
    };
    auto look_up = [&](int block) __attribute__((always_inline)) {
        if (page_shift >= 0) look_up_with(std::true_type{}, block);
        else look_up_with(std::false_type{}, block);
    };
    auto fetch_with = [&](auto shift_tag, int block, bf16* stage) __attribute__((always_inline)) {      // after look_up(block)
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            const int tile_index = block * BLOCK_TILES + tile_of(pass);
            const int tile_in_page = tile_in_its_page(shift_tag, tile_index);
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
    auto fetch = [&](int block, bf16* stage) __attribute__((always_inline)) {
        if (page_shift >= 0) fetch_with(std::true_type{}, block, stage);
        else fetch_with(std::false_type{}, block, stage);
    };
    // A block at an end of what the tile's tokens see, once it lies in LDS: values at positions that no token
    // sees may be stale memory, and the places of tiles that were not brought in hold what was there before.
    // Both are cleared (their scores are masked where they are computed).
    auto clear_unseen = [&](int block, bf16* stage) __attribute__((always_inline)) {
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            if (tile_of(pass) >= BLOCK_TILES) continue;
            uint4* place = reinterpret_cast<uint4*>(stage + HALF_CHUNKS * 8 + (tile_of(pass) * TILE_CHUNKS + piece_of(pass)) * 8);
            PFrag8 values;
            values.raw = make_uint4(0, 0, 0, 0);
            if (wanted(block, pass)) {
                values.raw = *place;
                // one dim, positions 0 .. 7 or 8 .. 15 of the tile: a block of 32 dims is [position / 8][32][8], a last
                // block of 16 dims [position / 8][16][8]
                const int element = piece_of(pass) * 8;
                const int width = (HD % 32 != 0 && element / 512 == HD / 32) ? 16 : 32;
                const int first_key = block * BLOCK_KEYS + 16 * tile_of(pass) + 8 * ((element % 512) / (8 * width));
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (!seen(first_key + i)) values.v[i] = static_cast<__bf16>(0.0f);
            }
            *place = values.raw;
        }
    };
    const int first_block = group_low / BLOCK_KEYS;
    const int last_block = group_last / BLOCK_KEYS;
    // The wave's loads into LDS have landed (the compiler does not wait for loads that return nothing), and so
    // have everyone's; everyone is done with the stage that is written next.
    auto landed = [&](int block, bf16* stage) __attribute__((always_inline)) {
        wait_for_loads();
        __syncthreads();
        if (block <= last_block && !inside(block)) {
            clear_unseen(block, stage);
            __syncthreads();
        }
    };

    // HALVES (1 or 2) runs of 32 keys against the wave's 32 tokens; the runs are numbered within the block. Two
    // runs at once share one maximum, one exchange between the halves of the wave and one look at whether anything
    // must be rescaled, and their two chains of products hide each other's latency. MASKED: some key is hidden
    // from some token (the causal diagonal, the window's edge, the end of the sequence).
    // Scores stay in the product's units; p = 2^((s - max) * scale_log2) is one multiply-add and one exponent.
    // First product: row `column` = the key of the run whose number is `column` with bits 2 and 3 exchanged (tile
    // column / 16), 8 dims (chunk 2 ks + half) per lane. Second: row = dim `column` of a block of 32 dims; the
    // lane's 8 k-slots are the keys its scores came for, positions 8 half .. + 7 of the tile, one read of 16 bytes;
    // the 64 lanes read 1024 consecutive bytes, which LDS gives without bank conflicts.
    // The addresses are formed step by step (stage, then tile, then lane). The compiler follows an address back
    // to its LDS variable over a few additions only, and of a read that it cannot place it assumes that the loads
    // on their way into the other stage may write it: the first reads of every run of keys therefore wait for
    // those loads. Formed as one sum (stage plus a per-lane term plus a constant) the reads do not wait, and the
    // kernel is 5 % slower (836 against 791 us for 8192 tokens, 2680 against 2545 for 16384; waiting for the
    // loads in other places does not give the same, nor does holding one tile's waves back for a while at the
    // start of a block). Measured, not understood.
    const int key_of_row = (column & ~12) | ((column & 4) << 1) | ((column & 8) >> 1);
    auto process_keys = [&](auto masked_tag, auto halves_tag, const bf16* stage, int first_run, int key0) __attribute__((always_inline)) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        constexpr int HALVES = decltype(halves_tag)::value;
        const bf16* k_rows = stage + (2 * first_run + column / 16) * TILE_ELEMENTS + (half * 16 + key_of_row % 16) * 8;
        floatx16 s[HALVES];
#pragma unroll
        for (int r = 0; r < HALVES; ++r)
#pragma unroll
            for (int i = 0; i < 16; ++i) s[r][i] = 0.0f;
        // The keys' operands are read kAhead products ahead of their use (the runs by turns, so that two chains of
        // products are under way), and the compiler is told to keep reads and products in this order: left to
        // itself it reads each operand right before its product and waits for it.
        constexpr int PRODUCTS = HALVES * K_STEPS;
        constexpr int kAhead = PRODUCTS < 4 ? PRODUCTS : 4;
        PFrag8 k_frag[PRODUCTS];
        auto read_keys = [&](int j) {
            k_frag[j].raw = *reinterpret_cast<const uint4*>(k_rows + (j % HALVES) * 2 * TILE_ELEMENTS + (j / HALVES) * 256);
        };
#pragma unroll
        for (int j = 0; j < kAhead; ++j) read_keys(j);
        __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
#pragma unroll
        for (int j = 0; j < PRODUCTS; ++j) {
            if (j + kAhead < PRODUCTS) read_keys(j + kAhead);
            s[j % HALVES] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_frag[j].v, q_frag[j / HALVES].v, s[j % HALVES], 0, 0, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (j + kAhead < PRODUCTS) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        // s[r][i] is row 8 (i / 4) + 4 half + i % 4: key key0 + 32 r + 16 (i / 8) + 8 half + i % 8, token `column`.
        if (MASKED) {
#pragma unroll
            for (int r = 0; r < HALVES; ++r)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int key = key0 + 32 * r + 16 * (i / 8) + 8 * half + (i % 8);
                    if (key > my_position || key < my_low) s[r][i] = -INFINITY;
                }
        }
        float tile_max = fmaxf(fmaxf(s[0][0], s[0][1]), s[0][2]);
#pragma unroll
        for (int i = 3; i < 15; i += 2) tile_max = fmaxf(fmaxf(tile_max, s[0][i]), s[0][i + 1]);
        tile_max = fmaxf(tile_max, s[0][15]);
#pragma unroll
        for (int r = 1; r < HALVES; ++r)
#pragma unroll
            for (int i = 0; i < 16; i += 2) tile_max = fmaxf(fmaxf(tile_max, s[r][i]), s[r][i + 1]);
        // Far into a prompt a step rarely holds a new maximum for any of the wave's tokens: then the two halves
        // need not compare notes, and nothing is rescaled (the same numbers either way).
        float rescale = 1.0f;
        if (__any(tile_max > running_max)) {
            tile_max = reduce_lanes_32_apart(tile_max, [](float a, float b) { return fmaxf(a, b); });
            const float new_max = fmaxf(running_max, tile_max);
            // A token may see nothing of a step that others see (the window's edge): its maximum stays -inf.
            const float safe_max = (MASKED && new_max == -INFINITY) ? 0.0f : new_max;
            running_offset = -safe_max * scale_log2;
            // exactly 1 for a token whose maximum stays (the rounding of maximum * scale would else leave a factor
            // of 1 +- 1e-7, and every sum would be multiplied by it)
            rescale = new_max == running_max ? 1.0f : __builtin_amdgcn_exp2f(fmaf(running_max, scale_log2, running_offset));
            running_max = new_max;
        }
        const float offset = running_offset;
        float step_sum = 0.0f;
        PFrag8 p_frag[2 * HALVES];
#pragma unroll
        for (int r = 0; r < HALVES; ++r)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float p = __builtin_amdgcn_exp2f(fmaf(s[r][i], scale_log2, offset));
                step_sum += p;
                p_frag[2 * r + i / 8].v[i % 8] = static_cast<__bf16>(p);
            }
        running_sum = running_sum * rescale + step_sum;
        // Once the running maxima have settled, no column's sums need rescaling: one branch for the whole wave.
        if (__any(rescale != 1.0f)) {
#pragma unroll
            for (int d = 0; d < D_BLOCKS; ++d) o_acc[d] *= rescale;
        }
        // O^T += V^T . P^T, 16 keys (one tile) a product.
        const bf16* v_rows = stage + HALF_CHUNKS * 8 + 2 * first_run * TILE_ELEMENTS + column * 8 + half * 256;
#pragma unroll
        for (int t = 0; t < 2 * HALVES; ++t)
#pragma unroll
            for (int d = 0; d < D_BLOCKS; ++d) {
                PFrag8 v_frag;
                v_frag.raw = make_uint4(0, 0, 0, 0);
                if (HD % 32 == 0 || d < D_BLOCKS - 1) {
                    v_frag.raw = *reinterpret_cast<const uint4*>(v_rows + t * TILE_ELEMENTS + d * 512);
                } else if (column < 16) {      // the last block has 16 dims: [position / 8][16][8]
                    v_frag.raw = *reinterpret_cast<const uint4*>((stage + (half * 16 + column) * 8) +
                                                                 (HALF_CHUNKS * 8 + (2 * first_run + t) * TILE_ELEMENTS + d * 512));
                }
                o_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v_frag.v, p_frag[t].v, o_acc[d], 0, 0, 0);
            }
    };

    auto next_seen = [&](int block) {      // the next block after this one of which something is seen
        ++block;
        while (block * BLOCK_KEYS <= group_last && !block_seen(block)) ++block;
        return block;
    };
    // (The lambdas above and below are marked always_inline: left to its own count of instructions the compiler
    // makes a function of one of them, whose call then costs registers kept in memory.)
    // One block: the next one is sent for, this one is used. Called by turns with the stages exchanged.
    int block = first_block;
    int following = next_seen(first_block);
    auto walk = [&](const bf16* stage, bf16* next_stage) __attribute__((always_inline)) {
        if (following <= last_block) {
            fetch(following, next_stage);
            const int after = next_seen(following);
            if (after <= last_block) look_up(after);
        }
        // Unrolled: every read from LDS then has an address of the stage plus a constant (an address that a loop
        // carries along would make every read wait for the loads on their way into the other stage).
#pragma unroll
        for (int pair = 0; pair < STEPS / 2; ++pair) {
            const int key0 = block * BLOCK_KEYS + 64 * pair;
            bool see[2], hidden[2];
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                see[r] = block_valid > 0 && key0 + 32 * r <= block_last && key0 + 32 * r + 31 >= block_low;
                hidden[r] = key0 + 32 * r + 31 > block_position || key0 + 32 * r < block_last_low;
            }
            if (see[0] && see[1] && !hidden[0] && !hidden[1]) {
                process_keys(std::false_type{}, std::integral_constant<int, 2>{}, stage, 2 * pair, key0);
            } else {
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    if (!see[r]) continue;      // nothing of this run is visible to the wave
                    if (hidden[r]) process_keys(std::true_type{}, std::integral_constant<int, 1>{}, stage, 2 * pair + r, key0 + 32 * r);
                    else process_keys(std::false_type{}, std::integral_constant<int, 1>{}, stage, 2 * pair + r, key0 + 32 * r);
                }
            }
        }
        wait_for_loads();
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
    running_sum = reduce_lanes_32_apart(running_sum, [](float a, float b) { return a + b; });

    // o_acc[d][i]: dim 32 d + 8 (i / 4) + 4 half + i % 4 of token `column`.
    if (column < block_valid) {
        const float inverse = 1.0f / running_sum;
        bf16* out_row = out + (static_cast<int64_t>(first_token + block_first + column) * heads + head) * HD;
#pragma unroll
        for (int d = 0; d < D_BLOCKS; ++d)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int dim = d * 32 + 8 * j + 4 * half;
                if (HD % 32 != 0 && dim >= HD) continue;
                bf16x4 four;
#pragma unroll
                for (int i = 0; i < 4; ++i) four[i] = static_cast<__bf16>(o_acc[d][4 * j + i] * inverse);
                *reinterpret_cast<bf16x4*>(out_row + dim) = four;
            }
    }
}

template <int HD_TILES>
static int launch_prefill(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_table,
                          int table_width, const int32_t* tiles, int n_tiles, const int32_t* positions, void* out,
                          float scale, int window, int heads, int kv_heads, int page_size, hipStream_t stream) {
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
