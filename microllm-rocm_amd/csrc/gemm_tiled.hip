// Matrix products with many rows (prompts): C = A . W^T for bfloat16 A [M, K] (row-major) and the same packed
// weight the streaming kernel reads ([N/16][K/32][4][16][8]), on v_mfma_f32_16x16x32_bf16.
//
// A workgroup of 8 waves (two on every SIMD) owns a 256 x 256 tile of C, a wave 128 x 64 of it (8 x 4 MFMA tiles,
// 128 accumulator registers); or a tile of 192, 160 or 128 rows (a wave 6, 5 or 4 row tiles), where tiles of 256
// rows would leave many compute units without one. k is walked in stages of 64. A stage's 256 rows of A and of W (64 KB) are brought
// into one of two LDS slots by direct global-to-LDS loads, 1 KB a wave-wide instruction: of A 8 rows of 128 bytes
// (whole cache lines: with half lines, 64 bytes of 16 rows, the loads alone take a quarter longer), of W a piece as
// it lies in memory. A row's eight 16-byte chunks are stored at places exchanged by (row / 2), so that the 64 lanes
// of an operand read (row = lane % 16, chunk = 4 step + lane / 16) fall on all banks.
// A wave holds the operands of two k steps of 32 in registers: while it multiplies one step's (32 products), the
// next step's 12 reads from LDS are issued between the products, one after every second, and have arrived when the
// products are done. The workgroup meets once a stage, when the next stage has landed and the slot of the stage
// before is free for the stage after next. The reads and the products are volatile asm, which pins their order;
// the compiler neither sees the reads (and so orders nothing against the loads in flight) nor moves the products.
// Timed on MI355X against reads and a barrier before each stage's products, with half lines of A:
// 8192 x 37888 x 3584 2200 -> 1800 us (1.24 PFLOP/s), 2048 x 37888 x 3584 580 -> 480 us.
// Taken apart at 8192 x 37888 x 3584: products and barriers alone 1230 us, the loads alone (one stage in flight)
// 1550, everything 1790.
// Workgroups are numbered so that the 32 that run together on one of the 8 XCDs (each with a second-level cache of
// its own) own about 4 x 8 neighbouring tiles of C, and so share their rows of A and of W there, and so that every
// XCD gets the same number of tiles.
#include <utility>

#include "cache_layout.h"
#include "common.h"
#include "microllm_hip.h"

namespace mll {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) bf16 lds_bf16;

constexpr int kTileN = 256;
constexpr int kMaxWaveTilesM = 8;                         // a wave's part of C is at most 128 x 64
constexpr int kTiledWaves = 8;
constexpr int kTiledThreads = kTiledWaves * kWave;
constexpr int kPieceElements = 512;                       // of W: 16 rows x 32 k in MFMA operand order, 1 KB
constexpr int kWaveTilesN = 4;                            // a wave's 64 columns of C
constexpr int kSlotBytes = 65536;                         // a stage of 64 of k: up to 32 KB of A, then 32 KB of W
constexpr int kSlotElements = kSlotBytes / 2;
constexpr int kWBytes = 32768;                            // where W begins in a slot
constexpr int kSuperM = 4, kSuperN = 8;                   // tiles of C that run together on an XCD

__device__ __align__(16) const unsigned zero_piece[256] = {};      // a piece of W past the end of k

__device__ inline float silu_fast(float value) { return value / (1.0f + __expf(-value)); }

__device__ inline unsigned lds_address(bf16* place) { return static_cast<unsigned>(reinterpret_cast<uintptr_t>((lds_bf16*)place)); }

template <int WM>
struct TiledOperands {       // of one k step: the wave's WM pieces of A and 4 of W, 16 bytes a lane each
    uintx4 a[WM];
    uintx4 w[kWaveTilesN];
};

#define MLL_DS_READ(TARGET, ADDRESS, BYTES) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(TARGET) : "v"(ADDRESS), "n"(BYTES))
#define MLL_MFMA(ACC, W, A) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(ACC) : "v"(W), "v"(A))

// The INDEX-th of the 4 + WM reads of k step STEP (0, 1) of a stage: pieces of A are 2 KB apart in a slot, tiles of W
// too, with the tile's second step 1 KB after its first. An INDEX beyond the reads is nothing.
template <int WM, int INDEX, int STEP>
__device__ __attribute__((always_inline)) inline void read_operand(TiledOperands<WM>& f, unsigned a_address, unsigned w_address) {
    constexpr int W = kWBytes + STEP * 1024;
    if constexpr (INDEX == 0) MLL_DS_READ(f.w[0], w_address, W);
    if constexpr (INDEX == 1) MLL_DS_READ(f.w[1], w_address, W + 2048);
    if constexpr (INDEX == 2) MLL_DS_READ(f.a[0], a_address, 0);
    if constexpr (INDEX == 3) MLL_DS_READ(f.a[1], a_address, 2048);
    if constexpr (INDEX == 4) MLL_DS_READ(f.w[2], w_address, W + 4096);
    if constexpr (INDEX == 5) MLL_DS_READ(f.w[3], w_address, W + 6144);
    if constexpr (INDEX >= 6 && INDEX < 4 + WM) MLL_DS_READ(f.a[INDEX - 4], a_address, (INDEX - 4) * 2048);
}
template <int WM, int STEP, int... INDEX>
__device__ __attribute__((always_inline)) inline void read_operands(TiledOperands<WM>& f, unsigned a_address, unsigned w_address,
                                                                    std::integer_sequence<int, INDEX...>) {
    (read_operand<WM, INDEX, STEP>(f, a_address, w_address), ...);
}

// The four products of row tile MT of a k step, and after every second of them a read of the next step's operands
// (the first 4 + WM of the 2 WM places take one).
template <int WM, int NEXT_STEP, int MT>
__device__ __attribute__((always_inline)) inline void products_of_row_tile(floatx4 (&acc)[kWaveTilesN][WM], const TiledOperands<WM>& now,
                                                                           TiledOperands<WM>& next, unsigned a_address, unsigned w_address) {
    MLL_MFMA(acc[0][MT], now.w[0], now.a[MT]);
    MLL_MFMA(acc[1][MT], now.w[1], now.a[MT]);
    read_operand<WM, 2 * MT, NEXT_STEP>(next, a_address, w_address);
    MLL_MFMA(acc[2][MT], now.w[2], now.a[MT]);
    MLL_MFMA(acc[3][MT], now.w[3], now.a[MT]);
    read_operand<WM, 2 * MT + 1, NEXT_STEP>(next, a_address, w_address);
}
template <int WM, int NEXT_STEP, int... MT>
__device__ __attribute__((always_inline)) inline void products(floatx4 (&acc)[kWaveTilesN][WM], const TiledOperands<WM>& now,
                                                               TiledOperands<WM>& next, unsigned a_address, unsigned w_address,
                                                               std::integer_sequence<int, MT...>) {
    (products_of_row_tile<WM, NEXT_STEP, MT>(acc, now, next, a_address, w_address), ...);
}

// The reads into `f` have arrived (and, LOADS, the wave's loads into LDS have landed). `f` passes through the
// statements, so that nothing that uses it is placed before.
template <bool LOADS, int WM>
__device__ __attribute__((always_inline)) inline void operands_arrived(TiledOperands<WM>& f) {
    if constexpr (LOADS)
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)"
                     : "+v"(f.a[0]), "+v"(f.a[1]), "+v"(f.a[2]), "+v"(f.a[3]), "+v"(f.w[0]), "+v"(f.w[1]), "+v"(f.w[2]), "+v"(f.w[3])
                     :: "memory");
    else
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(f.a[0]), "+v"(f.a[1]), "+v"(f.a[2]), "+v"(f.a[3]), "+v"(f.w[0]), "+v"(f.w[1]), "+v"(f.w[2]), "+v"(f.w[3])
                     :: "memory");
#pragma unroll
    for (int i = 4; i < WM; ++i) asm volatile("" : "+v"(f.a[i]));
}

// EPILOGUE: 0 = float32 [M, N]; 1 = bfloat16 [M, N]; 2 = bfloat16 [M, N / 2] = silu(even rows of W) * (odd rows);
// 3 = queries, keys and values: bias, rotation, queries to `store.q_out`, keys and values into their pages (W's rows
// in rotary pair order; see MllQkvStore).
// WM: a workgroup's tile of C has 32 WM rows (a wave WM row tiles of 16), 4 to 8: fewer where 256 rows a tile would
// leave many compute units without one.
// With epilogue 0 the stages of k may be dealt to gridDim.y workgroups, each writing its own [M, N] of partial sums.
template <int EPILOGUE, int WM>
__global__ __launch_bounds__(kTiledThreads, 1) void gemm_tiled_kernel(const bf16* __restrict__ a, const bf16* __restrict__ w_packed,
                                                                      void* __restrict__ out, int m, int n, int k, int n_tiles,
                                                                      int k_steps, int m_blocks, int n_blocks, MllQkvStore store) {
    static_assert(WM >= 4 && WM <= kMaxWaveTilesM, "a wave takes 4 to 8 row tiles");
    constexpr int TILE_M = 32 * WM;
    constexpr int A_LOADS = 4 * WM;                       // a stage of A: 2 WM pieces of 16 rows, two loads of 8 rows each
    constexpr int A_TURNS = (A_LOADS + kTiledWaves - 1) / kTiledWaves;
    // Two slots. In a slot: A as [2 WM pieces of 16 rows][row][8 places of 16 bytes], the row's chunk c of 8 elements
    // at place c ^ (row / 2); then W as [16 tiles][2 k steps][1 KB in MFMA operand order]. Only the direct loads write
    // this memory and only the asm reads read it.
    __shared__ __align__(16) bf16 slots[2 * kSlotElements];

    // Workgroups 8 apart in number run on one XCD, 32 of them at a time. The tiles of C are put in a row, blocks of
    // 4 x 8 neighbouring tiles after one another (down the rows of C first, narrower at the edges), and every XCD
    // takes an equal stretch of that row: the workgroups that run together there own neighbouring tiles, and no XCD
    // has more than one tile more than another.
    const int tiles = m_blocks * n_blocks;
    const int per_xcd = (tiles + 7) / 8;
    const int place = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (blockIdx.x / 8 >= per_xcd || place >= tiles) return;
    const int column = place / (m_blocks * kSuperN);                       // of blocks, kSuperN tiles wide
    const int width = min(kSuperN, n_blocks - column * kSuperN);
    const int in_column = place - column * m_blocks * kSuperN;
    const int block = in_column / (kSuperM * width);                       // in the column, kSuperM tiles high
    const int height = min(kSuperM, m_blocks - block * kSuperM);
    const int in_block = in_column - block * kSuperM * width;
    const int m_block = block * kSuperM + in_block % height;
    const int n_block = column * kSuperN + in_block / height;

    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int col = lane % 16, quad = lane / 16;
    const int wave_m = wave / 4, wave_n = wave % 4;        // which (16 WM) x 64 of the tile
    const int m0 = m_block * TILE_M, n_tile0 = n_block * (kTileN / 16);

    // What this wave copies per stage. Of A the loads wave, wave + 8, ... of the stage's 4 WM: load i brings 8 rows
    // (half h = i % 2 of piece i / 2; lane L: row L / 8 of the 8, place L % 8 of the row). Of W tiles 2 * wave and
    // 2 * wave + 1, a k step an instruction.
    const bf16* a_block = a + static_cast<int64_t>(m0) * k;
    int a_offset[A_TURNS];    // of the lane's 16 bytes from a_block, at stage 0
    const int a_loads = (A_LOADS - wave + kTiledWaves - 1) / kTiledWaves;      // of this wave
#pragma unroll
    for (int t = 0; t < A_TURNS; ++t) {
        const int load = min(wave + t * kTiledWaves, A_LOADS - 1);
        const int row_in_piece = 8 * (load % 2) + lane / 8;
        const int row = min((load / 2) * 16 + row_in_piece, m - 1 - m0);           // rows past the end repeat the last one
        a_offset[t] = row * k + (((lane % 8) ^ (row_in_piece / 2)) * 8);
    }
    const bf16* w_tile[2];    // the lane's 16 bytes of the tile's piece at k step 0
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int tile = min(n_tile0 + wave * 2 + p, n_tiles - 1);
        w_tile[p] = w_packed + static_cast<int64_t>(tile) * k_steps * kPieceElements + lane * 8;
    }
    const int all_stages = (k_steps + 1) / 2;
    const int stages_per_split = (all_stages + gridDim.y - 1) / gridDim.y;
    const int first_stage = blockIdx.y * stages_per_split;
    const int stages = min(all_stages, first_stage + stages_per_split);
    const int last = stages - 1;
    // A k step past the end (k an odd multiple of 32; the stage after the last, which the loop's second half may
    // take) gets zeros for W and, for A, values that lie in the row: the chunks of the stage's second half step
    // back by 64 bytes there, the stage after the last is the last again.
    auto copy_stage = [&](int stage, int slot) __attribute__((always_inline)) {
        bf16* a_place = slots + slot * kSlotElements;
        bf16* w_place = a_place + kWBytes / 2;
        const int a_stage = min(stage, last);
        const bool half_stage = 2 * a_stage + 1 >= k_steps;
#pragma unroll
        for (int t = 0; t < A_TURNS; ++t) {
            if (t < a_loads) {
                const int piece = (wave + t * kTiledWaves) / 2, h = wave % 2;      // the wave's loads are all of one half
                const bool upper = (((lane >> 2) & 1) ^ h) != 0;      // the lane's chunk is one of the row's second four
                const bf16* a_source = a_block + a_stage * 64 + a_offset[t] - ((half_stage && upper) ? 32 : 0);
                // (the place is computed here: with a subscript of a captured array in this call the host pass
                // drops the kernel's stub without a word)
                __builtin_amdgcn_global_load_lds(a_source, a_place + piece * 1024 + h * 512, 16, 0, 0);
            }
        }
#pragma unroll
        for (int p = 0; p < 2; ++p) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const bool real = stage <= last && 2 * stage + h < k_steps;
                const bf16* w_source = real ? w_tile[p] + static_cast<int64_t>(2 * stage + h) * kPieceElements
                                            : reinterpret_cast<const bf16*>(zero_piece) + lane * 8;
                __builtin_amdgcn_global_load_lds(w_source, w_place + (wave * 2 + p) * 1024 + h * 512, 16, 0, 0);
            }
        }
    };
    // Where the lane reads its operands: row `col` of a piece, chunk 4 step + quad at its place.
    const unsigned base = lds_address(slots);
    const unsigned a_row = base + wave_m * WM * 2048 + col * 128;
    const unsigned a_step0 = a_row + ((quad ^ (col / 2)) * 16), a_step1 = a_row + (((4 + quad) ^ (col / 2)) * 16);
    const unsigned w_lane = base + wave_n * kWaveTilesN * 2048 + lane * 16;

    floatx4 acc[kWaveTilesN][WM];     // acc[nt][mt][i] = C[m = mt*16 + col][n = nt*16 + quad*4 + i] of the wave's part
#pragma unroll
    for (int nt = 0; nt < kWaveTilesN; ++nt)
#pragma unroll
        for (int mt = 0; mt < WM; ++mt) acc[nt][mt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

    if (first_stage < stages) {
        int stage = first_stage;
        copy_stage(stage, 0);
        copy_stage(stage + 1, 1);
        TiledOperands<WM> even, odd;      // of a stage's first and second k step
        // The first stage's loads of this wave have landed when only the second stage's are on their way.
        if (a_loads == A_TURNS) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(A_TURNS + 4) : "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" :: "n"(A_TURNS + 3) : "memory");
        __builtin_amdgcn_s_barrier();
        read_operands<WM, 0>(even, a_step0, w_lane, std::make_integer_sequence<int, 4 + WM>{});
        // A stage that lies in slot SLOT. Its first step is multiplied while its second is read. Then the wave's
        // loads of the next stage have landed; after the barrier everyone's have, and everyone has read this stage,
        // whose slot the stage after next may take. The second step is multiplied while the next stage's first is read.
#define MLL_TILED_STAGE(SLOT)                                                                              \
    {                                                                                                      \
        operands_arrived<false>(even);                                                                     \
        products<WM, 1>(acc, even, odd, a_step1 + SLOT * kSlotBytes, w_lane + SLOT * kSlotBytes, std::make_integer_sequence<int, WM>{}); \
        operands_arrived<true>(odd);                                                                       \
        __builtin_amdgcn_s_barrier();                                                                      \
        copy_stage(stage + 2, SLOT);                                                                       \
        products<WM, 0>(acc, odd, even, a_step0 + (1 - SLOT) * kSlotBytes, w_lane + (1 - SLOT) * kSlotBytes, std::make_integer_sequence<int, WM>{}); \
        ++stage;                                                                                           \
    }
        // Two stages a round; a stage past the end multiplies by zeros.
        while (stage < stages) {
            MLL_TILED_STAGE(0)
            MLL_TILED_STAGE(1)
        }
#undef MLL_TILED_STAGE
        // No load may be on its way into LDS when the workgroup ends, and the last products must have written
        // their results before these are read (the compiler does not know that the asm statements are products).
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
    }

    if constexpr (EPILOGUE == 3) {
        // The lane's 4 columns of a tile lie in one head (head_dim is a multiple of 16). In a query or key head
        // columns 2p and 2p + 1 hold dims p and p + n_freq, the two that rotate together, so the lane's columns are
        // dims p, p + n_freq, p + 1, p + 1 + n_freq with p even: two neighbours in each half, stored as one word
        // each. Dims beyond the rotated ones, and values, are in place.
        const CacheLayout layout(store.kv_heads, store.page_size, store.head_dim);
#pragma unroll
        for (int nt = 0; nt < kWaveTilesN; ++nt) {
            const int column = (n_tile0 + wave_n * kWaveTilesN + nt) * 16 + quad * 4;
            if (column >= n) continue;
            const int head = column / store.head_dim, within = column % store.head_dim;
            const bool is_query = head < store.heads;
            const bool is_value = head >= store.heads + store.kv_heads;
            const bool rotate = !is_value && within + 3 < 2 * store.n_freq;        // both pairs or, n_freq being even here, none
            const int pair = within / 2;
            // dims of the lane's four results, in the order of the accumulator
            int dim[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) dim[i] = rotate ? pair + i / 2 + (i % 2) * store.n_freq : within + i;
            float bias[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if (store.bias) {
#pragma unroll
                for (int i = 0; i < 4; ++i) bias[i] = store.bias[head * store.head_dim + dim[i]];
            }
#pragma unroll
            for (int mt = 0; mt < WM; ++mt) {
                const int row = m0 + wave_m * (WM * 16) + mt * 16 + col;
                if (row >= m) continue;
                float y[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) y[i] = acc[nt][mt][i] + bias[i];
                if (rotate) {
                    const floatx4 cs = *reinterpret_cast<const floatx4*>(store.cos_sin + (static_cast<int64_t>(row) * store.n_freq + pair) * 2);
                    const float x0 = y[0], x1 = y[1], x2 = y[2], x3 = y[3];
                    y[0] = rotate_first(x0, x1, cs[0], cs[1]);
                    y[1] = rotate_second(x0, x1, cs[0], cs[1]);
                    y[2] = rotate_first(x2, x3, cs[2], cs[3]);
                    y[3] = rotate_second(x2, x3, cs[2], cs[3]);
                }
                // y[0], y[2] are neighbours in dim (dim[0], dim[0] + 1) when rotated, and so are y[1], y[3]
                bf16x2 low, high;
                if (rotate) {
                    low[0] = static_cast<__bf16>(y[0]); low[1] = static_cast<__bf16>(y[2]);
                    high[0] = static_cast<__bf16>(y[1]); high[1] = static_cast<__bf16>(y[3]);
                } else {
                    low[0] = static_cast<__bf16>(y[0]); low[1] = static_cast<__bf16>(y[1]);
                    high[0] = static_cast<__bf16>(y[2]); high[1] = static_cast<__bf16>(y[3]);
                }
                const int low_dim = dim[0], high_dim = rotate ? dim[1] : dim[2];
                if (is_query) {
                    bf16* q_row = static_cast<bf16*>(store.q_out) + (static_cast<int64_t>(row) * store.heads + head) * store.head_dim;
                    *reinterpret_cast<bf16x2*>(q_row + low_dim) = low;
                    *reinterpret_cast<bf16x2*>(q_row + high_dim) = high;
                    continue;
                }
                if (!store.slot_mapping) continue;
                const int slot = store.slot_mapping[row];
                if (slot < 0) continue;
                const int page = slot / store.page_size, offset = slot % store.page_size;
                if (!is_value) {
                    bf16* pages = static_cast<bf16*>(store.k_cache);        // two neighbouring dims are neighbours in a page of keys
                    *reinterpret_cast<bf16x2*>(pages + layout.k_at(page, head - store.heads, offset, low_dim)) = low;
                    *reinterpret_cast<bf16x2*>(pages + layout.k_at(page, head - store.heads, offset, high_dim)) = high;
                } else {
                    bf16* pages = static_cast<bf16*>(store.v_cache);        // and 8 elements apart in a page of values
                    const int kv_head = head - store.heads - store.kv_heads;
#pragma unroll
                    for (int i = 0; i < 4; ++i) pages[layout.v_at(page, kv_head, offset, within + i)] = from_float<bf16>(y[i]);
                }
            }
        }
        return;
    }
#pragma unroll
    for (int mt = 0; mt < WM; ++mt) {
        const int row = m0 + wave_m * (WM * 16) + mt * 16 + col;
        if (row >= m) continue;
#pragma unroll
        for (int nt = 0; nt < kWaveTilesN; ++nt) {
            const int column = (n_tile0 + wave_n * kWaveTilesN + nt) * 16 + quad * 4;
            if (EPILOGUE == 0) {
                float* target = static_cast<float*>(out) + (static_cast<int64_t>(blockIdx.y) * m + row) * n + column;
                if (column + 3 < n && n % 4 == 0) {
                    *reinterpret_cast<floatx4*>(target) = acc[nt][mt];
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (column + i < n) target[i] = acc[nt][mt][i];
                }
            } else if (EPILOGUE == 1) {
                bf16* target = static_cast<bf16*>(out) + static_cast<int64_t>(row) * n + column;
                if (column + 3 < n && n % 4 == 0) {
                    bf16x4 four;
#pragma unroll
                    for (int i = 0; i < 4; ++i) four[i] = static_cast<__bf16>(acc[nt][mt][i]);
                    *reinterpret_cast<bf16x4*>(target) = four;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (column + i < n) target[i] = from_float<bf16>(acc[nt][mt][i]);
                }
            } else {
                bf16* target = static_cast<bf16*>(out) + static_cast<int64_t>(row) * (n / 2) + column / 2;
                if (column + 3 < n && n % 4 == 0) {
                    bf16x2 two;
#pragma unroll
                    for (int i = 0; i < 2; ++i) two[i] = static_cast<__bf16>(silu_fast(acc[nt][mt][2 * i]) * acc[nt][mt][2 * i + 1]);
                    *reinterpret_cast<bf16x2*>(target) = two;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i += 2)
                        if (column + i < n) target[i / 2] = from_float<bf16>(silu_fast(acc[nt][mt][i]) * acc[nt][mt][i + 1]);
                }
            }
        }
    }
}

template <int EPILOGUE, int WM>
static int launch_tiled_rows(const void* a, const void* w_packed, void* out, int m, int n, int k, int splits, hipStream_t stream,
                             const MllQkvStore& store) {
    const int n_tiles = (n + 15) / 16, k_steps = k / 32;
    const int m_blocks = (m + 32 * WM - 1) / (32 * WM), n_blocks = (n + kTileN - 1) / kTileN;
    const dim3 grid(8 * ((m_blocks * n_blocks + 7) / 8), splits);
    gemm_tiled_kernel<EPILOGUE, WM><<<grid, kTiledThreads, 0, stream>>>(static_cast<const bf16*>(a), static_cast<const bf16*>(w_packed),
                                                                        out, m, n, k, n_tiles, k_steps, m_blocks, n_blocks, store);
    return check_launch("gemm_tiled");
}

// How many rows a workgroup's tile gets: the height that is done first, if every round of 256 workgroups takes as
// long as a tile's loads (a stage of A and W: rows + 256 columns), which is what bounds this kernel. 2048 x 4608
// in tiles of 256 rows is 144 tiles, a round in which 112 compute units have none; in tiles of 160 rows 234.
// Every output's additions are the same whatever the height.
static int choose_tile_rows(int m, int n, int splits) {
    const int n_blocks = (n + kTileN - 1) / kTileN;
    int best = 256;
    int64_t best_cost = -1;
    for (int rows : {256, 192, 160, 128}) {
        const int64_t blocks = static_cast<int64_t>((m + rows - 1) / rows) * n_blocks * splits;
        const int64_t cost = ((blocks + 255) / 256) * (rows + kTileN);
        if (best_cost < 0 || cost < best_cost) best = rows, best_cost = cost;
    }
    return best;
}

template <int EPILOGUE>
static int launch_tiled(const void* a, const void* w_packed, void* out, int m, int n, int k, int splits, int tile_rows,
                        hipStream_t stream, const MllQkvStore& store = MllQkvStore{}) {
    if (tile_rows == 0) tile_rows = choose_tile_rows(m, n, splits);
    switch (tile_rows) {
        case 256: return launch_tiled_rows<EPILOGUE, 8>(a, w_packed, out, m, n, k, splits, stream, store);
        case 192: return launch_tiled_rows<EPILOGUE, 6>(a, w_packed, out, m, n, k, splits, stream, store);
        case 160: return launch_tiled_rows<EPILOGUE, 5>(a, w_packed, out, m, n, k, splits, stream, store);
        case 128: return launch_tiled_rows<EPILOGUE, 4>(a, w_packed, out, m, n, k, splits, stream, store);
        default: return fail("gemm_tiled: a tile has 256, 192, 160 or 128 rows (0: chosen here)");
    }
}

}  // namespace mll

using namespace mll;

extern "C" int mll_tiled_tile_rows(int m, int n, int splits) { return choose_tile_rows(m, n, splits < 1 ? 1 : splits); }

extern "C" int mll_gemm_tiled(const void* a, const void* w_packed, void* out, int epilogue, int m, int n, int k,
                              int splits, int tile_rows, hipStream_t stream) {
    MLL_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm_tiled: sizes must be positive");
    MLL_REQUIRE(k % 32 == 0, "gemm_tiled: k must be a multiple of 32");
    MLL_REQUIRE(splits >= 1 && splits <= 64 && (splits == 1 || epilogue == 0), "gemm_tiled: only the float32 epilogue takes k in parts");
    MLL_REQUIRE(static_cast<int64_t>(kTileN) * k < (int64_t{1} << 30), "gemm_tiled: k is too long");
    MLL_REQUIRE(epilogue != 2 || n % 2 == 0, "gemm_tiled: the gated epilogue needs an even number of weight rows");
    MLL_REQUIRE(reinterpret_cast<uintptr_t>(a) % 16 == 0, "gemm_tiled: the activations must be 16-byte aligned");
    if (m == 0) return 0;
    switch (epilogue) {
        case 0: return launch_tiled<0>(a, w_packed, out, m, n, k, splits, tile_rows, stream);
        case 1: return launch_tiled<1>(a, w_packed, out, m, n, k, splits, tile_rows, stream);
        case 2: return launch_tiled<2>(a, w_packed, out, m, n, k, splits, tile_rows, stream);
        default: return fail("gemm_tiled: unknown epilogue");
    }
}

extern "C" int mll_gemm_tiled_qkv(const void* a, const void* w_packed, int m, int k, const MllQkvStore* store, int tile_rows,
                                  hipStream_t stream) {
    MLL_REQUIRE(store != nullptr, "gemm_tiled_qkv: no store");
    MLL_REQUIRE(m >= 0 && k > 0 && k % 32 == 0, "gemm_tiled_qkv: k must be a positive multiple of 32");
    MLL_REQUIRE(static_cast<int64_t>(kTileN) * k < (int64_t{1} << 30), "gemm_tiled_qkv: k is too long");
    MLL_REQUIRE(store->heads > 0 && store->kv_heads >= 0 && store->head_dim > 0 && store->head_dim % 16 == 0,
                "gemm_tiled_qkv: head_dim must be a multiple of 16");
    MLL_REQUIRE(store->n_freq >= 0 && store->n_freq % 2 == 0 && 2 * store->n_freq <= store->head_dim,
                "gemm_tiled_qkv: the number of rotary pairs must be even and at most head_dim / 2");
    MLL_REQUIRE(store->n_freq == 0 || (store->cos_sin && reinterpret_cast<uintptr_t>(store->cos_sin) % 16 == 0),
                "gemm_tiled_qkv: rotation needs a 16-byte aligned cos/sin table");
    MLL_REQUIRE(store->q_out && reinterpret_cast<uintptr_t>(store->q_out) % 4 == 0, "gemm_tiled_qkv: no place for the queries");
    MLL_REQUIRE(!store->slot_mapping || (store->k_cache && store->v_cache && store->page_size > 0 && store->page_size % 16 == 0),
                "gemm_tiled_qkv: a slot mapping needs both caches and pages of a multiple of 16 positions");
    MLL_REQUIRE(reinterpret_cast<uintptr_t>(a) % 16 == 0, "gemm_tiled_qkv: the activations must be 16-byte aligned");
    if (m == 0) return 0;
    const int n = (store->heads + 2 * store->kv_heads) * store->head_dim;
    return launch_tiled<3>(a, w_packed, nullptr, m, n, k, 1, tile_rows, stream, *store);
}
