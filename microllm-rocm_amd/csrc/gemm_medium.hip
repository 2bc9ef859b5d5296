// Matrix products with 17 to 64 rows (decoding many requests, short portions of prompts): C = A . W^T for
// bfloat16 A [M, K] (row-major) and the packed weight the streaming kernel reads ([N/16][K/32][4][16][8]).
// Still bound by reading W once from HBM, but with this many rows the activations a wave needs per piece of W
// are several times the piece: here the 4 or 8 waves of a workgroup walk the same k steps, each over its own
// tiles of W, and share the activations through LDS (8 k steps at a time, double buffered, brought in MFMA
// operand order by all waves together). A wave keeps two batches of pieces of W in registers: one on its way
// while the other is multiplied.
//
// Where W has too few tiles to fill the GPU this way, k is split over `splits` workgroups (grid y), each of
// which writes its own float32 partial sum [split][M][N]; the consumer adds them in order. Which k steps a
// sum holds, and in which order, depends on (n, k, splits) alone: a row's result does not depend on the
// other rows.
#include "common.h"
#include "microllm_hip.h"

namespace mll {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

namespace medium {

constexpr int kStepsPerStage = 8;    // k steps of activations in one LDS buffer
constexpr int kBatch = 4;            // k steps of W a wave loads at a time; two batches make a stage

union Piece {
    bf16x8 v;
    uintx4 raw;
};

__device__ inline float silu_f(float value) { return value / (1.0f + __expf(-value)); }

template <int NT>
__device__ inline void load_batch(Piece (&pieces)[kBatch][NT], const bf16* const (&w_ptr)[NT], const bool (&w_live)[NT],
                                  int first_step, int end_step) {
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
        const int ks = first_step + u;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            pieces[u][nt].raw = uintx4{0u, 0u, 0u, 0u};
            if (ks < end_step && w_live[nt]) {
                const uintx4* source = reinterpret_cast<const uintx4*>(w_ptr[nt] + static_cast<int64_t>(ks) * 512);
                pieces[u][nt].raw = __builtin_nontemporal_load(source);      // W is read once a step: past the caches
            }
        }
    }
}

// EPILOGUE: 0 = float32 [splits][M, N]; 1 = bfloat16 [M, N]; 2 = bfloat16 [M, N / 2] = silu(even rows of W) * (odd
// rows). 1 and 2 need splits == 1.
template <int MT, int NT, int kWaves, int EPILOGUE>
__global__ __launch_bounds__(kWaves * kWave) void gemm_medium_kernel(
    const bf16* __restrict__ a, const bf16* __restrict__ w_packed, void* __restrict__ out,
    int m, int n, int k, int n_tiles, int k_steps, int steps_per_split) {
    constexpr int kStagePieces = MT * kStepsPerStage;             // pieces of A in a buffer, 1 KB each
    constexpr int kPiecesPerWave = kStagePieces / kWaves;
    static_assert(kStagePieces % kWaves == 0, "the waves share the copying evenly");
    extern __shared__ uintx4 stage[];                             // [2][MT][kStepsPerStage][64 lanes]

    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int col = lane % 16, quad = lane / 16;
    const int tile0 = (blockIdx.x * kWaves + wave) * NT;
    const int first_step = blockIdx.y * steps_per_split;
    const int end_step = min(k_steps, first_step + steps_per_split);
    const int n_stages = (end_step - first_step + kStepsPerStage - 1) / kStepsPerStage;

    const bf16* w_ptr[NT];
    bool w_live[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        w_live[nt] = tile0 + nt < n_tiles;
        w_ptr[nt] = w_packed + static_cast<int64_t>(w_live[nt] ? tile0 + nt : 0) * k_steps * 512 + lane * 8;
    }

    // This wave's share of a buffer: pieces wave, wave + kWaves, ...; piece p holds rows 16 * (p / 8) .. + 15 at k step p % 8.
    auto load_share = [&](uintx4 (&share)[kPiecesPerWave], int stage_first_step) {
#pragma unroll
        for (int j = 0; j < kPiecesPerWave; ++j) {
            const int piece = wave + kWaves * j;
            const int row = (piece / kStepsPerStage) * 16 + col;
            const int ks = stage_first_step + piece % kStepsPerStage;
            const int k_offset = ks * 32 + quad * 8;
            share[j] = uintx4{0u, 0u, 0u, 0u};
            if (row < m && ks < end_step && k_offset < k)
                share[j] = *reinterpret_cast<const uintx4*>(a + static_cast<int64_t>(row) * k + k_offset);
        }
    };
    auto store_share = [&](const uintx4 (&share)[kPiecesPerWave], int buffer) {
#pragma unroll
        for (int j = 0; j < kPiecesPerWave; ++j)
            stage[(buffer * kStagePieces + wave + kWaves * j) * kWave + lane] = share[j];
    };

    floatx4 acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

    auto multiply = [&](const Piece (&pieces)[kBatch][NT], int buffer, int step_in_stage) {
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            Piece a_piece[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                a_piece[mt].raw = stage[(buffer * kStagePieces + mt * kStepsPerStage + step_in_stage + u) * kWave + lane];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pieces[u][nt].v, a_piece[mt].v, acc[nt][mt], 0, 0, 0);
        }
    };

    uintx4 share[kPiecesPerWave];
    Piece w_even[kBatch][NT], w_odd[kBatch][NT];
    load_share(share, first_step);
    load_batch<NT>(w_even, w_ptr, w_live, first_step, end_step);
    store_share(share, 0);
    __syncthreads();
    for (int s = 0; s < n_stages; ++s) {
        const int stage_step = first_step + s * kStepsPerStage;
        const int buffer = s % 2;
        if (s + 1 < n_stages) load_share(share, stage_step + kStepsPerStage);
        load_batch<NT>(w_odd, w_ptr, w_live, stage_step + kBatch, end_step);
        multiply(w_even, buffer, 0);
        load_batch<NT>(w_even, w_ptr, w_live, stage_step + kStepsPerStage, end_step);
        multiply(w_odd, buffer, kBatch);
        // The other buffer was last read in the stage before this one, and every wave has passed that stage's barrier.
        if (s + 1 < n_stages) store_share(share, 1 - buffer);
        __syncthreads();
    }

    // acc[nt][mt][i] = C[row mt*16 + col][column (tile0 + nt)*16 + quad*4 + i]
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int n_tile = tile0 + nt;
        if (n_tile >= n_tiles) continue;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int row = mt * 16 + col;
            if (row >= m) continue;
            if (EPILOGUE == 0) {
                float* target = static_cast<float*>(out) + (static_cast<int64_t>(blockIdx.y) * m + row) * n;
                const int column = n_tile * 16 + quad * 4;
                if (column + 3 < n && n % 4 == 0) {
                    *reinterpret_cast<floatx4*>(target + column) = acc[nt][mt];
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (column + i < n) target[column + i] = acc[nt][mt][i];
                }
            } else if (EPILOGUE == 1) {
                bf16* target = static_cast<bf16*>(out) + static_cast<int64_t>(row) * n;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int column = n_tile * 16 + quad * 4 + i;
                    if (column < n) target[column] = from_float<bf16>(acc[nt][mt][i]);
                }
            } else {
                bf16* target = static_cast<bf16*>(out) + static_cast<int64_t>(row) * (n / 2);
#pragma unroll
                for (int i = 0; i < 4; i += 2) {
                    const int column = n_tile * 8 + quad * 2 + i / 2;
                    if (column < n / 2) target[column] = from_float<bf16>(silu_f(acc[nt][mt][i]) * acc[nt][mt][i + 1]);
                }
            }
        }
    }
}

template <int MT, int NT, int kWaves, int EPILOGUE>
static void launch_one(const bf16* a, const bf16* w, void* out, int m, int n, int k, int n_tiles, int k_steps,
                       int splits, hipStream_t stream) {
    const dim3 grid((n_tiles + kWaves * NT - 1) / (kWaves * NT), splits);
    // Each split takes whole stages, so that the stages of a sum begin at the same k whatever the split.
    const int stages = (k_steps + kStepsPerStage - 1) / kStepsPerStage;
    const int steps_per_split = ((stages + splits - 1) / splits) * kStepsPerStage;
    const size_t lds = 2 * MT * kStepsPerStage * kWave * sizeof(uintx4);
    gemm_medium_kernel<MT, NT, kWaves, EPILOGUE><<<grid, kWaves * kWave, lds, stream>>>(a, w, out, m, n, k, n_tiles, k_steps, steps_per_split);
}

template <int EPILOGUE>
static int launch_medium(const void* a, const void* w_packed, void* out, int m, int n, int k, int tiles_per_wave,
                         int waves, int splits, hipStream_t stream) {
    const int n_tiles = (n + 15) / 16;
    const int k_steps = (k + 31) / 32;
    const bf16* a_ = static_cast<const bf16*>(a);
    const bf16* w_ = static_cast<const bf16*>(w_packed);
    const int m_tiles = (m + 15) / 16;
#define MLL_MEDIUM_CASE(MT)                                                                                          \
    case MT:                                                                                                         \
        if (tiles_per_wave == 2 && waves == 8) launch_one<MT, 2, 8, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, splits, stream); \
        else if (tiles_per_wave == 2) launch_one<MT, 2, 4, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, splits, stream);          \
        else if (waves == 8) launch_one<MT, 1, 8, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, splits, stream);                  \
        else launch_one<MT, 1, 4, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, splits, stream);                                   \
        break;
    switch (m_tiles) {
        MLL_MEDIUM_CASE(1)
        MLL_MEDIUM_CASE(2)
        MLL_MEDIUM_CASE(3)
        MLL_MEDIUM_CASE(4)
        default: return fail("gemm_medium: more than 64 rows");
    }
#undef MLL_MEDIUM_CASE
    return check_launch("gemm_medium");
}

}  // namespace medium
}  // namespace mll

using namespace mll;

extern "C" int mll_gemm_medium(const void* a, const void* w_packed, void* out, int epilogue, int m, int n, int k,
                               int tiles_per_wave, int waves, int splits, hipStream_t stream) {
    MLL_REQUIRE(m >= 0 && m <= 64, "gemm_medium: takes at most 64 rows");
    MLL_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_medium: k must be a positive multiple of 8");
    MLL_REQUIRE(tiles_per_wave == 1 || tiles_per_wave == 2, "gemm_medium: a wave takes one or two tiles of the weight");
    MLL_REQUIRE(waves == 4 || waves == 8, "gemm_medium: workgroups of 4 or 8 waves");
    MLL_REQUIRE(splits >= 1 && splits <= 64, "gemm_medium: between 1 and 64 splits of k");
    MLL_REQUIRE(epilogue == 0 || splits == 1, "gemm_medium: only float32 partial sums can be split over k");
    MLL_REQUIRE(epilogue != 2 || n % 2 == 0, "gemm_medium: the gated epilogue needs an even number of weight rows");
    MLL_REQUIRE(reinterpret_cast<uintptr_t>(a) % 16 == 0, "gemm_medium: the activations must be 16-byte aligned");
    if (m == 0) return 0;
    switch (epilogue) {
        case 0: return medium::launch_medium<0>(a, w_packed, out, m, n, k, tiles_per_wave, waves, splits, stream);
        case 1: return medium::launch_medium<1>(a, w_packed, out, m, n, k, tiles_per_wave, waves, splits, stream);
        case 2: return medium::launch_medium<2>(a, w_packed, out, m, n, k, tiles_per_wave, waves, splits, stream);
        default: return fail("gemm_medium: unknown epilogue");
    }
}
