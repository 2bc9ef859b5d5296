// Matrix products with many rows (prompts): C = A . W^T for bfloat16 A [M, K] (row-major) and the same packed
// weight the streaming kernel reads ([N/16][K/32][4][16][8]), on v_mfma_f32_16x16x32_bf16.
//
// A workgroup of 8 waves (two on every SIMD, so that one wave's reads from LDS run beside the other's products)
// owns a 256 x 256 tile of C, a wave 128 x 64 of it (8 x 4 MFMA tiles, 128 accumulator registers). Per stage of
// 64 of k the workgroup's 2 x (16 + 16) pieces of A and W (1 KB each: 16 rows x 32 k in MFMA operand order) are
// brought into LDS by direct global-to-LDS loads, one piece per wave-wide instruction, two stages deep (128 KB):
// the next stage's pieces arrive while this stage's 64 products per wave run. The stages are separate LDS
// variables: of one array the compiler cannot tell that a load into one half does not write what is read from
// the other, and waits for the load before every read. A piece of W is contiguous in memory as it is; a piece of
// A is gathered from 16 rows, 64 bytes of each. Addresses are a base the scalar unit steps along k and one
// offset per lane and piece.
// Workgroups that share a tile of W are numbered so that they run on the same XCD and share its L2.
#include "common.h"
#include "microllm_hip.h"

namespace mll {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kTileM = 256, kTileN = 256;
constexpr int kTiledWaves = 8;
constexpr int kTiledThreads = kTiledWaves * kWave;
constexpr int kPieceElements = 512;                       // 16 rows x 32 k
constexpr int kPiecesPerSide = kTileM / 16;               // 16 pieces of A and 16 of W per k step
constexpr int kStageSteps = 2;                            // k steps of 32 in a stage
constexpr int kSideElements = kStageSteps * kPiecesPerSide * kPieceElements;   // 32 KB of A or of W in a stage
constexpr int kWaveTilesM = 8, kWaveTilesN = 4;           // a wave's 128 x 64 of C

union TFrag {
    bf16x8 v;
    uint4 raw;
};

__device__ inline float silu_fast(float value) { return value / (1.0f + __expf(-value)); }

// EPILOGUE: 0 = float32 [M, N]; 1 = bfloat16 [M, N]; 2 = bfloat16 [M, N / 2] = silu(even rows of W) * (odd rows).
// With epilogue 0 the stages of k may be dealt to gridDim.y workgroups, each writing its own [M, N] of partial sums.
template <int EPILOGUE>
__global__ __launch_bounds__(kTiledThreads, 1) void gemm_tiled_kernel(const bf16* __restrict__ a, const bf16* __restrict__ w_packed,
                                                                      void* __restrict__ out, int m, int n, int k, int n_tiles,
                                                                      int k_steps, int m_blocks, int n_blocks) {
    __shared__ __align__(16) bf16 a_even[kSideElements];      // [k step in the stage][piece][512]
    __shared__ __align__(16) bf16 w_even[kSideElements];
    __shared__ __align__(16) bf16 a_odd[kSideElements];
    __shared__ __align__(16) bf16 w_odd[kSideElements];

    // Workgroups 8 apart in number run on one XCD: give them the tiles of C that share a tile of W.
    const int xcd = blockIdx.x % 8;
    const int local = blockIdx.x / 8;
    const int n_block = (local / m_blocks) * 8 + xcd;
    const int m_block = local % m_blocks;
    if (n_block >= n_blocks) return;

    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int col = lane % 16, quad = lane / 16;
    const int wave_m = wave / 4, wave_n = wave % 4;        // which 128 x 64 of the tile
    const int m0 = m_block * kTileM, n_tile0 = n_block * (kTileN / 16);

    // What this wave copies per k step: pieces 2 * wave and 2 * wave + 1 of A and of W.
    const bf16* a_block = a + static_cast<int64_t>(m0) * k;
    int a_offset[2];          // of the lane's 16 bytes in the piece's rows, from a_block, at k = 0
    const bf16* w_piece[2];   // the piece at k step 0 (the same for all lanes)
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int piece = wave * 2 + p;
        const int row = min(piece * 16 + col, m - 1 - m0);            // rows past the end repeat the last one
        a_offset[p] = row * k + quad * 8;
        const int tile = min(n_tile0 + piece, n_tiles - 1);
        w_piece[p] = w_packed + static_cast<int64_t>(tile) * k_steps * kPieceElements;
    }
    auto copy_stage = [&](int stage, bf16* a_stage, bf16* w_stage) {
#pragma unroll
        for (int step = 0; step < kStageSteps; ++step) {
            const int ks = stage * kStageSteps + step;
            if (ks >= k_steps) break;
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const int piece = wave * 2 + p;
                const bf16* a_source = a_block + ks * 32 + a_offset[p];
                const bf16* w_source = w_piece[p] + static_cast<int64_t>(ks) * kPieceElements + lane * 8;
                bf16* a_place = a_stage + (step * kPiecesPerSide + piece) * kPieceElements;
                bf16* w_place = w_stage + (step * kPiecesPerSide + piece) * kPieceElements;
                __builtin_amdgcn_global_load_lds(a_source, a_place, 16, 0, 0);
                __builtin_amdgcn_global_load_lds(w_source, w_place, 16, 0, 0);
            }
        }
    };

    floatx4 acc[kWaveTilesN][kWaveTilesM];     // acc[nt][mt][i] = C[m = mt*16 + col][n = nt*16 + quad*4 + i] of the wave's part
#pragma unroll
    for (int nt = 0; nt < kWaveTilesN; ++nt)
#pragma unroll
        for (int mt = 0; mt < kWaveTilesM; ++mt) acc[nt][mt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

    auto multiply_stage = [&](int stage, const bf16* a_stage, const bf16* w_stage) {
#pragma unroll
        for (int step = 0; step < kStageSteps; ++step) {
            if (stage * kStageSteps + step >= k_steps) break;
            TFrag a_frag[kWaveTilesM], w_frag[kWaveTilesN];
#pragma unroll
            for (int t = 0; t < kWaveTilesM; ++t)
                a_frag[t].raw = *reinterpret_cast<const uint4*>(
                    a_stage + (step * kPiecesPerSide + wave_m * kWaveTilesM + t) * kPieceElements + lane * 8);
#pragma unroll
            for (int t = 0; t < kWaveTilesN; ++t)
                w_frag[t].raw = *reinterpret_cast<const uint4*>(
                    w_stage + (step * kPiecesPerSide + wave_n * kWaveTilesN + t) * kPieceElements + lane * 8);
#pragma unroll
            for (int nt = 0; nt < kWaveTilesN; ++nt)
#pragma unroll
                for (int mt = 0; mt < kWaveTilesM; ++mt)
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_frag[nt].v, a_frag[mt].v, acc[nt][mt], 0, 0, 0);
        }
    };
    auto landed = [&]() {
        wait_for_loads();    // this wave's pieces of the stage are in LDS
        __syncthreads();     // everyone's are, and everyone is done with the stage before
    };

    const int all_stages = (k_steps + kStageSteps - 1) / kStageSteps;
    const int stages_per_split = (all_stages + gridDim.y - 1) / gridDim.y;
    const int first_stage = blockIdx.y * stages_per_split;
    const int stages = min(all_stages, first_stage + stages_per_split);
    if (first_stage < stages) copy_stage(first_stage, a_even, w_even);
    for (int stage = first_stage; stage < stages; stage += 2) {
        landed();
        if (stage + 1 < stages) copy_stage(stage + 1, a_odd, w_odd);
        multiply_stage(stage, a_even, w_even);
        if (stage + 1 < stages) {
            landed();
            if (stage + 2 < stages) copy_stage(stage + 2, a_even, w_even);
            multiply_stage(stage + 1, a_odd, w_odd);
        }
    }

#pragma unroll
    for (int mt = 0; mt < kWaveTilesM; ++mt) {
        const int row = m0 + wave_m * 128 + mt * 16 + col;
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

template <int EPILOGUE>
static int launch_tiled(const void* a, const void* w_packed, void* out, int m, int n, int k, int splits, hipStream_t stream) {
    const int n_tiles = (n + 15) / 16, k_steps = k / 32;
    const int m_blocks = (m + kTileM - 1) / kTileM, n_blocks = (n + kTileN - 1) / kTileN;
    const dim3 grid(8 * ((n_blocks + 7) / 8) * m_blocks, splits);
    gemm_tiled_kernel<EPILOGUE><<<grid, kTiledThreads, 0, stream>>>(static_cast<const bf16*>(a), static_cast<const bf16*>(w_packed),
                                                            out, m, n, k, n_tiles, k_steps, m_blocks, n_blocks);
    return check_launch("gemm_tiled");
}

}  // namespace mll

using namespace mll;

extern "C" int mll_gemm_tiled(const void* a, const void* w_packed, void* out, int epilogue, int m, int n, int k,
                              int splits, hipStream_t stream) {
    MLL_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm_tiled: sizes must be positive");
    MLL_REQUIRE(k % 32 == 0, "gemm_tiled: k must be a multiple of 32");
    MLL_REQUIRE(splits >= 1 && splits <= 64 && (splits == 1 || epilogue == 0), "gemm_tiled: only the float32 epilogue takes k in parts");
    MLL_REQUIRE(static_cast<int64_t>(kTileM) * k < (int64_t{1} << 30), "gemm_tiled: k is too long");
    MLL_REQUIRE(epilogue != 2 || n % 2 == 0, "gemm_tiled: the gated epilogue needs an even number of weight rows");
    MLL_REQUIRE(reinterpret_cast<uintptr_t>(a) % 16 == 0, "gemm_tiled: the activations must be 16-byte aligned");
    if (m == 0) return 0;
    switch (epilogue) {
        case 0: return launch_tiled<0>(a, w_packed, out, m, n, k, splits, stream);
        case 1: return launch_tiled<1>(a, w_packed, out, m, n, k, splits, stream);
        case 2: return launch_tiled<2>(a, w_packed, out, m, n, k, splits, stream);
        default: return fail("gemm_tiled: unknown epilogue");
    }
}
