// Matrix products with many rows (prompts): C = A . W^T for bfloat16 A [M, K] (row-major) and the same packed
// weight the streaming kernel reads ([N/16][K/32][4][16][8]), on v_mfma_f32_16x16x32_bf16.
//
// A workgroup of 4 waves owns a 256 x 256 tile of C, a wave 128 x 128 of it (8 x 8 MFMA tiles, 256 accumulator
// registers). Per k step of 32 the workgroup's 16 + 16 pieces of A and W (1 KB each: 16 rows x 32 k in MFMA
// operand order) are brought into LDS by direct global-to-LDS loads, one piece per wave-wide instruction, two
// stages deep (64 KB): the next step's pieces arrive while this step's 64 products per wave run. A piece of W
// is contiguous in memory as it is; a piece of A is gathered from 16 rows, 64 bytes of each.
// Workgroups that share a tile of W are numbered so that they run on the same XCD and share its L2.
//
// This kernel reaches about half the library's rate on MI355X (0.5 against 1.0 PFLOP/s at 2048 rows); the engine
// takes it only where a weight is kept in the packed order alone.
#include "common.h"
#include "microllm_hip.h"

namespace mll {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kTileM = 256, kTileN = 256;
constexpr int kPieceElements = 512;                       // 16 rows x 32 k
constexpr int kPiecesPerSide = kTileM / 16;               // 16 pieces of A and 16 of W per k step
constexpr int kStageElements = 2 * kPiecesPerSide * kPieceElements;   // 32 KB
constexpr int kStages = 2;

union TFrag {
    bf16x8 v;
    uint4 raw;
};

__device__ inline float silu_fast(float value) { return value / (1.0f + __expf(-value)); }

// EPILOGUE: 0 = float32 [M, N]; 1 = bfloat16 [M, N]; 2 = bfloat16 [M, N / 2] = silu(even rows of W) * (odd rows).
template <int EPILOGUE>
__global__ __launch_bounds__(256, 1) void gemm_tiled_kernel(const bf16* __restrict__ a, const bf16* __restrict__ w_packed,
                                                            void* __restrict__ out, int m, int n, int k, int n_tiles,
                                                            int k_steps, int m_blocks, int n_blocks) {
    extern __shared__ __align__(16) bf16 stages[];         // [kStages][A pieces | W pieces][512]

    // Workgroups 8 apart in number run on one XCD: give them the tiles of C that share a tile of W.
    const int xcd = blockIdx.x % 8;
    const int local = blockIdx.x / 8;
    const int n_block = (local / m_blocks) * 8 + xcd;
    const int m_block = local % m_blocks;
    if (n_block >= n_blocks) return;

    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int col = lane % 16, quad = lane / 16;
    const int wave_m = wave / 2, wave_n = wave % 2;        // which 128 x 128 quarter of the tile
    const int m0 = m_block * kTileM, n_tile0 = n_block * (kTileN / 16);

    // What this wave copies per k step: pieces 4 * wave .. + 3 of A and of W.
    const bf16* a_source[4];
    const bf16* w_source[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int piece = wave * 4 + p;
        const int row = min(m0 + piece * 16 + col, m - 1);            // rows past the end repeat the last one
        a_source[p] = a + static_cast<int64_t>(row) * k + quad * 8;
        const int tile = min(n_tile0 + piece, n_tiles - 1);
        w_source[p] = w_packed + static_cast<int64_t>(tile) * k_steps * kPieceElements + lane * 8;
    }
    auto copy_step = [&](int ks, int stage) {
        bf16* base = stages + stage * kStageElements;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int piece = wave * 4 + p;
            __builtin_amdgcn_global_load_lds(a_source[p] + ks * 32, base + piece * kPieceElements, 16, 0, 0);
            __builtin_amdgcn_global_load_lds(w_source[p] + static_cast<int64_t>(ks) * kPieceElements,
                                             base + (kPiecesPerSide + piece) * kPieceElements, 16, 0, 0);
        }
    };

    floatx4 acc[8][8];     // [n tile][m tile] of the wave's quarter; acc[nt][mt][i] = C[m = mt*16 + col][n = nt*16 + quad*4 + i]
#pragma unroll
    for (int nt = 0; nt < 8; ++nt)
#pragma unroll
        for (int mt = 0; mt < 8; ++mt) acc[nt][mt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

    copy_step(0, 0);
    for (int ks = 0; ks < k_steps; ++ks) {
        const int stage = ks % kStages;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's pieces of step ks are in LDS
        __syncthreads();     // everyone's are, and everyone is done with step ks - 1's stage
        if (ks + 1 < k_steps) copy_step(ks + 1, (ks + 1) % kStages);
        const bf16* base = stages + stage * kStageElements;
        TFrag a_frag[8], w_frag[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            a_frag[t].raw = *reinterpret_cast<const uint4*>(base + (wave_m * 8 + t) * kPieceElements + lane * 8);
            w_frag[t].raw = *reinterpret_cast<const uint4*>(base + (kPiecesPerSide + wave_n * 8 + t) * kPieceElements + lane * 8);
        }
#pragma unroll
        for (int nt = 0; nt < 8; ++nt)
#pragma unroll
            for (int mt = 0; mt < 8; ++mt)
                acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_frag[nt].v, a_frag[mt].v, acc[nt][mt], 0, 0, 0);
    }

#pragma unroll
    for (int mt = 0; mt < 8; ++mt) {
        const int row = m0 + wave_m * 128 + mt * 16 + col;
        if (row >= m) continue;
#pragma unroll
        for (int nt = 0; nt < 8; ++nt) {
            const int column = (n_tile0 + wave_n * 8 + nt) * 16 + quad * 4;
            if (EPILOGUE == 0) {
                float* target = static_cast<float*>(out) + static_cast<int64_t>(row) * n + column;
                if (column + 3 < n && n % 4 == 0) {
                    *reinterpret_cast<floatx4*>(target) = acc[nt][mt];
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (column + i < n) target[i] = acc[nt][mt][i];
                }
            } else if (EPILOGUE == 1) {
                bf16* target = static_cast<bf16*>(out) + static_cast<int64_t>(row) * n + column;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (column + i < n) target[i] = from_float<bf16>(acc[nt][mt][i]);
            } else {
                bf16* target = static_cast<bf16*>(out) + static_cast<int64_t>(row) * (n / 2) + column / 2;
#pragma unroll
                for (int i = 0; i < 4; i += 2)
                    if (column + i < n) target[i / 2] = from_float<bf16>(silu_fast(acc[nt][mt][i]) * acc[nt][mt][i + 1]);
            }
        }
    }
}

template <int EPILOGUE>
static int launch_tiled(const void* a, const void* w_packed, void* out, int m, int n, int k, hipStream_t stream) {
    const int n_tiles = (n + 15) / 16, k_steps = k / 32;
    const int m_blocks = (m + kTileM - 1) / kTileM, n_blocks = (n + kTileN - 1) / kTileN;
    const int grid = 8 * ((n_blocks + 7) / 8) * m_blocks;
    const size_t lds = kStages * kStageElements * sizeof(bf16);       // 64 KB
    gemm_tiled_kernel<EPILOGUE><<<grid, 256, lds, stream>>>(static_cast<const bf16*>(a), static_cast<const bf16*>(w_packed),
                                                            out, m, n, k, n_tiles, k_steps, m_blocks, n_blocks);
    return check_launch("gemm_tiled");
}

}  // namespace mll

using namespace mll;

extern "C" int mll_gemm_tiled(const void* a, const void* w_packed, void* out, int epilogue, int m, int n, int k,
                              hipStream_t stream) {
    MLL_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm_tiled: sizes must be positive");
    MLL_REQUIRE(k % 32 == 0, "gemm_tiled: k must be a multiple of 32");
    MLL_REQUIRE(epilogue != 2 || n % 2 == 0, "gemm_tiled: the gated epilogue needs an even number of weight rows");
    MLL_REQUIRE(reinterpret_cast<uintptr_t>(a) % 16 == 0, "gemm_tiled: the activations must be 16-byte aligned");
    if (m == 0) return 0;
    switch (epilogue) {
        case 0: return launch_tiled<0>(a, w_packed, out, m, n, k, stream);
        case 1: return launch_tiled<1>(a, w_packed, out, m, n, k, stream);
        case 2: return launch_tiled<2>(a, w_packed, out, m, n, k, stream);
        default: return fail("gemm_tiled: unknown epilogue");
    }
}
