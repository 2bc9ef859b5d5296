// Matrix products with few rows (decoding): C = A . W^T for bfloat16 A [M <= 64, K] and a weight that was
// packed once, at load time, into the order the MFMA consumes it, so that a wave streams its 16 rows of W as
// consecutive 1 KB pieces. The kernel is bound by reading W once from HBM.
//
// Packed layout: [N/16][K/32][quad 0..3][row 0..15][8 elements]; lane (row + 16 * quad) of a wave reads its
// 16 bytes of piece (n_tile, k_step) at byte offset lane * 16: the A operand of v_mfma_f32_16x16x32_bf16.
// The product is computed transposed (C^T = W . A^T): the activations are the B operand, 16 rows per tile.
// A workgroup owns NT tiles of W; its waves (1 to 16, more when W has few rows, so that the GPU is filled)
// take the k steps in turn and their sums are added in wave order through LDS: the result is the same in
// every run and does not depend on the other rows of A.
#include "cache_layout.h"
#include "common.h"
#include "microllm_hip.h"

namespace mll {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));


constexpr int kChunk = 8;   // k steps a wave takes in a row

union Piece {
    bf16x8 v;
    uintx4 raw;
};

__device__ inline float silu_f(float value) {
    return value / (1.0f + __expf(-value));
}

// EPILOGUE: 0 = float32 [M, N]; 1 = bfloat16 [M, N]; 2 = bfloat16 [M, N / 2] = silu(even rows of W) * (odd rows).
// 3 = the q/k/v projection of an attention layer finished in place: bias, rotation of the position, queries to
// `q_out`, keys and values into their pages (at most 16 rows; see MllQkvStore).
// TEMPORAL: W is read with ordinary loads instead of non-temporal ones (measured on MI355X: better for weights
// of a few tens of MB, worse for the large ones).
template <int MT, int NT, int EPILOGUE, bool TEMPORAL>
__global__ __launch_bounds__(1024) void gemm_skinny_kernel(
    const bf16* __restrict__ a, const bf16* __restrict__ w_packed, void* __restrict__ out,
    int m, int n, int k, int n_tiles, int k_steps, MllQkvStore store) {
    extern __shared__ float reduce_shared[];   // [waves][NT * MT][64 lanes][4]
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int waves = blockDim.x / kWave;
    const int col = lane % 16, quad = lane / 16;
    const int tile0 = blockIdx.x * NT;

    floatx4 acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

    const bf16* w_ptr[NT];
    bool w_live[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        w_live[nt] = tile0 + nt < n_tiles;
        w_ptr[nt] = w_packed + static_cast<int64_t>(w_live[nt] ? tile0 + nt : tile0) * k_steps * 512 + lane * 8;
    }
    const bf16* a_ptr[MT];
    bool a_live[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int row = mt * 16 + col;
        a_live[mt] = row < m;
        a_ptr[mt] = a + static_cast<int64_t>(a_live[mt] ? row : 0) * k + quad * 8;
    }

    // A wave takes kChunk consecutive k steps at a time, then skips what the other waves take; which k steps a
    // wave sums, and in which order, depends on (n, k) alone, not on the number of rows or tiles. The loads of
    // DEPTH steps are issued before their products, so that a wave keeps several KB of W in flight.
    constexpr int DEPTH = (MT + NT <= 2) ? 8 : ((MT + NT <= 4) ? 4 : 2);
    for (int chunk = wave * kChunk; chunk < k_steps; chunk += waves * kChunk) {
#pragma unroll
        for (int base = chunk; base < chunk + kChunk; base += DEPTH) {
            Piece w_piece[DEPTH][NT];
            Piece a_piece[DEPTH][MT];
#pragma unroll
            for (int u = 0; u < DEPTH; ++u) {
                const int ks = base + u;
                const bool live = ks < k_steps;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    w_piece[u][nt].raw = uintx4{0u, 0u, 0u, 0u};
                    if (live && w_live[nt])
                        w_piece[u][nt].raw =
                            TEMPORAL ? *reinterpret_cast<const uintx4*>(w_ptr[nt] + static_cast<int64_t>(ks) * 512)
                                     : __builtin_nontemporal_load(
                                           reinterpret_cast<const uintx4*>(w_ptr[nt] + static_cast<int64_t>(ks) * 512));
                }
                const int k_offset = ks * 32;
                const bool in_k = live && k_offset + quad * 8 < k;
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    a_piece[u][mt].raw = uintx4{0u, 0u, 0u, 0u};
                    if (a_live[mt] && in_k) a_piece[u][mt].raw = *reinterpret_cast<const uintx4*>(a_ptr[mt] + k_offset);
                }
            }
#pragma unroll
            for (int u = 0; u < DEPTH; ++u)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_piece[u][nt].v, a_piece[u][mt].v, acc[nt][mt], 0, 0, 0);
        }
    }

    // The waves' sums, added in wave order by wave 0.
    if (waves > 1) {
        floatx4* slots = reinterpret_cast<floatx4*>(reduce_shared);
        if (wave > 0) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) slots[((wave - 1) * NT * MT + nt * MT + mt) * kWave + lane] = acc[nt][mt];
        }
        __syncthreads();
        if (wave > 0) return;
        for (int other = 0; other < waves - 1; ++other)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[nt][mt] += slots[(other * NT * MT + nt * MT + mt) * kWave + lane];
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
                float* target = static_cast<float*>(out) + static_cast<int64_t>(row) * n;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int column = n_tile * 16 + quad * 4 + i;
                    if (column < n) target[column] = acc[nt][mt][i];
                }
            } else if (EPILOGUE == 1) {
                bf16* target = static_cast<bf16*>(out) + static_cast<int64_t>(row) * n;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int column = n_tile * 16 + quad * 4 + i;
                    if (column < n) target[column] = from_float<bf16>(acc[nt][mt][i]);
                }
            } else if (EPILOGUE == 2) {
                bf16* target = static_cast<bf16*>(out) + static_cast<int64_t>(row) * (n / 2);
#pragma unroll
                for (int i = 0; i < 4; i += 2) {
                    const int column = n_tile * 8 + quad * 2 + i / 2;
                    if (column < n / 2) target[column] = from_float<bf16>(silu_f(acc[nt][mt][i]) * acc[nt][mt][i + 1]);
                }
            } else {
                // The lane's 4 columns lie in one head (head_dim is a multiple of 16). In a query or key head the
                // weight's rows were ordered so that columns 2p and 2p + 1 hold dims p and p + n_freq: the two that
                // rotate together.
                const int column = n_tile * 16 + quad * 4;
                if (column >= n) continue;
                const int head = column / store.head_dim, within = column % store.head_dim;
                const bool is_query = head < store.heads;
                const bool is_value = head >= store.heads + store.kv_heads;
                const int slot = store.slot_mapping ? store.slot_mapping[row] : -1;
                const CacheLayout layout(store.kv_heads, store.page_size, store.head_dim);
                bf16* q_row = static_cast<bf16*>(store.q_out) + (static_cast<int64_t>(row) * store.heads + head) * store.head_dim;
#pragma unroll
                for (int i = 0; i < 4; i += 2) {
                    const bool rotate = !is_value && within + i < 2 * store.n_freq;
                    const int pair = (within + i) / 2;
                    const int first = rotate ? pair : within + i;
                    const int second = rotate ? pair + store.n_freq : within + i + 1;
                    float x1 = acc[nt][mt][i], x2 = acc[nt][mt][i + 1];
                    if (store.bias) {
                        x1 += store.bias[head * store.head_dim + first];
                        x2 += store.bias[head * store.head_dim + second];
                    }
                    float y1 = x1, y2 = x2;
                    if (rotate) {
                        const float2 both = reinterpret_cast<const float2*>(store.cos_sin)[static_cast<int64_t>(row) * store.n_freq + pair];
                        const float c = both.x, sn = both.y;
                        y1 = x1 * c - x2 * sn;
                        y2 = x1 * sn + x2 * c;
                    }
                    if (is_query) {
                        q_row[first] = from_float<bf16>(y1);
                        q_row[second] = from_float<bf16>(y2);
                    } else if (slot >= 0 && !is_value) {
                        bf16* pages = static_cast<bf16*>(store.k_cache);
                        pages[layout.k_at(slot / store.page_size, head - store.heads, slot % store.page_size, first)] = from_float<bf16>(y1);
                        pages[layout.k_at(slot / store.page_size, head - store.heads, slot % store.page_size, second)] = from_float<bf16>(y2);
                    } else if (slot >= 0) {
                        bf16* pages = static_cast<bf16*>(store.v_cache);
                        const int kv_head = head - store.heads - store.kv_heads;
                        pages[layout.v_at(slot / store.page_size, kv_head, slot % store.page_size, first)] = from_float<bf16>(y1);
                        pages[layout.v_at(slot / store.page_size, kv_head, slot % store.page_size, second)] = from_float<bf16>(y2);
                    }
                }
            }
        }
    }
}

template <int MT, int NT, int EPILOGUE>
static void launch_one(const bf16* a, const bf16* w, void* out, int m, int n, int k, int n_tiles,
                       int k_steps, const MllQkvStore& store, hipStream_t stream) {
    const int groups = (n_tiles + NT - 1) / NT;
    // Waves per workgroup: enough that about eight thousand waves would stream W one tile each, at most 16, and
    // no more than there are chunks of k for them. A function of (n, k) alone, like the split of k it implies.
    int waves = 1;
    while (waves < 16 && n_tiles * waves * 2 <= 8192 && waves * 2 * kChunk <= k_steps) waves *= 2;
    const size_t lds = waves > 1 ? static_cast<size_t>(waves - 1) * NT * MT * kWave * sizeof(floatx4) : 0;
    const bool temporal = static_cast<int64_t>(n_tiles) * k_steps * 1024 < (64ll << 20);   // bytes of the packed weight
    if (temporal)
        gemm_skinny_kernel<MT, NT, EPILOGUE, true><<<groups, waves * kWave, lds, stream>>>(a, w, out, m, n, k, n_tiles, k_steps, store);
    else
        gemm_skinny_kernel<MT, NT, EPILOGUE, false><<<groups, waves * kWave, lds, stream>>>(a, w, out, m, n, k, n_tiles, k_steps, store);
}

template <int EPILOGUE>
static int launch_skinny(const void* a, const void* w_packed, void* out, int m, int n, int k,
                         const MllQkvStore& store, hipStream_t stream) {
    const int n_tiles = (n + 15) / 16;
    const int k_steps = (k + 31) / 32;
    const bf16* a_ = static_cast<const bf16*>(a);
    const bf16* w_ = static_cast<const bf16*>(w_packed);
    const int m_tiles = (m + 15) / 16;
    // Few tiles of W: one per workgroup, so that the GPU is filled. Many tiles of W, or several rows of A and at
    // least 128 workgroups left: two, so that every piece of A is used twice (all measured on MI355X; four tiles
    // a workgroup were slower).
    const bool wide = n_tiles >= 2048;
    if constexpr (EPILOGUE == 3) {
        if (m_tiles != 1) return fail("gemm_skinny: the q/k/v epilogue takes at most 16 rows");
        if (m > 4 && n_tiles >= 256) launch_one<1, 2, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, store, stream);
        else launch_one<1, 1, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, store, stream);
        return check_launch("gemm_skinny");
    }
    switch (m_tiles) {
        case 1:
            if (wide || (m > 4 && n_tiles >= 256)) launch_one<1, 2, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, store, stream);
            else launch_one<1, 1, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, store, stream);
            break;
        case 2:
            if (wide) launch_one<2, 2, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, store, stream);
            else launch_one<2, 1, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, store, stream);
            break;
        case 3: launch_one<3, 2, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, store, stream); break;
        case 4: launch_one<4, 2, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, store, stream); break;
        default: return fail("gemm_skinny: more than 64 rows");
    }
    return check_launch("gemm_skinny");
}

}  // namespace mll

using namespace mll;

extern "C" int mll_gemm_skinny(const void* a, const void* w_packed, void* out, int epilogue, int m, int n, int k,
                               hipStream_t stream) {
    MLL_REQUIRE(m >= 0 && m <= 64, "gemm_skinny: takes at most 64 rows");
    MLL_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_skinny: k must be a positive multiple of 8");
    MLL_REQUIRE(epilogue != 2 || n % 2 == 0, "gemm_skinny: the gated epilogue needs an even number of weight rows");
    if (m == 0) return 0;
    switch (epilogue) {
        case 0: return launch_skinny<0>(a, w_packed, out, m, n, k, MllQkvStore{}, stream);
        case 1: return launch_skinny<1>(a, w_packed, out, m, n, k, MllQkvStore{}, stream);
        case 2: return launch_skinny<2>(a, w_packed, out, m, n, k, MllQkvStore{}, stream);
        default: return fail("gemm_skinny: unknown epilogue");
    }
}

extern "C" int mll_gemm_skinny_qkv(const void* a, const void* w_packed, int m, int k, const MllQkvStore* store,
                                   hipStream_t stream) {
    MLL_REQUIRE(store != nullptr, "gemm_skinny_qkv: no epilogue description");
    MLL_REQUIRE(m >= 0 && m <= 16, "gemm_skinny_qkv: takes at most 16 rows");
    MLL_REQUIRE(k > 0 && k % 8 == 0, "gemm_skinny_qkv: k must be a positive multiple of 8");
    MLL_REQUIRE(store->heads > 0 && store->kv_heads >= 0, "gemm_skinny_qkv: bad head counts");
    MLL_REQUIRE(store->head_dim >= 16 && store->head_dim % 16 == 0, "gemm_skinny_qkv: head_dim must be a multiple of 16");
    MLL_REQUIRE(store->n_freq >= 0 && 2 * store->n_freq <= store->head_dim, "gemm_skinny_qkv: more rotary pairs than dims");
    MLL_REQUIRE(store->n_freq == 0 || store->cos_sin, "gemm_skinny_qkv: rotation needs the table of cos and sin");
    MLL_REQUIRE(store->q_out, "gemm_skinny_qkv: the query output is needed");
    MLL_REQUIRE(!store->slot_mapping || (store->k_cache && store->v_cache && store->page_size > 0 && store->page_size % 16 == 0),
                "gemm_skinny_qkv: writing pages needs both caches and a page size that is a multiple of 16");
    if (m == 0) return 0;
    const int n = (store->heads + 2 * store->kv_heads) * store->head_dim;
    return launch_skinny<3>(a, w_packed, nullptr, m, n, k, *store, stream);
}
