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
// `q_out`, keys and values into their pages (at most 16 rows; see MllQkvStore). 4 = the product is added to the
// float32 residual stream and the sum, times the next norm's weight, is written as the next product's input,
// with each workgroup's share of the rows' sums of squares (at most 16 rows; see MllResidualNorm).
// Whatever the epilogue, a row of the product is first multiplied by the factor that MllRowScale describes,
// if one is given (at most 16 rows).
// W is read past the caches (non-temporal loads): a step reads every weight once, and all of them together are far
// more than the caches hold. Measured on MI355X inside the decode step, against ordinary loads for weights under 64 MB:
// 7B sizes +1 % at batch 8, +1.6 % at batch 1, +0.7 % at batch 64; 0.5B sizes +4 % at batch 1, the same otherwise.
template <int MT, int NT, int EPILOGUE, bool SCALED, bool PAIRED>
__global__ __launch_bounds__(1024) void gemm_skinny_kernel(
    const bf16* __restrict__ a, const bf16* __restrict__ w_packed, void* __restrict__ out,
    int m, int n, int k, int n_tiles, int k_steps, MllSkinnyExtras extras) {
    extern __shared__ float reduce_shared[];
    const MllQkvStore& store = extras.store;   // [waves][NT * MT][64 lanes][4]
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

    // What the epilogue reads beside the product is asked for here, before the streaming begins, so that these
    // loads are not waited for at the end. The sums of squares for the rows' factors (SCALED) go straight from
    // memory into LDS, behind the waves' slots: [m][stride] as it lies in memory, 1 KB per wave-wide load.
    float* factor_shared = reduce_shared + static_cast<size_t>(waves - 1) * NT * MT * kWave * 4;
    if (SCALED && wave == 0) {
        const int count = m * extras.scale.stride;                  // floats; stride is a multiple of 4
        for (int first = 0; first < count; first += 256) {
            const int index = first + lane * 4;
            if (index < count)
                __builtin_amdgcn_global_load_lds(extras.scale.sumsq + index, factor_shared + first, 16, 0, 0);
        }
    }
    float bias_first[NT][2], bias_second[NT][2];
    float2 cos_sin[NT][2];
    int slot = -1;
    if (EPILOGUE == 3 && wave == 0 && col < m) {
        if (extras.store.slot_mapping) slot = extras.store.slot_mapping[col];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int column = (tile0 + nt) * 16 + quad * 4;
            const int head = column / extras.store.head_dim, within = column % extras.store.head_dim;
            const bool is_value = head >= extras.store.heads + extras.store.kv_heads;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const bool rotate = !is_value && within + 2 * half < 2 * extras.store.n_freq;
                const int pair = (within + 2 * half) / 2;
                const int first = rotate ? pair : within + 2 * half;
                const int second = rotate ? pair + extras.store.n_freq : within + 2 * half + 1;
                const bool live = column < n;
                bias_first[nt][half] = (live && extras.store.bias) ? extras.store.bias[head * extras.store.head_dim + first] : 0.0f;
                bias_second[nt][half] = (live && extras.store.bias) ? extras.store.bias[head * extras.store.head_dim + second] : 0.0f;
                cos_sin[nt][half] = make_float2(1.0f, 0.0f);
                if (live && rotate)
                    cos_sin[nt][half] = reinterpret_cast<const float2*>(extras.store.cos_sin)[static_cast<int64_t>(col) * extras.store.n_freq + pair];
            }
        }
    }
    float h_before[NT][4], norm_weight[NT][4];
    if (EPILOGUE == 4 && wave == 0) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int column = (tile0 + nt) * 16 + quad * 4 + i;
                const bool live = col < m && column < n;
                h_before[nt][i] = live ? extras.residual.h[static_cast<int64_t>(col) * n + column] : 0.0f;
                norm_weight[nt][i] = live ? extras.residual.norm_weight[column] : 0.0f;
            }
    }

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
    // PAIRED (one tile of rows, more than two rows): the activations are read two k steps at a time: lanes 0..7 of every 16 read rows
    // 0..7 (then 8..15) at one step and lanes 8..15 the same rows at the next, so that a load touches whole 128-byte
    // lines of 8 rows instead of half lines of 16; lanes 8 apart then exchange what the other needs.
    const bool upper = col >= 8;
    const bool low_live = (col & 7) < m, high_live = (col & 7) + 8 < m;
    const bf16* a_low = a + static_cast<int64_t>(low_live ? (col & 7) : 0) * k + quad * 8;
    const bf16* a_high = a + static_cast<int64_t>(high_live ? (col & 7) + 8 : 0) * k + quad * 8;

    // A wave takes kChunk consecutive k steps at a time, then skips what the other waves take (the last wave
    // begins, so that wave 0, which also writes the result, never has more chunks than another); which k steps a
    // wave sums, and in which order, depends on (n, k) alone, not on the number of rows or tiles. The loads of
    // DEPTH steps are issued before their products, so that a wave keeps several KB of W in flight.
    constexpr int DEPTH = (MT + NT <= 2) ? 8 : ((MT + NT <= 4) ? 4 : 2);
    for (int chunk = (waves - 1 - wave) * kChunk; chunk < k_steps; chunk += waves * kChunk) {
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
                        w_piece[u][nt].raw = __builtin_nontemporal_load(
                            reinterpret_cast<const uintx4*>(w_ptr[nt] + static_cast<int64_t>(ks) * 512));
                }
                if constexpr (PAIRED) {
                    // a_piece[u] of an even u: rows 0..7 (both steps of the pair); of the odd u after it: rows 8..15
                    const int own = (ks & ~1) + (upper ? 1 : 0);
                    const int k_offset = own * 32;
                    const bool in_k = own < k_steps && k_offset + quad * 8 < k;
                    const bool rows_live = (u & 1) ? high_live : low_live;
                    a_piece[u][0].raw = uintx4{0u, 0u, 0u, 0u};
                    if (rows_live && in_k)
                        a_piece[u][0].raw = *reinterpret_cast<const uintx4*>(((u & 1) ? a_high : a_low) + k_offset);
                } else {
                    const int k_offset = ks * 32;
                    const bool in_k = live && k_offset + quad * 8 < k;
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
                        a_piece[u][mt].raw = uintx4{0u, 0u, 0u, 0u};
                        if (a_live[mt] && in_k) a_piece[u][mt].raw = *reinterpret_cast<const uintx4*>(a_ptr[mt] + k_offset);
                    }
                }
            }
            if constexpr (PAIRED) {
                // low = rows 0..7 at the pair's first step (lanes 0..7) and its second (lanes 8..15), high = rows
                // 8..15 likewise. The first step's operand: own low | the partner's high; the second's: the partner's
                // low | own high.
#pragma unroll
                for (int u = 0; u < DEPTH; u += 2) {
                    const uintx4 low = a_piece[u][0].raw, high = a_piece[u + 1][0].raw;
                    uintx4 low_swapped, high_swapped;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        low_swapped[i] = static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(low[i]), 0x128, 0xf, 0xf, false));
                        high_swapped[i] = static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(high[i]), 0x128, 0xf, 0xf, false));
                    }
                    a_piece[u][0].raw = upper ? high_swapped : low;
                    a_piece[u + 1][0].raw = upper ? high : low_swapped;
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

    // The factor of row `col`: the four lanes of a row take every fourth run of four sums; the order of the
    // additions is fixed by the number of sums.
    float row_factor = 1.0f;
    if (SCALED) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // the loads into LDS have landed (the wave issued them itself)
        floatx4 parts = floatx4{0.0f, 0.0f, 0.0f, 0.0f};      // four sums side by side, then the four together
        if (col < m) {
            const float* sums = factor_shared + col * extras.scale.stride;
#pragma unroll 4
            for (int run = quad; 4 * run < extras.scale.groups; run += 4) {
                floatx4 four = *reinterpret_cast<const floatx4*>(sums + 4 * run);
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (4 * run + i >= extras.scale.groups) four[i] = 0.0f;
                parts += four;
            }
        }
        float part = (parts[0] + parts[1]) + (parts[2] + parts[3]);
        part = sum_lanes_16_apart(part);
        row_factor = 1.0f / sqrtf(part / static_cast<float>(extras.scale.width) + extras.scale.eps);
    }

    // acc[nt][mt][i] = C[row mt*16 + col][column (tile0 + nt)*16 + quad*4 + i]
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int n_tile = tile0 + nt;
        if (n_tile >= n_tiles) continue;       // the same for every lane of the wave
        float squares = 0.0f;                  // epilogue 4: this lane's share of its row's sum of squares over the tile
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int row = mt * 16 + col;
            if (row >= m) continue;
            if (SCALED) acc[nt][mt] *= row_factor;
            if (EPILOGUE == 4) {
                const MllResidualNorm& residual = extras.residual;
                const int column = n_tile * 16 + quad * 4;
                float* h_row = residual.h + static_cast<int64_t>(row) * n;
                bf16* x_row = static_cast<bf16*>(residual.x_out) + static_cast<int64_t>(row) * n;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (column + i >= n) continue;
                    const float value = h_before[nt][i] + acc[nt][mt][i];
                    h_row[column + i] = value;
                    x_row[column + i] = from_float<bf16>(value * norm_weight[nt][i]);
                    squares += value * value;
                }
            } else if (EPILOGUE == 0) {
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
                const CacheLayout layout(store.kv_heads, store.page_size, store.head_dim);
                bf16* q_row = static_cast<bf16*>(store.q_out) + (static_cast<int64_t>(row) * store.heads + head) * store.head_dim;
#pragma unroll
                for (int i = 0; i < 4; i += 2) {
                    const bool rotate = !is_value && within + i < 2 * store.n_freq;
                    const int pair = (within + i) / 2;
                    const int first = rotate ? pair : within + i;
                    const int second = rotate ? pair + store.n_freq : within + i + 1;
                    const float x1 = acc[nt][mt][i] + bias_first[nt][i / 2], x2 = acc[nt][mt][i + 1] + bias_second[nt][i / 2];
                    float y1 = x1, y2 = x2;
                    if (rotate) {
                        const float c = cos_sin[nt][i / 2].x, sn = cos_sin[nt][i / 2].y;
                        y1 = rotate_first(x1, x2, c, sn);
                        y2 = rotate_second(x1, x2, c, sn);
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
        if (EPILOGUE == 4) {
            // The row's sum over the tile's 16 columns: the four lanes of a row, in a fixed order. One entry per
            // tile of W, so that the sums do not depend on how many tiles a workgroup takes.
            squares = sum_lanes_16_apart(squares);
            if (quad == 0 && col < m) extras.residual.sumsq_out[static_cast<int64_t>(col) * extras.residual.sumsq_stride + n_tile] = squares;
        }
    }
}

template <int MT, int NT, int EPILOGUE>
static void launch_one(const bf16* a, const bf16* w, void* out, int m, int n, int k, int n_tiles,
                       int k_steps, const MllSkinnyExtras& extras, hipStream_t stream) {
    const int groups = (n_tiles + NT - 1) / NT;
    // Waves per workgroup: enough that about sixteen thousand waves would stream W one tile each (timed inside the
    // decode step of 7B sizes: 1 % faster than eight thousand at 8 and 16 rows, the same at one; thirty-two thousand
    // lose at one row), at most 16, and no more than there are chunks of k for them. A function of (n, k) alone,
    // like the split of k it implies.
    int waves = 1;
    while (waves < 16 && n_tiles * waves * 2 <= 16384 && waves * 2 * kChunk <= k_steps) waves *= 2;
    size_t lds = waves > 1 ? static_cast<size_t>(waves - 1) * NT * MT * kWave * sizeof(floatx4) : 0;
    const bool scaled = extras.scale.sumsq != nullptr;
    // PAIRED pays from three rows on (measured on MI355X: 18944 x 3584 at 8 rows 27 -> 25.6 us, at 16 rows 34 -> 30.7;
    // at one row 22.8 -> 24.4).
#define MLL_SKINNY_LAUNCH(SCALED_, PAIRED_)                                                                            \
    gemm_skinny_kernel<MT, NT, EPILOGUE, SCALED_, PAIRED_><<<groups, waves * kWave, lds, stream>>>(                    \
        a, w, out, m, n, k, n_tiles, k_steps, extras)
    if constexpr (MT == 1) {
        const bool paired = m > 2;
        if (scaled) {
            lds += (static_cast<size_t>(m) * extras.scale.stride * sizeof(float) + 1023) / 1024 * 1024;
            if (paired) MLL_SKINNY_LAUNCH(true, true); else MLL_SKINNY_LAUNCH(true, false);
        } else {
            if (paired) MLL_SKINNY_LAUNCH(false, true); else MLL_SKINNY_LAUNCH(false, false);
        }
    } else {
        MLL_SKINNY_LAUNCH(false, false);
    }
#undef MLL_SKINNY_LAUNCH
}

// Tiles of W a workgroup takes. Few tiles of W: one, so that the GPU is filled. Many tiles of W, or several rows of
// A and at least 128 workgroups left: two, so that every piece of A is used twice (all measured on MI355X; four
// tiles a workgroup were slower).
static int tiles_per_group(int m, int n_tiles) {
    if (m <= 16) return (n_tiles >= 2048 || (m > 4 && n_tiles >= 256)) ? 2 : 1;
    if (m <= 32) return n_tiles >= 2048 ? 2 : 1;
    return 2;
}

template <int EPILOGUE>
static int launch_skinny(const void* a, const void* w_packed, void* out, int m, int n, int k,
                         const MllSkinnyExtras& extras, hipStream_t stream) {
    const int n_tiles = (n + 15) / 16;
    const int k_steps = (k + 31) / 32;
    const bf16* a_ = static_cast<const bf16*>(a);
    const bf16* w_ = static_cast<const bf16*>(w_packed);
    const int m_tiles = (m + 15) / 16;
    const bool two = tiles_per_group(m, n_tiles) == 2;
    if constexpr (EPILOGUE >= 3) {
        if (m_tiles != 1) return fail("gemm_skinny: this epilogue takes at most 16 rows");
        if (two) launch_one<1, 2, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, extras, stream);
        else launch_one<1, 1, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, extras, stream);
        return check_launch("gemm_skinny");
    }
    switch (m_tiles) {
        case 1:
            if (two) launch_one<1, 2, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, extras, stream);
            else launch_one<1, 1, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, extras, stream);
            break;
        case 2:
            if (two) launch_one<2, 2, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, extras, stream);
            else launch_one<2, 1, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, extras, stream);
            break;
        case 3: launch_one<3, 2, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, extras, stream); break;
        case 4: launch_one<4, 2, EPILOGUE>(a_, w_, out, m, n, k, n_tiles, k_steps, extras, stream); break;
        default: return fail("gemm_skinny: more than 64 rows");
    }
    return check_launch("gemm_skinny");
}

}  // namespace mll

using namespace mll;

static int check_scale(const MllRowScale* scale, int m) {
    if (scale == nullptr || scale->sumsq == nullptr) return 0;
    MLL_REQUIRE(m <= 16, "gemm_skinny: a row factor needs at most 16 rows");
    MLL_REQUIRE(scale->groups > 0 && scale->width > 0 && scale->eps >= 0.0f, "gemm_skinny: bad row factor description");
    MLL_REQUIRE(scale->stride >= scale->groups && scale->stride % 4 == 0 && reinterpret_cast<uintptr_t>(scale->sumsq) % 16 == 0,
                "gemm_skinny: the rows of sums must be 16-byte aligned");
    MLL_REQUIRE(scale->stride <= 512, "gemm_skinny: a row factor from more than 512 sums (a norm wider than 8192)");
    return 0;
}

extern "C" int mll_gemm_skinny(const void* a, const void* w_packed, void* out, int epilogue, int m, int n, int k,
                               const MllRowScale* scale, hipStream_t stream) {
    MLL_REQUIRE(m >= 0 && m <= 64, "gemm_skinny: takes at most 64 rows");
    MLL_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_skinny: k must be a positive multiple of 8");
    MLL_REQUIRE(epilogue != 2 || n % 2 == 0, "gemm_skinny: the gated epilogue needs an even number of weight rows");
    if (check_scale(scale, m) != 0) return 1;
    if (m == 0) return 0;
    MllSkinnyExtras extras{};
    if (scale) extras.scale = *scale;
    switch (epilogue) {
        case 0: return launch_skinny<0>(a, w_packed, out, m, n, k, extras, stream);
        case 1: return launch_skinny<1>(a, w_packed, out, m, n, k, extras, stream);
        case 2: return launch_skinny<2>(a, w_packed, out, m, n, k, extras, stream);
        default: return fail("gemm_skinny: unknown epilogue");
    }
}

extern "C" int mll_gemm_skinny_qkv(const void* a, const void* w_packed, int m, int k, const MllQkvStore* store,
                                   const MllRowScale* scale, hipStream_t stream) {
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
    if (check_scale(scale, m) != 0) return 1;
    if (m == 0) return 0;
    const int n = (store->heads + 2 * store->kv_heads) * store->head_dim;
    MllSkinnyExtras extras{};
    extras.store = *store;
    if (scale) extras.scale = *scale;
    return launch_skinny<3>(a, w_packed, nullptr, m, n, k, extras, stream);
}

extern "C" int mll_gemm_skinny_residual(const void* a, const void* w_packed, int m, int n, int k,
                                        const MllResidualNorm* residual, const MllRowScale* scale, hipStream_t stream) {
    MLL_REQUIRE(residual != nullptr && residual->h && residual->norm_weight && residual->x_out && residual->sumsq_out,
                "gemm_skinny_residual: the residual stream, the norm's weight and both outputs are needed");
    MLL_REQUIRE(m >= 0 && m <= 16, "gemm_skinny_residual: takes at most 16 rows");
    MLL_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_skinny_residual: k must be a positive multiple of 8");
    MLL_REQUIRE(residual->sumsq_stride >= (n + 15) / 16, "gemm_skinny_residual: the rows of sums are too short");
    if (check_scale(scale, m) != 0) return 1;
    if (m == 0) return 0;
    MllSkinnyExtras extras{};
    extras.residual = *residual;
    if (scale) extras.scale = *scale;
    return launch_skinny<4>(a, w_packed, nullptr, m, n, k, extras, stream);
}
