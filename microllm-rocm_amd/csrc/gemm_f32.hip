// The float32 matrix product of the true 32-bit path: C = A * W^T (+ bias), tiles staged through LDS.
// Every output element is summed by one thread in ascending k, so a row's result is the same whatever
// other rows the call holds and whichever of the kernels here computes it.
#include "common.h"
#include "microllm_hip.h"

namespace mll {

// The reduction may be cut into parts of k_split terms, one a blockIdx.z: part z sums k in [z * k_split, (z + 1) *
// k_split) in ascending order into C[z] (its own [m, n] array), the bias goes to part 0, and whoever reads the result
// adds the parts in order. The cut depends on the weight's shape alone (mll_gemm_f32_splits), never on the rows of the
// call, so a row's bits stay what they are under every batch. Inside a kernel `k` then is the part's end, and sums
// start at k_lo.
#define MLL_F32_SPLIT_RANGE                                                          \
    const int ld = k; /* elements from one row of A or W to the next */              \
    const int k_lo = blockIdx.z * k_split;                                           \
    k = min(k, k_lo + k_split);                                                      \
    c += static_cast<int64_t>(blockIdx.z) * m * n;                                   \
    if (blockIdx.z != 0) bias = nullptr;

// Tiles for more than 16 rows. A workgroup of THREADS threads takes (THREADS / 16) * TR rows and 16 * TC columns of
// C; a thread TR x TC elements (rows r + (THREADS / 16) * i, columns c + 16 * j), each summed by that thread alone in
// ascending k with one fused multiply-add a term: the bits of the kernels for few rows below. Both operands come in
// chunks of DEPTH of k with 16-byte loads of whole rows (the next chunk is on its way while this one is summed) and lie
// in LDS as [row][k] with rows four banks apart, so that a thread's four consecutive k are one read and the rows a
// wave reads at one k fall on different banks. Two shapes are used: 64 x 64 with 4 x 4 elements a thread (one read
// from LDS for eight multiply-adds) wherever that gives the GPU enough workgroups (prompts; weights of many rows), and
// 16 x 32 with 2 x 2 (one for four) where C is small: 64 rows of a weight of 3584 are 224 tiles of 64 x 64 but 896
// of 16 x 32.
template <int THREADS, int TR, int TC, int DEPTH, bool VECTOR>
__global__ __launch_bounds__(THREADS) void gemm_f32_tile_kernel(const float* __restrict__ a, const float* __restrict__ w,
                                                                const float* __restrict__ bias, float* __restrict__ c,
                                                                int m, int n, int k, int k_split) {
    MLL_F32_SPLIT_RANGE
    constexpr int ROW_STEP = THREADS / 16;
    constexpr int ROWS = ROW_STEP * TR;
    constexpr int COLUMNS = 16 * TC;
    constexpr int QUADS = DEPTH / 4;                       // float4 in a row of a chunk
    constexpr int LOADS_A = ROWS * QUADS / THREADS;
    constexpr int LOADS_W = COLUMNS * QUADS / THREADS;
    static_assert(ROWS * QUADS % THREADS == 0 && COLUMNS * QUADS % THREADS == 0, "a chunk is dealt evenly to the threads");
    __shared__ __align__(16) float a_tile[ROWS][DEPTH + 4];
    __shared__ __align__(16) float w_tile[COLUMNS][DEPTH + 4];
    const int row0 = blockIdx.y * ROWS;
    const int col0 = blockIdx.x * COLUMNS;
    const int column = threadIdx.x % 16;
    const int row = threadIdx.x / 16;
    auto load4 = [&](const float* matrix, int rows, int first_row, int index, int k0) {
        const int r = index / QUADS, kk = k0 + (index % QUADS) * 4;
        const bool live = first_row + r < rows;
        const float* source = matrix + static_cast<int64_t>(live ? first_row + r : 0) * ld + kk;
        if (VECTOR) return (live && kk < k) ? *reinterpret_cast<const float4*>(source) : make_float4(0.f, 0.f, 0.f, 0.f);
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (live && kk + e < k) ? source[e] : 0.0f;
        return make_float4(v[0], v[1], v[2], v[3]);
    };
    float4 a_next[LOADS_A], w_next[LOADS_W];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int j = 0; j < LOADS_A; ++j) a_next[j] = load4(a, m, row0, threadIdx.x + j * THREADS, k0);
#pragma unroll
        for (int j = 0; j < LOADS_W; ++j) w_next[j] = load4(w, n, col0, threadIdx.x + j * THREADS, k0);
    };
    float acc[TR][TC];
#pragma unroll
    for (int i = 0; i < TR; ++i)
#pragma unroll
        for (int j = 0; j < TC; ++j) acc[i][j] = 0.0f;
    fetch(k_lo);
    for (int k0 = k_lo; k0 < k; k0 += DEPTH) {
#pragma unroll
        for (int j = 0; j < LOADS_A; ++j) {
            const int index = threadIdx.x + j * THREADS;
            *reinterpret_cast<float4*>(&a_tile[index / QUADS][(index % QUADS) * 4]) = a_next[j];
        }
#pragma unroll
        for (int j = 0; j < LOADS_W; ++j) {
            const int index = threadIdx.x + j * THREADS;
            *reinterpret_cast<float4*>(&w_tile[index / QUADS][(index % QUADS) * 4]) = w_next[j];
        }
        __syncthreads();
        if (k0 + DEPTH < k) fetch(k0 + DEPTH);
#pragma unroll
        for (int kk = 0; kk < DEPTH; kk += 4) {
            float4 av[TR], wv[TC];
#pragma unroll
            for (int i = 0; i < TR; ++i) av[i] = *reinterpret_cast<const float4*>(&a_tile[row + ROW_STEP * i][kk]);
#pragma unroll
            for (int j = 0; j < TC; ++j) wv[j] = *reinterpret_cast<const float4*>(&w_tile[column + 16 * j][kk]);
#pragma unroll
            for (int i = 0; i < TR; ++i)
#pragma unroll
                for (int j = 0; j < TC; ++j) acc[i][j] = fmaf(av[i].x, wv[j].x, acc[i][j]);
#pragma unroll
            for (int i = 0; i < TR; ++i)
#pragma unroll
                for (int j = 0; j < TC; ++j) acc[i][j] = fmaf(av[i].y, wv[j].y, acc[i][j]);
#pragma unroll
            for (int i = 0; i < TR; ++i)
#pragma unroll
                for (int j = 0; j < TC; ++j) acc[i][j] = fmaf(av[i].z, wv[j].z, acc[i][j]);
#pragma unroll
            for (int i = 0; i < TR; ++i)
#pragma unroll
                for (int j = 0; j < TC; ++j) acc[i][j] = fmaf(av[i].w, wv[j].w, acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < TR; ++i)
#pragma unroll
        for (int j = 0; j < TC; ++j) {
            const int r = row0 + row + ROW_STEP * i, col = col0 + column + 16 * j;
            if (r < m && col < n) c[static_cast<int64_t>(r) * n + col] = acc[i][j] + (bias ? bias[col] : 0.0f);
        }
}

// The same product for at most 16 rows (decoding): a workgroup takes 16 columns of C, so that a weight of a few
// thousand rows fills the GPU where tiles of 64 would leave most of it idle, and one thread one output element.
// Each thread sums in ascending k with the same fused multiply-adds as the tiled kernel: the two give the same
// bits, so a token's result does not depend on how many rows the step had.
constexpr int kSmallColumns = 16;
constexpr int kSmallDepth = 256;      // of k in a chunk (128: 3 to 7 % slower)
constexpr int kSmallParts = kSmallDepth / 64;

// VECTOR: k is a multiple of 4 and both matrices are 16-byte aligned, so a thread's four consecutive elements are
// one load.
template <bool VECTOR>
__global__ __launch_bounds__(256) void gemm_f32_small_kernel(const float* __restrict__ a, const float* __restrict__ w,
                                                             const float* __restrict__ bias, float* __restrict__ c,
                                                             int m, int n, int k, int k_split) {
    MLL_F32_SPLIT_RANGE
    // Rows of kSmallDepth + 4 floats: 16-byte aligned, so that four consecutive k are one read, and four banks on
    // from row to row, so that the 16 rows (or columns) that a wave reads at one k fall on different banks.
    __shared__ __align__(16) float a_tile[16][kSmallDepth + 4];
    __shared__ __align__(16) float w_tile[kSmallColumns][kSmallDepth + 4];
    const int col0 = blockIdx.x * kSmallColumns;
    const int column = threadIdx.x % kSmallColumns;     // this thread's output: row `row`, column col0 + `column`
    const int row = threadIdx.x / kSmallColumns;
    // What a thread brings in of a chunk of kSmallDepth of k: of row load_row of A and of W, elements
    // load_k .. load_k + 3 of every 64.
    const int load_row = threadIdx.x / 16;
    const int load_k = (threadIdx.x % 16) * 4;
    const bool a_live = load_row < m, w_live = col0 + load_row < n;
    const float* a_row = a + static_cast<int64_t>(a_live ? load_row : 0) * ld;
    const float* w_row = w + static_cast<int64_t>(w_live ? col0 + load_row : 0) * ld;
    float4 a_next[kSmallParts], w_next[kSmallParts];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int part = 0; part < kSmallParts; ++part) {
            const int kk = k0 + 64 * part + load_k;
            if (VECTOR) {
                a_next[part] = (a_live && kk < k) ? *reinterpret_cast<const float4*>(a_row + kk) : make_float4(0.f, 0.f, 0.f, 0.f);
                w_next[part] = (w_live && kk < k) ? *reinterpret_cast<const float4*>(w_row + kk) : make_float4(0.f, 0.f, 0.f, 0.f);
            } else {
                float av[4], wv[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    av[e] = (a_live && kk + e < k) ? a_row[kk + e] : 0.0f;
                    wv[e] = (w_live && kk + e < k) ? w_row[kk + e] : 0.0f;
                }
                a_next[part] = make_float4(av[0], av[1], av[2], av[3]);
                w_next[part] = make_float4(wv[0], wv[1], wv[2], wv[3]);
            }
        }
    };
    float acc = 0.0f;
    fetch(k_lo);
    for (int k0 = k_lo; k0 < k; k0 += kSmallDepth) {
#pragma unroll
        for (int part = 0; part < kSmallParts; ++part) {
            const int at = 64 * part + load_k;
            *reinterpret_cast<float4*>(&a_tile[load_row][at]) = a_next[part];
            *reinterpret_cast<float4*>(&w_tile[load_row][at]) = w_next[part];
        }
        __syncthreads();
        if (k0 + kSmallDepth < k) fetch(k0 + kSmallDepth);      // the next chunk is on its way while this one is summed
        // Four k a read, summed one after the other in ascending k as before: the same bits.
#pragma unroll
        for (int kk = 0; kk < kSmallDepth; kk += 4) {
            const float4 av = *reinterpret_cast<const float4*>(&a_tile[row][kk]);
            const float4 wv = *reinterpret_cast<const float4*>(&w_tile[column][kk]);
            acc = fmaf(av.x, wv.x, acc);
            acc = fmaf(av.y, wv.y, acc);
            acc = fmaf(av.z, wv.z, acc);
            acc = fmaf(av.w, wv.w, acc);
        }
        __syncthreads();
    }
    const int col = col0 + column;
    if (row < m && col < n) c[static_cast<int64_t>(row) * n + col] = acc + (bias ? bias[col] : 0.0f);
}

// The same for weights with many rows (gate/up, the head), where the kernel above is bound by its reads from LDS (two a
// multiply-add): a workgroup of 128 threads takes 32 columns of C and a thread 2 rows x 2 columns (rows r and r + 8,
// columns c and c + 16): half the reads a multiply-add, and four chains of additions a thread. Every element is still
// summed by one thread in ascending k: the same bits. Measured on MI355X at 7B sizes, 8 rows: gate/up 179 -> 140 us
// (3.9 TB/s), the head 602 -> 450 (4.8 TB/s); with few columns it has too few waves (q/k/v 37 -> 65 us, down 136 -> 330).
// Where W has few rows the kernel above stays at 1.8 to 2.0 TB/s: a wave an element's worth of lanes is all the
// parallelism there is, and its reads from LDS (512 KB for 16 KB of W) are what a compute unit can give; neither four
// sums an element instead of one, nor two chunks in flight instead of one, nor reading LDS a batch ahead changes that.
constexpr int kWideThreads = 128;
constexpr int kWideDepth = 128;                      // of k in a chunk
constexpr int kWideQuads = kWideDepth / 4;           // float4 in a row of a chunk
constexpr int kWideFrom = 16384;                     // columns of C from which this kernel is taken whatever the parts

// TR x TC elements a thread: rows r (+ 8), columns c, c + 16, ... of the workgroup's 8 TR rows and 16 TC columns. Per
// four k a thread reads TR + TC times from LDS for 4 TR TC multiply-adds, and every element of W is read by 8 threads:
// with 2 x 2 that is 16 reads an element of W, which is what bounds the kernel (4.1 TB/s of W for gate/up at 8 rows,
// where half of the 16 rows are empty); 1 x 4 for at most 8 rows makes it 10 (4.8 TB/s; the head 4.95 -> 5.4).
template <bool VECTOR, int TR, int TC>
__global__ __launch_bounds__(kWideThreads) void gemm_f32_small_wide_kernel(const float* __restrict__ a, const float* __restrict__ w,
                                                                           const float* __restrict__ bias, float* __restrict__ c,
                                                                           int m, int n, int k, int k_split) {
    MLL_F32_SPLIT_RANGE
    constexpr int ROWS = 8 * TR, COLUMNS = 16 * TC;
    constexpr int LOADS_A = ROWS * kWideQuads / kWideThreads, LOADS_W = COLUMNS * kWideQuads / kWideThreads;
    __shared__ __align__(16) float a_tile[ROWS][kWideDepth + 4];
    __shared__ __align__(16) float w_tile[COLUMNS][kWideDepth + 4];
    const int col0 = blockIdx.x * COLUMNS;
    const int column = threadIdx.x % 16;      // this thread's outputs: rows `row` (+ 8); columns col0 + `column` + 16 j
    const int row = threadIdx.x / 16;
    // What a thread brings in of a chunk: float4 number threadIdx.x + j * 128 of the chunk's rows of A (ROWS rows of
    // kWideQuads) and of W (COLUMNS rows).
    auto load4 = [&](const float* matrix, int rows, int first_row, int index, int k0) {
        const int r = index / kWideQuads, kk = k0 + (index % kWideQuads) * 4;
        const bool live = first_row + r < rows;
        const float* source = matrix + static_cast<int64_t>(live ? first_row + r : 0) * ld + kk;
        if (VECTOR) return (live && kk < k) ? *reinterpret_cast<const float4*>(source) : make_float4(0.f, 0.f, 0.f, 0.f);
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (live && kk + e < k) ? source[e] : 0.0f;
        return make_float4(v[0], v[1], v[2], v[3]);
    };
    float4 a_next[LOADS_A], w_next[LOADS_W];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int j = 0; j < LOADS_A; ++j) a_next[j] = load4(a, m, 0, threadIdx.x + j * kWideThreads, k0);
#pragma unroll
        for (int j = 0; j < LOADS_W; ++j) w_next[j] = load4(w, n, col0, threadIdx.x + j * kWideThreads, k0);
    };
    float acc[TR][TC];
#pragma unroll
    for (int i = 0; i < TR; ++i)
#pragma unroll
        for (int j = 0; j < TC; ++j) acc[i][j] = 0.0f;
    fetch(k_lo);
    for (int k0 = k_lo; k0 < k; k0 += kWideDepth) {
#pragma unroll
        for (int j = 0; j < LOADS_A; ++j) {
            const int index = threadIdx.x + j * kWideThreads;
            *reinterpret_cast<float4*>(&a_tile[index / kWideQuads][(index % kWideQuads) * 4]) = a_next[j];
        }
#pragma unroll
        for (int j = 0; j < LOADS_W; ++j) {
            const int index = threadIdx.x + j * kWideThreads;
            *reinterpret_cast<float4*>(&w_tile[index / kWideQuads][(index % kWideQuads) * 4]) = w_next[j];
        }
        __syncthreads();
        if (k0 + kWideDepth < k) fetch(k0 + kWideDepth);      // the next chunk is on its way while this one is summed
        // Four k a read, added one after the other in ascending k.
#pragma unroll
        for (int kk = 0; kk < kWideDepth; kk += 4) {
            float4 av[TR], wv[TC];
#pragma unroll
            for (int i = 0; i < TR; ++i) av[i] = *reinterpret_cast<const float4*>(&a_tile[row + 8 * i][kk]);
#pragma unroll
            for (int j = 0; j < TC; ++j) wv[j] = *reinterpret_cast<const float4*>(&w_tile[column + 16 * j][kk]);
#pragma unroll
            for (int i = 0; i < TR; ++i)
#pragma unroll
                for (int j = 0; j < TC; ++j) acc[i][j] = fmaf(av[i].x, wv[j].x, acc[i][j]);
#pragma unroll
            for (int i = 0; i < TR; ++i)
#pragma unroll
                for (int j = 0; j < TC; ++j) acc[i][j] = fmaf(av[i].y, wv[j].y, acc[i][j]);
#pragma unroll
            for (int i = 0; i < TR; ++i)
#pragma unroll
                for (int j = 0; j < TC; ++j) acc[i][j] = fmaf(av[i].z, wv[j].z, acc[i][j]);
#pragma unroll
            for (int i = 0; i < TR; ++i)
#pragma unroll
                for (int j = 0; j < TC; ++j) acc[i][j] = fmaf(av[i].w, wv[j].w, acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < TR; ++i)
#pragma unroll
        for (int j = 0; j < TC; ++j) {
            const int r = row + 8 * i, col = col0 + column + 16 * j;
            if (r < m && col < n) c[static_cast<int64_t>(r) * n + col] = acc[i][j] + (bias ? bias[col] : 0.0f);
        }
}

template <int TR, int TC>
static void launch_small_wide(const float* a, const float* w, const float* bias, float* c, int m, int n, int k, int k_split,
                              unsigned parts, bool vector, hipStream_t stream) {
    const dim3 grid((n + 16 * TC - 1) / (16 * TC), 1, parts);
    if (vector) gemm_f32_small_wide_kernel<true, TR, TC><<<grid, kWideThreads, 0, stream>>>(a, w, bias, c, m, n, k, k_split);
    else gemm_f32_small_wide_kernel<false, TR, TC><<<grid, kWideThreads, 0, stream>>>(a, w, bias, c, m, n, k, k_split);
}

}  // namespace mll

using namespace mll;

// Into how many parts the reduction over k is cut for a weight [n, k]: a function of the weight's shape alone. A
// weight with few rows of its own (q/k/v, o, down) gives the GPU too few tiles of C; its parts go to workgroups of
// their own. Parts are at least 448 terms long and at most 8.
// Which kernel takes a product of at most 16 rows: 0 the choice below; for measurements and tests 1 (an element a
// thread), 2 (2 x 2) or 4 (1 x 4, at most 8 rows). The same bits whichever.
static int f32_small_variant = 0;
extern "C" int mll_gemm_f32_small_variant(int variant) {
    const int before = f32_small_variant;
    f32_small_variant = (variant == 1 || variant == 2 || variant == 4) ? variant : 0;
    return before;
}

extern "C" int mll_gemm_f32_splits(int n, int k) {
    if (n >= kWideFrom) return 1;
    int splits = 1;
    while (splits < 8 && (n / kSmallColumns) * splits < 2048 && k / (2 * splits) >= 448) splits *= 2;
    return splits;
}

// C[splits][m][n]; splits is 1 or mll_gemm_f32_splits(n, k).
extern "C" int mll_gemm_f32(const float* a, const float* w, const float* bias, float* c,
                            int m, int n, int k, int splits, hipStream_t stream) {
    MLL_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm_f32: sizes must be positive");
    MLL_REQUIRE(splits == 1 || splits == mll_gemm_f32_splits(n, k), "gemm_f32: the reduction is cut as mll_gemm_f32_splits says, or not at all");
    if (m == 0) return 0;
    const int k_split = splits == 1 ? k : ((k + splits - 1) / splits + 3) / 4 * 4;
    MLL_REQUIRE(static_cast<int64_t>(k_split) * (splits - 1) < k, "gemm_f32: a part of the reduction would be empty");
    const unsigned parts = static_cast<unsigned>(splits);
    const bool vector = k % 4 == 0 && reinterpret_cast<uintptr_t>(a) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
    if (m <= 16) {
        // Up to 8 rows: one row and four columns a thread where that still gives the GPU its workgroups (weights of
        // many rows; the others with their parts); else two rows and two columns where that does, else the kernel of
        // one element a thread. (Two rows and four columns for 9 to 16 rows are slower than two and two: gate/up at
        // 7B sizes 131 -> 156 us. A column a thread with all rows, which reads an element of W from LDS once, is
        // faster for one row alone (q/k/v 20 -> 16.5 us, down 60 -> 51) and 1 % in the step; from two rows on the
        // rows of A, read by all lanes at one address, cost more than is saved: 8 rows 115 -> 310 us.)
        const int64_t quads = static_cast<int64_t>((n + 63) / 64) * splits, pairs = static_cast<int64_t>((n + 31) / 32) * splits;
        int variant = f32_small_variant;
        if (variant == 4 && m > 8) variant = 2;
        if (variant == 0) {
            if (m <= 8 && (n >= kWideFrom || quads >= 384)) variant = 4;
            else if (n >= kWideFrom || pairs >= 512) variant = 2;
            else variant = 1;
        }
        if (variant == 4) {
            launch_small_wide<1, 4>(a, w, bias, c, m, n, k, k_split, parts, vector, stream);
            return check_launch("gemm_f32");
        }
        if (variant == 2) {
            launch_small_wide<2, 2>(a, w, bias, c, m, n, k, k_split, parts, vector, stream);
            return check_launch("gemm_f32");
        }
        const dim3 grid((n + kSmallColumns - 1) / kSmallColumns, 1, parts);
        if (vector) gemm_f32_small_kernel<true><<<grid, 256, 0, stream>>>(a, w, bias, c, m, n, k, k_split);
        else gemm_f32_small_kernel<false><<<grid, 256, 0, stream>>>(a, w, bias, c, m, n, k, k_split);
        return check_launch("gemm_f32");
    }
    // Tiles of 64 x 64 wherever they are enough workgroups for the GPU; for at most 32 rows of a weight with many rows
    // tiles of 32 x 64 (the same 4 x 4 elements a thread: the head at 17 to 32 rows 940 -> 640 us); else tiles of 16 x 32.
    const int64_t column_tiles = (n + 63) / 64;
    if (m >= 512 && column_tiles * ((m + 127) / 128) * splits >= 512) {
        const dim3 grid(column_tiles, (m + 127) / 128, parts);
        MLL_REQUIRE(grid.y <= 65535, "gemm_f32: too many rows for one call");
        if (vector) gemm_f32_tile_kernel<256, 8, 4, 32, true><<<grid, 256, 0, stream>>>(a, w, bias, c, m, n, k, k_split);
        else gemm_f32_tile_kernel<256, 8, 4, 32, false><<<grid, 256, 0, stream>>>(a, w, bias, c, m, n, k, k_split);
    } else if (m > 32 && column_tiles * ((m + 63) / 64) * splits >= 384) {
        const dim3 grid(column_tiles, (m + 63) / 64, parts);
        MLL_REQUIRE(grid.y <= 65535, "gemm_f32: too many rows for one call");
        if (vector) gemm_f32_tile_kernel<256, 4, 4, 32, true><<<grid, 256, 0, stream>>>(a, w, bias, c, m, n, k, k_split);
        else gemm_f32_tile_kernel<256, 4, 4, 32, false><<<grid, 256, 0, stream>>>(a, w, bias, c, m, n, k, k_split);
    } else if (m <= 32 && n >= kWideFrom) {
        const dim3 grid(column_tiles, (m + 31) / 32, parts);
        if (vector) gemm_f32_tile_kernel<128, 4, 4, 32, true><<<grid, 128, 0, stream>>>(a, w, bias, c, m, n, k, k_split);
        else gemm_f32_tile_kernel<128, 4, 4, 32, false><<<grid, 128, 0, stream>>>(a, w, bias, c, m, n, k, k_split);
    } else {
        const dim3 grid((n + 31) / 32, (m + 15) / 16, parts);
        MLL_REQUIRE(grid.y <= 65535, "gemm_f32: too many rows for one call");
        if (vector) gemm_f32_tile_kernel<128, 2, 2, 128, true><<<grid, 128, 0, stream>>>(a, w, bias, c, m, n, k, k_split);
        else gemm_f32_tile_kernel<128, 2, 2, 128, false><<<grid, 128, 0, stream>>>(a, w, bias, c, m, n, k, k_split);
    }
    return check_launch("gemm_f32");
}
