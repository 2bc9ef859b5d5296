// C interface of libmicrollm_hip: every function launches on `stream`, returns 0 or a
// non-zero code, and leaves a text for mll_last_error() when it refuses its arguments.
// Pointers are device pointers unless a comment says otherwise. `dtype` is 0 for float32 and
// 1 for bfloat16 and names the element type of activations, cache pages and, where stated,
// weights. Statistics, softmax and accumulators are float32 in every kernel.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {

const char* mll_last_error();
int mll_version();

// out[t, :] = table[ids[t], :] widened to float32. An id outside [0, vocab) gives a row of NaN.
int mll_embedding(const void* table, int table_dtype, const int32_t* ids, float* out,
                  int n_tokens, int width, int vocab, hipStream_t stream);

// For i < n_rows, r = rows ? rows[i] : i:  v = h[r] + (delta ? delta[r] : 0);
// if write_h, h[r] = v;  out[i] = v * rsqrt(mean(v^2) + eps) * weight.
// h is the float32 residual stream; out has element type `dtype`, delta `delta_dtype`
// (float32, or the same as out). delta may come in n_partials parts, partial_stride elements apart, which
// are added in order (the partial sums of a matrix product that was split over k).
int mll_rms_norm(float* h, const void* delta, int delta_dtype, int n_partials, int64_t partial_stride,
                 const int32_t* rows, const float* weight, float eps,
                 void* out, int dtype, int n_rows, int width, int write_h, hipStream_t stream);

// Adds a pending delta into the residual stream: h[r] += delta[r] for all rows.
int mll_residual_add(float* h, const void* delta, int dtype, int n_rows, int width, hipStream_t stream);

// out[t][i] = (cos, sin) of positions[t] * inv_freq[i], the angle in float64: float32 [n_tokens][n_freq][2].
int mll_rope_table(const int32_t* positions, const double* inv_freq, int n_freq, int n_tokens, float* out,
                   hipStream_t stream);

// Splits fused projections qkv[t] = [q (H*hd) | k (KVH*hd) | v (KVH*hd)], adds `bias` (nullable),
// rotates q and k by the split-half rule with angle position * inv_freq[i] in float64, or with the cos and sin
// of mll_rope_table's `cos_sin` if that is given (both null: no rotation; rotary_dim = 2 * n_freq <= hd), writes q to q_out[t] and k, v into the pages (laid out as
// cache_layout.h says): slot = slot_mapping[t] (negative: not stored), page = slot / page_size,
// offset = slot % page_size. k_cache / v_cache nullable together with slot_mapping. qkv has element type
// `in_dtype` (float32, or the same as `dtype`) and may come in n_partials parts, partial_stride elements
// apart, which are added in order; q_out and the pages have `dtype`. With pair_order the query and key heads
// of qkv hold dims p and p + n_freq side by side (columns 2p, 2p + 1), as a weight in rotary pair order gives
// them (see MllQkvStore); bias and outputs are in the ordinary order.
int mll_qkv_rope_store(const void* qkv, int in_dtype, int n_partials, int64_t partial_stride, int dtype,
                       const float* bias, const int32_t* positions,
                       const int32_t* slot_mapping, const double* inv_freq, const void* cos_sin, int n_freq,
                       void* q_out, void* k_cache, void* v_cache,
                       int n_tokens, int heads, int kv_heads, int head_dim, int page_size, int pair_order,
                       hipStream_t stream);

// Attention of every query token over its request's pages, for any dtype and head size.
// Key j is visible to a query at position p iff j <= p and (window <= 0 or p - j < window).
// block_table[seq, j / page_size] gives the page of key j. Reduction order depends only on
// (p, window), so the result does not depend on how tokens were cut into steps, to the last bit.
// A token whose seq_of_token is negative is skipped and its output row left as it is (a row that pads a step to
// a fixed shape).
// max_chunks 0: one wave per (token, head). max_chunks > 0: one wave per (token, head, chunk of
// mll_paged_attention_rowwise_chunk() keys) and a second kernel that merges the chunks in the same order with
// the same arithmetic (the same bits), for steps with few rows; no row's visible keys may then span more than
// max_chunks chunks (chunks lie at absolute positions), and part_o [n_tokens * heads * max_chunks * head_dim]
// and part_ml [n_tokens * heads * max_chunks * 2] floats are the workspace.
// usual_chunks (0: max_chunks): how many chunks the rows have in this step, where max_chunks leaves room for later
// steps of the same shape; it only decides how many heads a wave takes.
int mll_paged_attention_rowwise_chunk();
// In float32 with head sizes up to 128 a wave takes several query heads of a kv head (their keys and values read
// once) where the step still has waves enough for the GPU that way. This forces the count (1 to 8; 0: the launch
// chooses again) and returns the value before. The same bits whatever the count.
int mll_rowwise_heads_a_wave(int count);
int mll_paged_attention_rowwise(const void* q, int dtype, const void* k_cache, const void* v_cache,
                                const int32_t* block_table, int table_width,
                                const int32_t* seq_of_token, const int32_t* positions, void* out,
                                float* part_o, float* part_ml, int max_chunks, int usual_chunks, float scale, int window,
                                int n_tokens, int heads, int kv_heads, int head_dim, int page_size,
                                hipStream_t stream);

// The same attention for bfloat16 portions of prompts with MFMA: one workgroup per (two tiles of up to
// mll_paged_attention_prefill_tile() consecutive tokens of one request, query head). `tiles` holds, for each
// workgroup, (request index; first token in the flat list and number of tokens of the first tile; the same of the
// second, whose number may be 0); a tile never spans two requests and its tokens have consecutive positions.
// Workgroups take as long as the keys of both tiles together: pair a tile late in a prompt with an early one.
// An entry whose tiles are both empty is skipped (padding of the list to a fixed length).
int mll_paged_attention_prefill(const void* q, const void* k_cache, const void* v_cache,
                                const int32_t* block_table, int table_width, const int32_t* tiles,
                                int n_tiles, const int32_t* positions, void* out, float scale, int window,
                                int heads, int kv_heads, int head_dim, int page_size, hipStream_t stream);
int mll_paged_attention_prefill_tile();

// out[t, c] = silu(gate[t, c]) * up[t, c]; gate and up rows are `in_stride` elements apart.
int mll_silu_mul(const void* gate, const void* up, int64_t in_stride, void* out, int dtype,
                 int n_tokens, int width, hipStream_t stream);

// C[m, n] = sum_k A[m, k] * W[n, k] (+ bias[n]), all float32, k summed in ascending order by one
// thread per output element, so a row's result does not depend on the other rows. With splits > 1
// (only the number mll_gemm_f32_splits gives for the weight's shape) C is [splits, m, n]: sums over
// consecutive ranges of k, the bias in the first, for the reader to add in order.
int mll_gemm_f32_splits(int n, int k);
// Which kernel takes a product of at most 16 rows: 0 gives the choice back to the launch; 1 (an element a thread), 2
// (two rows and two columns) and 4 (one row and four columns; at most 8 rows) force one, for measurements and tests. Returns the value before. The same bits whichever.
int mll_gemm_f32_small_variant(int variant);
int mll_gemm_f32(const float* a, const float* w, const float* bias, float* c,
                 int m, int n, int k, int splits, hipStream_t stream);

// C = A . W^T for bfloat16 A [m <= 64, k] and a weight packed as [n/16][k/32][4][16][8] (zero padded):
// element (row, col) of W sits at piece (row / 16, col / 32), position ((col % 32) / 8, row % 16, col % 8).
// epilogue 0: float32 [m, n]; 1: bfloat16 [m, n]; 2: bfloat16 [m, n / 2] = silu(even weight rows' results) *
// (odd rows' results). The order of additions is fixed by (n, k): the same in every run and whatever the
// other rows of A.
// With `scale` (may be null; at most 16 rows) row r of the product is first multiplied by
// 1 / sqrt(sum_{g < groups} sumsq[r][g] / width + eps): the factor of an RMS norm whose input came without it.
struct MllRowScale {
    const float* sumsq;   // [m][stride], 16-byte aligned; the first `groups` of a row count
    int groups;
    int stride;           // a multiple of 4
    int width;
    float eps;
};
int mll_gemm_skinny(const void* a, const void* w_packed, void* out, int epilogue, int m, int n, int k,
                    const MllRowScale* scale, hipStream_t stream);

// What the q/k/v projection's product does with its result instead of writing it out: the work of
// mll_qkv_rope_store. The packed weight's rows must be in rotary pair order: in every query and key head, row
// 2p holds dim p and row 2p + 1 dim p + n_freq for p < n_freq, the other dims follow in place; value heads are
// as they are. bias (float32, may be null) and the outputs are in the ordinary order.
struct MllQkvStore {
    const float* bias;
    const int32_t* slot_mapping;   // [m] page * page_size + offset, or null: keys and values are not kept
    const float* cos_sin;          // [m][n_freq][2]: mll_rope_table's
    int n_freq;
    void* q_out;                   // bfloat16 [m, heads * head_dim]
    void* k_cache;                 // bfloat16 pages
    void* v_cache;
    int heads, kv_heads, head_dim, page_size;
};
// Queries, keys and values of at most 16 rows: A [m, k] . W^T with n = (heads + 2 kv_heads) * head_dim, finished
// as `store` says.
int mll_gemm_skinny_qkv(const void* a, const void* w_packed, int m, int k, const MllQkvStore* store,
                        const MllRowScale* scale, hipStream_t stream);

// The product of at most 16 rows added to the residual stream, and the next RMS norm begun: h += A . W^T;
// x_out = h * norm_weight (the norm's input without the rows' factors); sumsq_out[r][g] = the sum of h[r]^2 over
// columns 16 g .. 16 g + 15, g < ceil(n / 16): what MllRowScale takes.
struct MllResidualNorm {
    float* h;                  // [m][n]
    const float* norm_weight;  // [n]
    void* x_out;               // bfloat16 [m][n]
    float* sumsq_out;          // [m][sumsq_stride]; the first ceil(n / 16) of a row are written
    int sumsq_stride;
};
int mll_gemm_skinny_residual(const void* a, const void* w_packed, int m, int n, int k, const MllResidualNorm* residual,
                             const MllRowScale* scale, hipStream_t stream);

// What the kernel takes beside the product's operands (internal to the library's launches).
struct MllSkinnyExtras {
    MllQkvStore store;
    MllRowScale scale;
    MllResidualNorm residual;
};

// The same product for up to 64 rows with the activations shared through LDS by the waves of a workgroup
// (faster than mll_gemm_skinny from 17 rows on). A wave takes tiles_per_wave (1 or 2) tiles of W. With
// splits > 1 (epilogue 0 only) k is cut into that many ranges and out is [splits][m][n]: partial sums that the
// caller adds in order. The order of additions is fixed by (n, k, splits).
int mll_gemm_medium(const void* a, const void* w_packed, void* out, int epilogue, int m, int n, int k,
                    int tiles_per_wave, int waves, int splits, hipStream_t stream);

// The same product for many rows: 256 x 256 tiles of C per workgroup, pieces of A and W brought into LDS by
// direct global-to-LDS loads. A is row-major [m, k] with k a multiple of 32; epilogues 0, 1 and 2 of
// mll_gemm_skinny. With epilogue 0, `splits` > 1 deals the stages of 64 of k to that many workgroups per tile:
// out is then [splits, m, n] partial sums for the caller to add in order. For weights that are kept in the packed
// order alone.
// tile_rows: the rows of a workgroup's tile of the result, 256, 192, 160 or 128, or 0 for mll_tiled_tile_rows's
// choice; the result's bits do not depend on it.
int mll_gemm_tiled(const void* a, const void* w_packed, void* out, int epilogue, int m, int n, int k,
                   int splits, int tile_rows, hipStream_t stream);
int mll_tiled_tile_rows(int m, int n, int splits);
// Queries, keys and values of many rows: the tiled product finished as mll_gemm_skinny_qkv finishes its own (the
// same MllQkvStore, the weight in rotary pair order). k a multiple of 32, store->n_freq even, no rows' factors; a
// workgroup owns a whole tile of the result and the reduction is never taken in parts.
int mll_gemm_tiled_qkv(const void* a, const void* w_packed, int m, int k, const MllQkvStore* store, int tile_rows,
                       hipStream_t stream);

// Calibration: a kernel that reads `bytes` of memory once with `blocks` workgroups, and one in which every wave of
// `blocks` workgroups of 4 issues iterations * 16 independent v_mfma_f32_16x16x32_bf16 (16384 flops each). The caller
// times them. `sink` is 4 bytes of device memory that are never written with ordinary data.
int mll_measure_read(const void* data, int64_t bytes, void* sink, int blocks, hipStream_t stream);
int mll_measure_mfma(int iterations, void* sink, int blocks, hipStream_t stream);

// Index of the first maximum of each row; a row that holds a non-finite value gives -1.
// `parts` is device scratch of n_rows * mll_argmax_slices(vocab) * 16 bytes (contents need not be cleared).
int mll_argmax(const float* logits, int32_t* out, void* parts, int n_rows, int vocab, hipStream_t stream);
int mll_argmax_slices(int vocab);

// mll_argmax for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc). It has no counterpart in the reference. The slices' scratch is a static
// array in device memory of MLL_ARGMAX_STATIC_MAX_PARTS * 16 bytes (1 MiB), one per GPU, held until the process
// ends; the call allocates and frees nothing. It refuses n_rows * mll_argmax_slices(vocab) beyond
// MLL_ARGMAX_STATIC_MAX_PARTS (at 64 slices, vocabularies from 129 025 tokens on: 1024 rows). The GPU whose
// scratch is used is the current one, which must be the stream's; the first call on a GPU looks the array's
// address up (make that call outside a graph capture). All calls on one GPU share the array: calls that overlap
// on one GPU (two streams, two threads) race; calls on one stream do not. The array keeps the last call's
// contents and needs no clearing: each call writes every entry it reads.
#define MLL_ARGMAX_STATIC_MAX_PARTS 65536
int mll_argmax_static(const float* logits, int32_t* out, int n_rows, int vocab, hipStream_t stream);

// Draws one token per row from softmax(logits / temperature) restricted to the top_k largest
// logits (top_k <= 0: all; ties at the k-th value go to the lower token ids), by inverse CDF in
// token order with the given uniform in [0, 1). temperature == 0 or top_k == 1 gives the
// argmax. A non-finite logit gives -1. top_k may be null (no row is restricted: the search for the
// k-th value is left out). `workspace`: mll_sample_workspace(n_rows, vocab) bytes of device scratch,
// 4-byte aligned; its contents need not be cleared.
int mll_sample(const float* logits, const float* temperature, const int32_t* top_k,
               const float* uniform, int32_t* out, void* workspace, int n_rows, int vocab,
               hipStream_t stream);
int64_t mll_sample_workspace(int n_rows, int vocab);

}  // extern "C"
