// Row-wise kernels around the matrix products: embedding gather, RMSNorm with the residual
// sum, bias + rotation + page write of the attention projections, and SiLU-mul.
#include "cache_layout.h"
#include "common.h"
#include "microllm_hip.h"

namespace mll {

static thread_local std::string g_error;
void set_error(const std::string& text) { g_error = text; }
int fail(const std::string& text) {
    g_error = text;
    return 1;
}

// ---------------------------------------------------------------------------------------------
template <typename W>
__global__ void embedding_kernel(const W* __restrict__ table, const int32_t* __restrict__ ids,
                                 float* __restrict__ out, int width, int vocab) {
    const int token = blockIdx.x;
    const int id = ids[token];
    float* row_out = out + static_cast<int64_t>(token) * width;
    if (id < 0 || id >= vocab) {
        for (int column = threadIdx.x; column < width; column += blockDim.x) row_out[column] = NAN;
        return;
    }
    const W* row = table + static_cast<int64_t>(id) * width;
    for (int column = threadIdx.x; column < width; column += blockDim.x) row_out[column] = to_float(row[column]);
}

// ---------------------------------------------------------------------------------------------
// One block per output row. The sum of squares is taken in float32: per-thread strided partial
// sums, a butterfly inside each wave, then the waves in ascending order.
template <typename T, typename D>
__global__ void rms_norm_kernel(float* __restrict__ h, const D* __restrict__ delta,
                                int n_partials, int64_t partial_stride,
                                const int32_t* __restrict__ rows, const float* __restrict__ weight,
                                float eps, T* __restrict__ out, int width, int write_h) {
    __shared__ float scratch[16];
    const int index = blockIdx.x;
    const int64_t source = rows ? rows[index] : index;
    float* h_row = h + source * width;
    const D* delta_row = delta ? delta + source * width : nullptr;
    T* out_row = out + static_cast<int64_t>(index) * width;

    float partial = 0.0f;
    for (int column = threadIdx.x; column < width; column += blockDim.x) {
        float value = h_row[column];
        if (delta_row) {
            float sum = to_float(delta_row[column]);
            for (int part = 1; part < n_partials; ++part) sum += to_float(delta_row[part * partial_stride + column]);
            value += sum;
        }
        if (write_h) h_row[column] = value;
        partial += value * value;
    }
    const float total = block_sum(partial, scratch);
    const float inverse_rms = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
    for (int column = threadIdx.x; column < width; column += blockDim.x) {
        float value = h_row[column];  // already holds the sum when write_h
        if (delta_row && !write_h) {
            float sum = to_float(delta_row[column]);
            for (int part = 1; part < n_partials; ++part) sum += to_float(delta_row[part * partial_stride + column]);
            value += sum;
        }
        out_row[column] = from_float<T>(value * inverse_rms * weight[column]);
    }
}

__device__ inline float4 load_four(const float* source) { return *reinterpret_cast<const float4*>(source); }
__device__ inline float4 load_four(const bf16* source) {
    return make_float4(to_float(source[0]), to_float(source[1]), to_float(source[2]), to_float(source[3]));
}

// The same for rows of float4: one pass, the row kept in registers between the sum of squares and the
// scaling. Taken when the width is a multiple of 4 and at most 4 * CHUNKS * blockDim.x.
template <typename T, typename D, int CHUNKS>
__global__ void rms_norm_vec4_kernel(float* __restrict__ h, const D* __restrict__ delta,
                                     int n_partials, int64_t partial_stride,
                                     const int32_t* __restrict__ rows, const float* __restrict__ weight,
                                     float eps, T* __restrict__ out, int width, int write_h) {
    __shared__ float scratch[16];
    const int index = blockIdx.x;
    const int64_t source = rows ? rows[index] : index;
    float* h_row = h + source * width;
    const D* delta_row = delta ? delta + source * width : nullptr;
    T* out_row = out + static_cast<int64_t>(index) * width;
    const int quads = width / 4;

    float4 value[CHUNKS];
    float partial = 0.0f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int q = threadIdx.x + c * blockDim.x;
        value[c] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (q < quads) {
            value[c] = reinterpret_cast<const float4*>(h_row)[q];
            if (delta_row) {
                // The parts of the delta are added first, in order, and their sum to the stream. Up to sixteen parts
                // are asked for at a time and then added: a part an iteration waits for memory once a part (64 rows
                // of 3584 in 16 parts: 11.4 us that way, 8.5 with eight at a time).
                constexpr int kAtATime = CHUNKS == 1 ? 16 : 8;
                float4 sum = load_four(delta_row + 4 * q);
                for (int base = 1; base < n_partials; base += kAtATime) {
                    float4 more[kAtATime];
#pragma unroll
                    for (int j = 0; j < kAtATime; ++j)
                        if (base + j < n_partials) more[j] = load_four(delta_row + (base + j) * partial_stride + 4 * q);
#pragma unroll
                    for (int j = 0; j < kAtATime; ++j)
                        if (base + j < n_partials) {
                            sum.x += more[j].x;
                            sum.y += more[j].y;
                            sum.z += more[j].z;
                            sum.w += more[j].w;
                        }
                }
                value[c].x += sum.x;
                value[c].y += sum.y;
                value[c].z += sum.z;
                value[c].w += sum.w;
            }
            if (write_h) reinterpret_cast<float4*>(h_row)[q] = value[c];
            partial += value[c].x * value[c].x + value[c].y * value[c].y + value[c].z * value[c].z + value[c].w * value[c].w;
        }
    }
    const float total = block_sum(partial, scratch);
    const float inverse_rms = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int q = threadIdx.x + c * blockDim.x;
        if (q < quads) {
            const float4 w = reinterpret_cast<const float4*>(weight)[q];
            out_row[4 * q + 0] = from_float<T>(value[c].x * inverse_rms * w.x);
            out_row[4 * q + 1] = from_float<T>(value[c].y * inverse_rms * w.y);
            out_row[4 * q + 2] = from_float<T>(value[c].z * inverse_rms * w.z);
            out_row[4 * q + 3] = from_float<T>(value[c].w * inverse_rms * w.w);
        }
    }
}

template <typename T, typename D>
static void launch_rms_norm(float* h, const D* delta, int n_partials, int64_t partial_stride, const int32_t* rows,
                            const float* weight, float eps, T* out, int n_rows, int width, int write_h,
                            hipStream_t stream) {
    const bool delta_aligned = delta == nullptr || sizeof(D) != sizeof(float) ||
                               (reinterpret_cast<uintptr_t>(delta) % 16 == 0 && (n_partials == 1 || partial_stride % 4 == 0));
    const bool aligned = width % 4 == 0 && delta_aligned &&
                         reinterpret_cast<uintptr_t>(h) % 16 == 0 && reinterpret_cast<uintptr_t>(weight) % 16 == 0;
    const int quads = width / 4;
    if (aligned && quads <= 1024 && n_rows >= 512 && quads >= 256 && sizeof(T) == 2) {
        // Many rows (a prompt): four chunks a thread in blocks a quarter the size, so that a compute unit holds more
        // rows at once and a thread has more loads on their way (2048 rows of 3584: 26.5 -> 24.2 us). The squares
        // are then added in another order, so the choice may follow the number of rows only where a result is
        // rounded to bfloat16 anyway: in the float32 engine a row's bits must not depend on the step's other rows.
        const int threads = ((quads + 3) / 4 + 63) / 64 * 64;
        rms_norm_vec4_kernel<T, D, 4><<<n_rows, threads, 0, stream>>>(h, delta, n_partials, partial_stride, rows, weight, eps, out, width, write_h);
    } else if (aligned && quads <= 1024) {
        const int threads = max(64, (quads + 63) / 64 * 64);
        rms_norm_vec4_kernel<T, D, 1><<<n_rows, threads, 0, stream>>>(h, delta, n_partials, partial_stride, rows, weight, eps, out, width, write_h);
    } else if (aligned && quads <= 4096) {
        rms_norm_vec4_kernel<T, D, 4><<<n_rows, 1024, 0, stream>>>(h, delta, n_partials, partial_stride, rows, weight, eps, out, width, write_h);
    } else {
        const int threads = width >= 2048 ? 512 : 256;
        rms_norm_kernel<T, D><<<n_rows, threads, 0, stream>>>(h, delta, n_partials, partial_stride, rows, weight, eps,
                                                              out, width, write_h);
    }
}

template <typename T>
__global__ void residual_add_kernel(float* __restrict__ h, const T* __restrict__ delta, int64_t count) {
    const int64_t index = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index < count) h[index] += to_float(delta[index]);
}

// ---------------------------------------------------------------------------------------------
// cos and sin of position * inv_freq for every token of a step: angles in float64, so that the float32 values
// are the correctly rounded ones for any position. out[token][pair] = (cos, sin).
__global__ void rope_table_kernel(const int32_t* __restrict__ positions, const double* __restrict__ inv_freq,
                                  int n_freq, int64_t count, float2* __restrict__ out) {
    const int64_t index = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= count) return;
    const double angle = static_cast<double>(positions[index / n_freq]) * inv_freq[index % n_freq];
    out[index] = make_float2(static_cast<float>(cos(angle)), static_cast<float>(sin(angle)));
}

// One block per token (and group of heads). cos and sin come from the step's table, or are computed here
// the same way; they are put into LDS once and shared by the block's heads.
constexpr int kMaxHeadDim = 512;

template <typename In, typename T>
__global__ void qkv_rope_store_kernel(const In* __restrict__ qkv, int n_partials, int64_t partial_stride,
                                      const float* __restrict__ bias,
                                      const int32_t* __restrict__ positions,
                                      const int32_t* __restrict__ slot_mapping,
                                      const double* __restrict__ inv_freq, const float2* __restrict__ cos_sin, int n_freq,
                                      T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                      int heads, int kv_heads, int head_dim, int page_size, int pair_order) {
    __shared__ float cos_table[kMaxHeadDim / 2];
    __shared__ float sin_table[kMaxHeadDim / 2];
    const int token = blockIdx.x;
    const int position = positions[token];
    const int heads_per_block = gridDim.y == 1 ? heads + 2 * kv_heads : max(1, static_cast<int>(blockDim.x) / (head_dim / 2));
    const int first_head = blockIdx.y * heads_per_block;
    for (int index = threadIdx.x; index < n_freq; index += blockDim.x) {
        if (cos_sin) {
            const float2 both = cos_sin[static_cast<int64_t>(token) * n_freq + index];
            cos_table[index] = both.x;
            sin_table[index] = both.y;
        } else {
            const double angle = static_cast<double>(position) * inv_freq[index];
            cos_table[index] = static_cast<float>(cos(angle));
            sin_table[index] = static_cast<float>(sin(angle));
        }
    }
    __syncthreads();

    const int half = head_dim / 2;
    const int total_heads = heads + 2 * kv_heads;
    const int64_t in_row = static_cast<int64_t>(token) * total_heads * head_dim;
    const int slot = slot_mapping ? slot_mapping[token] : -1;
    const int64_t page = slot >= 0 ? slot / page_size : 0;
    const int offset = slot >= 0 ? slot % page_size : 0;
    const CacheLayout layout(kv_heads, page_size, head_dim);

    const int block_heads = min(heads_per_block, total_heads - first_head);
    for (int item = threadIdx.x; item < block_heads * half; item += blockDim.x) {
        const int head = first_head + item / half;
        const int pair = item % half;
        const bool is_value = head >= heads + kv_heads;
        int first, second;
        bool rotate;
        if (pair < n_freq) {
            first = pair;
            second = pair + n_freq;
            rotate = !is_value;
        } else {  // dims beyond the rotary part pass through, two per item
            first = 2 * n_freq + 2 * (pair - n_freq);
            second = first + 1;
            rotate = false;
        }
        const int column = head * head_dim;
        // With pair_order the input's query and key heads hold the two dims of a rotary pair side by side.
        const bool paired = pair_order && !is_value && pair < n_freq;
        const int in_first = paired ? 2 * pair : first, in_second = paired ? 2 * pair + 1 : second;
        float x1 = to_float(qkv[in_row + column + in_first]);
        float x2 = to_float(qkv[in_row + column + in_second]);
        for (int base = 1; base < n_partials; base += 8) {      // eight parts asked for at a time, then added in order
            float more1[8], more2[8];
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (base + j < n_partials) {
                    more1[j] = to_float(qkv[(base + j) * partial_stride + in_row + column + in_first]);
                    more2[j] = to_float(qkv[(base + j) * partial_stride + in_row + column + in_second]);
                }
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (base + j < n_partials) {
                    x1 += more1[j];
                    x2 += more2[j];
                }
        }
        if (bias) {
            x1 += bias[column + first];
            x2 += bias[column + second];
        }
        float y1 = x1, y2 = x2;
        if (rotate) {
            const float c = cos_table[pair], s = sin_table[pair];
            y1 = rotate_first(x1, x2, c, s);
            y2 = rotate_second(x1, x2, c, s);
        }
        if (head < heads) {
            T* q_row = q_out + (static_cast<int64_t>(token) * heads + head) * head_dim;
            q_row[first] = from_float<T>(y1);
            q_row[second] = from_float<T>(y2);
        } else if (slot >= 0 && !is_value) {
            const int kv_head = head - heads;
            k_cache[layout.k_at(page, kv_head, offset, first)] = from_float<T>(y1);
            k_cache[layout.k_at(page, kv_head, offset, second)] = from_float<T>(y2);
        } else if (slot >= 0) {
            const int kv_head = head - heads - kv_heads;
            v_cache[layout.v_at(page, kv_head, offset, first)] = from_float<T>(y1);
            v_cache[layout.v_at(page, kv_head, offset, second)] = from_float<T>(y2);
        }
    }
}

// The same for float32 projections in the ordinary column order whose heads rotate whole (2 n_freq = head_dim, a
// multiple of 8) with the step's table of cos and sin: a thread takes four pairs of a query or key head, or eight
// dims of a value head, with 16-byte loads. out is bfloat16 or float32.
template <typename T>
__device__ inline void store_four(T* target, float a, float b, float c, float d);
template <>
__device__ inline void store_four<float>(float* target, float a, float b, float c, float d) {
    *reinterpret_cast<float4*>(target) = make_float4(a, b, c, d);
}
template <>
__device__ inline void store_four<bf16>(bf16* target, float a, float b, float c, float d) {
    union { uint2 raw; bf16 v[4]; } four;
    four.v[0] = from_float<bf16>(a);
    four.v[1] = from_float<bf16>(b);
    four.v[2] = from_float<bf16>(c);
    four.v[3] = from_float<bf16>(d);
    *reinterpret_cast<uint2*>(target) = four.raw;
}

template <typename T>
__global__ void qkv_rope_store_vec4_kernel(const float* __restrict__ qkv, int n_partials, int64_t partial_stride,
                                           const float* __restrict__ bias, const int32_t* __restrict__ slot_mapping,
                                           const float2* __restrict__ cos_sin, T* __restrict__ q_out,
                                           T* __restrict__ k_cache, T* __restrict__ v_cache, int n_tokens, int heads,
                                           int kv_heads, int head_dim, int page_size) {
    const int groups = head_dim / 8;                       // items per head
    const int total_heads = heads + 2 * kv_heads;
    const int64_t item = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (item >= static_cast<int64_t>(n_tokens) * total_heads * groups) return;
    const int token = static_cast<int>(item / (total_heads * groups));
    const int rest = static_cast<int>(item % (total_heads * groups));
    const int head = rest / groups, group = rest % groups;
    const bool is_value = head >= heads + kv_heads;
    const int half = head_dim / 2;
    // A query or key head: dims 4 g .. 4 g + 3 and their partners half a head on. A value head: dims 8 g .. 8 g + 7.
    const int first = is_value ? 8 * group : 4 * group;
    const int second = is_value ? first + 4 : first + half;
    const int64_t column = static_cast<int64_t>(token) * total_heads * head_dim + head * head_dim;
    float4 x1 = *reinterpret_cast<const float4*>(qkv + column + first);
    float4 x2 = *reinterpret_cast<const float4*>(qkv + column + second);
    for (int part = 1; part < n_partials; ++part) {
        const float4 more1 = *reinterpret_cast<const float4*>(qkv + part * partial_stride + column + first);
        const float4 more2 = *reinterpret_cast<const float4*>(qkv + part * partial_stride + column + second);
        x1.x += more1.x; x1.y += more1.y; x1.z += more1.z; x1.w += more1.w;
        x2.x += more2.x; x2.y += more2.y; x2.z += more2.z; x2.w += more2.w;
    }
    if (bias) {
        const float4 b1 = *reinterpret_cast<const float4*>(bias + head * head_dim + first);
        const float4 b2 = *reinterpret_cast<const float4*>(bias + head * head_dim + second);
        x1.x += b1.x; x1.y += b1.y; x1.z += b1.z; x1.w += b1.w;
        x2.x += b2.x; x2.y += b2.y; x2.z += b2.z; x2.w += b2.w;
    }
    float4 y1 = x1, y2 = x2;
    if (!is_value) {
        const float4* table = reinterpret_cast<const float4*>(cos_sin + static_cast<int64_t>(token) * half + first);
        const float4 a = table[0], b = table[1];       // (cos, sin) of pairs first, first + 1 | first + 2, first + 3
        y1.x = rotate_first(x1.x, x2.x, a.x, a.y);  y2.x = rotate_second(x1.x, x2.x, a.x, a.y);
        y1.y = rotate_first(x1.y, x2.y, a.z, a.w);  y2.y = rotate_second(x1.y, x2.y, a.z, a.w);
        y1.z = rotate_first(x1.z, x2.z, b.x, b.y);  y2.z = rotate_second(x1.z, x2.z, b.x, b.y);
        y1.w = rotate_first(x1.w, x2.w, b.z, b.w);  y2.w = rotate_second(x1.w, x2.w, b.z, b.w);
    }
    if (head < heads) {
        T* q_row = q_out + (static_cast<int64_t>(token) * heads + head) * head_dim;
        store_four<T>(q_row + first, y1.x, y1.y, y1.z, y1.w);
        store_four<T>(q_row + second, y2.x, y2.y, y2.z, y2.w);
        return;
    }
    const int slot = slot_mapping ? slot_mapping[token] : -1;
    if (slot < 0) return;
    const CacheLayout layout(kv_heads, page_size, head_dim);
    const int64_t page = slot / page_size;
    const int offset = slot % page_size;
    if (!is_value) {     // four dims that are a multiple of 4 lie side by side in a key page
        const int kv_head = head - heads;
        store_four<T>(k_cache + layout.k_at(page, kv_head, offset, first), y1.x, y1.y, y1.z, y1.w);
        store_four<T>(k_cache + layout.k_at(page, kv_head, offset, second), y2.x, y2.y, y2.z, y2.w);
    } else {             // in a value page the positions of a dim lie side by side, not the dims
        const int kv_head = head - heads - kv_heads;
        const float values[8] = {y1.x, y1.y, y1.z, y1.w, y2.x, y2.y, y2.z, y2.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) v_cache[layout.v_at(page, kv_head, offset, first + i)] = from_float<T>(values[i]);
    }
}

// ---------------------------------------------------------------------------------------------
__device__ inline float stable_sigmoid(float value) {
    if (value >= 0.0f) return 1.0f / (1.0f + expf(-value));
    const float e = expf(value);
    return e / (1.0f + e);
}

template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gate, const T* __restrict__ up, int64_t in_stride,
                                T* __restrict__ out, int width) {
    const int token = blockIdx.y;
    const int column = blockIdx.x * blockDim.x + threadIdx.x;
    if (column >= width) return;
    const float g = to_float(gate[token * in_stride + column]);
    const float u = to_float(up[token * in_stride + column]);
    out[static_cast<int64_t>(token) * width + column] = from_float<T>(g * stable_sigmoid(g) * u);
}

// The same for bfloat16 rows whose width is a multiple of 8: 16 bytes of gate and of up per thread.
__global__ void silu_mul_bf16x8_kernel(const bf16* __restrict__ gate, const bf16* __restrict__ up, int64_t in_stride,
                                       bf16* __restrict__ out, int width) {
    const int token = blockIdx.y;
    const int chunk = blockIdx.x * blockDim.x + threadIdx.x;
    if (chunk * 8 >= width) return;
    union { uint4 raw; bf16 v[8]; } g, u, z;
    g.raw = *reinterpret_cast<const uint4*>(gate + token * in_stride + chunk * 8);
    u.raw = *reinterpret_cast<const uint4*>(up + token * in_stride + chunk * 8);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float gv = to_float(g.v[i]);
        z.v[i] = from_float<bf16>(gv * stable_sigmoid(gv) * to_float(u.v[i]));
    }
    *reinterpret_cast<uint4*>(out + static_cast<int64_t>(token) * width + chunk * 8) = z.raw;
}

}  // namespace mll

using namespace mll;

extern "C" {

const char* mll_last_error() { return g_error.c_str(); }
int mll_version() { return 1; }

int mll_embedding(const void* table, int table_dtype, const int32_t* ids, float* out,
                  int n_tokens, int width, int vocab, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && width > 0 && vocab > 0, "embedding: sizes must be positive");
    if (n_tokens == 0) return 0;
    if (table_dtype == kF32) {
        embedding_kernel<float><<<n_tokens, 256, 0, stream>>>(static_cast<const float*>(table), ids, out, width, vocab);
    } else if (table_dtype == kBF16) {
        embedding_kernel<bf16><<<n_tokens, 256, 0, stream>>>(static_cast<const bf16*>(table), ids, out, width, vocab);
    } else {
        return fail("embedding: unknown table dtype");
    }
    return check_launch("embedding");
}

int mll_rms_norm(float* h, const void* delta, int delta_dtype, int n_partials, int64_t partial_stride,
                 const int32_t* rows, const float* weight, float eps,
                 void* out, int dtype, int n_rows, int width, int write_h, hipStream_t stream) {
    MLL_REQUIRE(n_partials >= 1, "rms_norm: the delta needs at least one part");
    MLL_REQUIRE(n_rows >= 0 && width > 0, "rms_norm: sizes must be positive");
    MLL_REQUIRE(eps > 0.0f, "rms_norm: eps must be positive");
    MLL_REQUIRE(!(write_h && rows), "rms_norm: cannot write h through a row selection");
    if (n_rows == 0) return 0;
    if (dtype == kF32 && delta_dtype == kF32) {
        launch_rms_norm<float, float>(h, static_cast<const float*>(delta), n_partials, partial_stride, rows, weight, eps,
                                      static_cast<float*>(out), n_rows, width, write_h, stream);
    } else if (dtype == kBF16 && delta_dtype == kF32) {
        launch_rms_norm<bf16, float>(h, static_cast<const float*>(delta), n_partials, partial_stride, rows, weight, eps,
                                     static_cast<bf16*>(out), n_rows, width, write_h, stream);
    } else if (dtype == kBF16 && delta_dtype == kBF16) {
        launch_rms_norm<bf16, bf16>(h, static_cast<const bf16*>(delta), n_partials, partial_stride, rows, weight, eps,
                                    static_cast<bf16*>(out), n_rows, width, write_h, stream);
    } else {
        return fail("rms_norm: unsupported combination of output and delta dtypes");
    }
    return check_launch("rms_norm");
}

int mll_residual_add(float* h, const void* delta, int dtype, int n_rows, int width, hipStream_t stream) {
    const int64_t count = static_cast<int64_t>(n_rows) * width;
    if (count == 0) return 0;
    const int blocks = static_cast<int>((count + 255) / 256);
    if (dtype == kF32) {
        residual_add_kernel<float><<<blocks, 256, 0, stream>>>(h, static_cast<const float*>(delta), count);
    } else if (dtype == kBF16) {
        residual_add_kernel<bf16><<<blocks, 256, 0, stream>>>(h, static_cast<const bf16*>(delta), count);
    } else {
        return fail("residual_add: unknown dtype");
    }
    return check_launch("residual_add");
}

int mll_qkv_rope_store(const void* qkv, int in_dtype, int n_partials, int64_t partial_stride, int dtype,
                       const float* bias, const int32_t* positions,
                       const int32_t* slot_mapping, const double* inv_freq, const void* cos_sin, int n_freq,
                       void* q_out, void* k_cache, void* v_cache,
                       int n_tokens, int heads, int kv_heads, int head_dim, int page_size, int pair_order,
                       hipStream_t stream) {
    MLL_REQUIRE(heads > 0 && kv_heads >= 0 && head_dim > 0, "qkv_rope_store: sizes must be positive");
    MLL_REQUIRE(n_partials >= 1, "qkv_rope_store: the input needs at least one part");
    MLL_REQUIRE(head_dim % 2 == 0 && head_dim <= kMaxHeadDim, "qkv_rope_store: head_dim must be even and at most 512");
    MLL_REQUIRE(n_freq >= 0 && 2 * n_freq <= head_dim, "qkv_rope_store: rotary part exceeds head_dim");
    MLL_REQUIRE(inv_freq != nullptr || cos_sin != nullptr || n_freq == 0, "qkv_rope_store: n_freq without frequencies or a table of cos and sin");
    MLL_REQUIRE(cos_sin == nullptr || reinterpret_cast<uintptr_t>(cos_sin) % 8 == 0, "qkv_rope_store: the table of cos and sin must be 8-byte aligned");
    MLL_REQUIRE(slot_mapping == nullptr || (k_cache && v_cache && page_size > 0 && page_size % 16 == 0),
                "qkv_rope_store: slot_mapping needs both caches and a page size that is a multiple of 16");
    if (n_tokens == 0) return 0;
    // A block takes as many heads of one token as give its 256 threads one pair each.
    const int heads_per_block = max(1, 256 / (head_dim / 2));
    const dim3 grid(n_tokens, (heads + 2 * kv_heads + heads_per_block - 1) / heads_per_block);
    const bool wide = in_dtype == kF32 && cos_sin != nullptr && !pair_order && 2 * n_freq == head_dim && head_dim % 8 == 0 &&
                      n_tokens > 64 && reinterpret_cast<uintptr_t>(qkv) % 16 == 0 && partial_stride % 4 == 0 &&
                      reinterpret_cast<uintptr_t>(cos_sin) % 16 == 0 && (bias == nullptr || reinterpret_cast<uintptr_t>(bias) % 16 == 0) &&
                      reinterpret_cast<uintptr_t>(q_out) % 16 == 0 && reinterpret_cast<uintptr_t>(k_cache) % 16 == 0;
    if (wide) {
        const int64_t items = static_cast<int64_t>(n_tokens) * (heads + 2 * kv_heads) * (head_dim / 8);
        const unsigned blocks = static_cast<unsigned>((items + 255) / 256);
        if (dtype == kF32)
            qkv_rope_store_vec4_kernel<float><<<blocks, 256, 0, stream>>>(
                static_cast<const float*>(qkv), n_partials, partial_stride, bias, slot_mapping, static_cast<const float2*>(cos_sin),
                static_cast<float*>(q_out), static_cast<float*>(k_cache), static_cast<float*>(v_cache), n_tokens, heads, kv_heads,
                head_dim, page_size);
        else
            qkv_rope_store_vec4_kernel<bf16><<<blocks, 256, 0, stream>>>(
                static_cast<const float*>(qkv), n_partials, partial_stride, bias, slot_mapping, static_cast<const float2*>(cos_sin),
                static_cast<bf16*>(q_out), static_cast<bf16*>(k_cache), static_cast<bf16*>(v_cache), n_tokens, heads, kv_heads,
                head_dim, page_size);
        return check_launch("qkv_rope_store");
    }
    if (dtype == kF32 && in_dtype == kF32) {
        qkv_rope_store_kernel<float, float><<<grid, 256, 0, stream>>>(
            static_cast<const float*>(qkv), n_partials, partial_stride, bias, positions, slot_mapping, inv_freq, static_cast<const float2*>(cos_sin), n_freq,
            static_cast<float*>(q_out), static_cast<float*>(k_cache), static_cast<float*>(v_cache),
            heads, kv_heads, head_dim, page_size, pair_order);
    } else if (dtype == kBF16 && in_dtype == kF32) {
        qkv_rope_store_kernel<float, bf16><<<grid, 256, 0, stream>>>(
            static_cast<const float*>(qkv), n_partials, partial_stride, bias, positions, slot_mapping, inv_freq, static_cast<const float2*>(cos_sin), n_freq,
            static_cast<bf16*>(q_out), static_cast<bf16*>(k_cache), static_cast<bf16*>(v_cache),
            heads, kv_heads, head_dim, page_size, pair_order);
    } else if (dtype == kBF16 && in_dtype == kBF16) {
        qkv_rope_store_kernel<bf16, bf16><<<grid, 256, 0, stream>>>(
            static_cast<const bf16*>(qkv), n_partials, partial_stride, bias, positions, slot_mapping, inv_freq, static_cast<const float2*>(cos_sin), n_freq,
            static_cast<bf16*>(q_out), static_cast<bf16*>(k_cache), static_cast<bf16*>(v_cache),
            heads, kv_heads, head_dim, page_size, pair_order);
    } else {
        return fail("qkv_rope_store: unsupported combination of input and output dtypes");
    }
    return check_launch("qkv_rope_store");
}

int mll_rope_table(const int32_t* positions, const double* inv_freq, int n_freq, int n_tokens, float* out,
                   hipStream_t stream) {
    MLL_REQUIRE(n_freq > 0 && n_tokens >= 0, "rope_table: sizes must be positive");
    MLL_REQUIRE(reinterpret_cast<uintptr_t>(out) % 8 == 0, "rope_table: the table must be 8-byte aligned");
    if (n_tokens == 0) return 0;
    const int64_t count = static_cast<int64_t>(n_tokens) * n_freq;
    rope_table_kernel<<<static_cast<unsigned>((count + 255) / 256), 256, 0, stream>>>(positions, inv_freq, n_freq, count,
                                                                                      reinterpret_cast<float2*>(out));
    return check_launch("rope_table");
}

int mll_silu_mul(const void* gate, const void* up, int64_t in_stride, void* out, int dtype,
                 int n_tokens, int width, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && width > 0 && in_stride >= width, "silu_mul: bad sizes");
    if (n_tokens == 0) return 0;
    MLL_REQUIRE(n_tokens <= 65535, "silu_mul: more than 65535 tokens in one call");
    const dim3 grid((width + 255) / 256, n_tokens);
    if (dtype == kF32) {
        silu_mul_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(gate), static_cast<const float*>(up),
                                                         in_stride, static_cast<float*>(out), width);
    } else if (dtype == kBF16 && width % 8 == 0 && in_stride % 8 == 0 && reinterpret_cast<uintptr_t>(gate) % 16 == 0 &&
               reinterpret_cast<uintptr_t>(up) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
        const dim3 wide_grid((width / 8 + 255) / 256, n_tokens);
        silu_mul_bf16x8_kernel<<<wide_grid, 256, 0, stream>>>(static_cast<const bf16*>(gate), static_cast<const bf16*>(up),
                                                             in_stride, static_cast<bf16*>(out), width);
    } else if (dtype == kBF16) {
        silu_mul_kernel<bf16><<<grid, 256, 0, stream>>>(static_cast<const bf16*>(gate), static_cast<const bf16*>(up),
                                                        in_stride, static_cast<bf16*>(out), width);
    } else {
        return fail("silu_mul: unknown dtype");
    }
    return check_launch("silu_mul");
}

}  // extern "C"
