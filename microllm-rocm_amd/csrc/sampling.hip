// Token selection on the device: argmax (first maximum, non-finite -> -1) and sampling from
// softmax(logits / temperature) over the top_k largest logits by inverse CDF in token order.
// One block of 1024 threads per row; thread t owns the contiguous tokens [t * chunk, (t+1) * chunk).
#include "common.h"
#include "microllm_hip.h"

namespace mll {

constexpr int kSampleThreads = 1024;
constexpr int kSampleWaves = kSampleThreads / kWave;

// Monotone map from float to unsigned: a larger float gives a larger key.
__device__ inline uint32_t order_key(float value) {
    const uint32_t bits = __float_as_uint(value);
    return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
}

struct Best {
    float value;
    int index;
};

__device__ inline Best better(Best a, Best b) {
    if (b.value > a.value || (b.value == a.value && b.index < a.index)) return b;
    return a;
}

// Block-wide first maximum; also reports whether any value was non-finite.
__device__ inline Best block_argmax(const float* row, int vocab, bool* bad, Best* best_scratch, int* bad_scratch) {
    Best best{-INFINITY, 0x7fffffff};
    int non_finite = 0;
    for (int index = threadIdx.x; index < vocab; index += blockDim.x) {
        const float value = row[index];
        if (!isfinite(value)) non_finite = 1;
        if (value > best.value) best = Best{value, index};  // ascending index: keeps the first maximum
    }
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) {
        Best other{__shfl_xor(best.value, offset, kWave), __shfl_xor(best.index, offset, kWave)};
        best = better(best, other);
        non_finite |= __shfl_xor(non_finite, offset, kWave);
    }
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) {
        best_scratch[wave] = best;
        bad_scratch[wave] = non_finite;
    }
    __syncthreads();
    Best total = best_scratch[0];
    int any_bad = bad_scratch[0];
    for (int index = 1; index < blockDim.x / kWave; ++index) {
        total = better(total, best_scratch[index]);
        any_bad |= bad_scratch[index];
    }
    *bad = any_bad != 0;
    return total;
}

// Two stages, so that a row of a large vocabulary is scanned by many blocks: blockIdx.y takes a slice of the
// row and leaves (value, index, any non-finite) in `parts`; the second stage picks among the slices.
constexpr int kArgmaxThreads = 256;

struct ArgmaxPart {
    float value;
    int index;
    int bad;
    int pad;
};

__global__ __launch_bounds__(kArgmaxThreads) void argmax_slices_kernel(const float* __restrict__ logits,
                                                                       ArgmaxPart* __restrict__ parts, int vocab,
                                                                       int slice) {
    __shared__ Best best_scratch[kArgmaxThreads / kWave];
    __shared__ int bad_scratch[kArgmaxThreads / kWave];
    const int begin = blockIdx.y * slice;
    const int count = max(0, min(slice, vocab - begin));
    const float* row = logits + static_cast<int64_t>(blockIdx.x) * vocab + begin;
    bool bad;
    const Best best = block_argmax(row, count, &bad, best_scratch, bad_scratch);
    if (threadIdx.x == 0)
        parts[blockIdx.x * gridDim.y + blockIdx.y] = ArgmaxPart{best.value, best.index == 0x7fffffff ? best.index : best.index + begin, bad ? 1 : 0, 0};
}

__global__ __launch_bounds__(kWave) void argmax_pick_kernel(const ArgmaxPart* __restrict__ parts,
                                                           int32_t* __restrict__ out, int n_slices) {
    Best best{-INFINITY, 0x7fffffff};
    int bad = 0;
    for (int index = threadIdx.x; index < n_slices; index += kWave) {
        const ArgmaxPart part = parts[blockIdx.x * n_slices + index];
        best = better(best, Best{part.value, part.index});
        bad |= part.bad;
    }
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) {
        best = better(best, Best{__shfl_xor(best.value, offset, kWave), __shfl_xor(best.index, offset, kWave)});
        bad |= __shfl_xor(bad, offset, kWave);
    }
    if (threadIdx.x == 0) out[blockIdx.x] = bad ? -1 : best.index;
}

// Exclusive scan of one value per thread over the block, in thread order; returns the exclusive
// prefix and writes the block total to *total. Scratch: one slot per wave.
template <typename V>
__device__ inline V block_exclusive_scan(V value, V* wave_scratch, V* total) {
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    V inclusive = value;
#pragma unroll
    for (int offset = 1; offset < kWave; offset <<= 1) {
        const V other = __shfl_up(inclusive, offset, kWave);
        if (lane >= offset) inclusive += other;
    }
    __syncthreads();
    if (lane == kWave - 1) wave_scratch[wave] = inclusive;
    __syncthreads();
    V before = V(0), sum = V(0);
    for (int index = 0; index < kSampleWaves; ++index) {
        if (index < wave) before += wave_scratch[index];
        sum += wave_scratch[index];
    }
    *total = sum;
    return before + inclusive - value;
}

__global__ __launch_bounds__(kSampleThreads) void sample_kernel(
    const float* __restrict__ logits, const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    const float* __restrict__ uniform, int32_t* __restrict__ out, int vocab) {
    __shared__ Best best_scratch[kSampleWaves];
    __shared__ int bad_scratch[kSampleWaves];
    __shared__ int histogram[256];
    __shared__ float float_scratch[kSampleWaves];
    __shared__ int int_scratch[kSampleWaves];
    __shared__ uint32_t shared_prefix;
    __shared__ int shared_remaining;
    __shared__ int shared_winner;

    const int row_index = blockIdx.x;
    const float* row = logits + static_cast<int64_t>(row_index) * vocab;
    bool bad;
    const Best best = block_argmax(row, vocab, &bad, best_scratch, bad_scratch);
    const float tau = temperature[row_index];
    int k = top_k ? top_k[row_index] : 0;
    if (bad || tau == 0.0f || k == 1) {
        if (threadIdx.x == 0) out[row_index] = bad ? -1 : best.index;
        return;
    }
    if (k <= 0 || k > vocab) k = vocab;

    // Radix select of the k-th largest key, 8 bits a pass from the top.
    uint32_t threshold_key = 0;   // smallest key still selected
    int take_equal = 0;           // how many tokens equal to the threshold are taken, lowest index first
    if (k < vocab) {
        uint32_t prefix = 0, mask = 0;
        int remaining = k;
        for (int shift = 24; shift >= 0; shift -= 8) {
            for (int index = threadIdx.x; index < 256; index += blockDim.x) histogram[index] = 0;
            __syncthreads();
            for (int index = threadIdx.x; index < vocab; index += blockDim.x) {
                const uint32_t key = order_key(row[index]);
                if ((key & mask) == prefix) atomicAdd(&histogram[(key >> shift) & 0xffu], 1);
            }
            __syncthreads();
            if (threadIdx.x == 0) {
                int left = remaining;
                int bucket = 255;
                for (; bucket > 0; --bucket) {
                    if (histogram[bucket] >= left) break;
                    left -= histogram[bucket];
                }
                shared_prefix = prefix | (static_cast<uint32_t>(bucket) << shift);
                shared_remaining = left;
            }
            __syncthreads();
            prefix = shared_prefix;
            remaining = shared_remaining;
            mask |= 0xffu << shift;
            __syncthreads();
        }
        threshold_key = prefix;
        take_equal = remaining;  // of the tokens whose key equals the threshold
    }

    const int chunk = (vocab + kSampleThreads - 1) / kSampleThreads;
    const int begin = min(threadIdx.x * chunk, vocab);
    const int end = min(begin + chunk, vocab);
    const float scaled_max = best.value / tau;

    // Rank of this thread's first threshold-equal token among all of them, in token order.
    int equal_before = 0;
    if (k < vocab) {
        int equal_here = 0;
        for (int index = begin; index < end; ++index) equal_here += order_key(row[index]) == threshold_key;
        int equal_total;
        equal_before = block_exclusive_scan<int>(equal_here, int_scratch, &equal_total);
    }

    auto weight_of = [&](int index, int* equal_rank) -> float {
        const float value = row[index];
        if (k < vocab) {
            const uint32_t key = order_key(value);
            if (key < threshold_key) return 0.0f;
            if (key == threshold_key && (*equal_rank)++ >= take_equal) return 0.0f;
        }
        return expf(value / tau - scaled_max);
    };

    float chunk_sum = 0.0f;
    int rank = equal_before;
    for (int index = begin; index < end; ++index) chunk_sum += weight_of(index, &rank);
    float total;
    const float before = block_exclusive_scan<float>(chunk_sum, float_scratch, &total);
    const float target = uniform[row_index] * total;

    if (threadIdx.x == 0) shared_winner = 0x7fffffff;
    __syncthreads();
    if (chunk_sum > 0.0f && target >= before && target < before + chunk_sum) {
        float running = before;
        int chosen = -1, last_selected = -1;
        rank = equal_before;
        for (int index = begin; index < end; ++index) {
            const float weight = weight_of(index, &rank);
            if (weight > 0.0f) {
                last_selected = index;
                running += weight;
                if (running > target) {
                    chosen = index;
                    break;
                }
            }
        }
        if (chosen < 0) chosen = last_selected;  // rounding at the chunk's end
        atomicMin(&shared_winner, chosen);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        // target == total can only come from rounding; the argmax is always a selected token.
        out[row_index] = shared_winner == 0x7fffffff ? best.index : shared_winner;
    }
}

}  // namespace mll

using namespace mll;

extern "C" int mll_argmax_slices(int vocab) { return max(1, min(64, (vocab + 2047) / 2048)); }

extern "C" int mll_argmax(const float* logits, int32_t* out, void* parts, int n_rows, int vocab, hipStream_t stream) {
    MLL_REQUIRE(n_rows >= 0 && vocab > 0, "argmax: sizes must be positive");
    MLL_REQUIRE(parts != nullptr, "argmax: needs the scratch for its slices");
    MLL_REQUIRE(n_rows <= 65535, "argmax: more than 65535 rows");
    if (n_rows == 0) return 0;
    const int slices = mll_argmax_slices(vocab);
    const int slice = (vocab + slices - 1) / slices;
    argmax_slices_kernel<<<dim3(n_rows, slices), kArgmaxThreads, 0, stream>>>(logits, static_cast<ArgmaxPart*>(parts), vocab, slice);
    argmax_pick_kernel<<<n_rows, kWave, 0, stream>>>(static_cast<const ArgmaxPart*>(parts), out, slices);
    return check_launch("argmax");
}

extern "C" int mll_sample(const float* logits, const float* temperature, const int32_t* top_k,
                          const float* uniform, int32_t* out, int n_rows, int vocab, hipStream_t stream) {
    MLL_REQUIRE(n_rows >= 0 && vocab > 0, "sample: sizes must be positive");
    MLL_REQUIRE(temperature && uniform, "sample: temperature and uniform are required");
    if (n_rows == 0) return 0;
    sample_kernel<<<n_rows, kSampleThreads, 0, stream>>>(logits, temperature, top_k, uniform, out, vocab);
    return check_launch("sample");
}
