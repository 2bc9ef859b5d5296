// Token selection on the device: argmax (first maximum, non-finite -> -1) and sampling from
// softmax(logits / temperature) over the top_k largest logits by inverse CDF in token order.
#include "common.h"
#include "microllm_hip.h"

#include <mutex>

namespace mll {

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
// prefix. Scratch: one slot per wave.
template <typename V>
__device__ inline V block_exclusive_scan(V value, V* wave_scratch) {
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
    V before = V(0);
    for (int index = 0; index < wave; ++index) before += wave_scratch[index];
    return before + inclusive - value;
}

// Sum over the wave, the same in every lane.
__device__ inline int wave_count(int value) {
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) value += __shfl_xor(value, offset, kWave);
    return value;
}

// Inclusive prefix sums over the wave in lane order.
template <typename V>
__device__ inline V wave_inclusive_scan(V value) {
    const int lane = threadIdx.x % kWave;
#pragma unroll
    for (int offset = 1; offset < kWave; offset <<= 1) {
        const V other = __shfl_up(value, offset, kWave);
        if (lane >= offset) value += other;
    }
    return value;
}

// ---- sampling ------------------------------------------------------------------------------------------------
// A row of a large vocabulary is too much for one workgroup (one compute unit waits for one load after the
// other): the row is cut into slices, a workgroup of 4 waves per slice, each wave taking a quarter (a "piece"),
// and the work into stages, one kernel each:
//   1. every slice's maximum, first maximum's index and whether it holds a non-finite value;
//   2. with top_k: the k-th largest key of the row by radix select, 11, 11 and 10 bits at a time: three kernels
//      that each add their slice's histogram of the next digit to the row's (integer adds: the order does not
//      matter); a kernel finds the digits of the earlier passes from those histograms itself;
//   3. every piece's sum of the weights exp(l/T - max/T) of the tokens above the k-th value, and how many tokens
//      equal it (which of those are in, the lowest ids first, depends on the pieces before);
//   4. one wave per row adds the pieces up in order, finds the piece into which uniform * total falls and walks
//      that piece token by token.
// Every sum has a fixed order: the drawn token depends on the row alone.
constexpr int kSliceThreads = 256;
constexpr int kSliceWaves = kSliceThreads / kWave;      // = pieces of a slice
constexpr int kRadixBins = 2048;
constexpr int kRadixPasses = 3;
constexpr int kBlockTokens = 4 * kWave;   // tokens a wave weighs at a time: four rows of one token per lane

struct SampleLayout {       // where a row's scratch lies, in 4-byte words from the row's start
    int slices, slice, piece;
    int parts, histograms, select, sums, equals, per_row;
};

__host__ __device__ inline SampleLayout sample_layout(int vocab) {
    SampleLayout layout;
    layout.slices = max(1, min(64, (vocab + 2047) / 2048));
    layout.slice = (vocab + layout.slices - 1) / layout.slices;
    layout.piece = (layout.slice + kSliceWaves - 1) / kSliceWaves;
    layout.parts = 0;
    layout.histograms = layout.parts + 4 * layout.slices;
    layout.select = layout.histograms + kRadixPasses * kRadixBins;
    layout.sums = layout.select + 4;
    layout.equals = layout.sums + kSliceWaves * layout.slices;
    layout.per_row = layout.equals + kSliceWaves * layout.slices;
    return layout;
}

__device__ inline void piece_bounds(const SampleLayout& layout, int vocab, int slice_index, int piece_index, int* begin, int* end) {
    const int slice_begin = min(slice_index * layout.slice, vocab);
    const int slice_end = min(slice_begin + layout.slice, vocab);
    *begin = min(slice_begin + piece_index * layout.piece, slice_end);
    *end = min(*begin + layout.piece, slice_end);
}

__device__ inline float value_of_key(uint32_t key) {
    return __uint_as_float((key & 0x80000000u) ? (key ^ 0x80000000u) : ~key);
}

// What a row asks for: drawn by weight among its top k, or simply its first maximum.
struct RowRule {
    float tau;
    int k;            // vocab: no restriction
    bool weighted;    // false: the first maximum (temperature 0 or top_k 1)
};

__device__ inline RowRule row_rule(const float* temperature, const int32_t* top_k, int row, int vocab) {
    RowRule rule;
    rule.tau = temperature[row];
    int k = top_k ? top_k[row] : 0;
    rule.weighted = !(rule.tau == 0.0f || k == 1);
    rule.k = (k <= 0 || k > vocab) ? vocab : k;
    return rule;
}

__global__ __launch_bounds__(kSliceThreads) void sample_slices_kernel(const float* __restrict__ logits,
                                                                      int32_t* __restrict__ workspace, int vocab) {
    __shared__ Best best_scratch[kSliceWaves];
    __shared__ int bad_scratch[kSliceWaves];
    const SampleLayout layout = sample_layout(vocab);
    int32_t* mine = workspace + static_cast<int64_t>(blockIdx.x) * layout.per_row;
    const int begin = min(static_cast<int>(blockIdx.y) * layout.slice, vocab);
    const int count = max(0, min(layout.slice, vocab - begin));
    bool bad;
    const Best best = block_argmax(logits + static_cast<int64_t>(blockIdx.x) * vocab + begin, count, &bad, best_scratch, bad_scratch);
    if (threadIdx.x == 0) {
        ArgmaxPart* parts = reinterpret_cast<ArgmaxPart*>(mine + layout.parts);
        parts[blockIdx.y] = ArgmaxPart{best.value, best.index == 0x7fffffff ? best.index : best.index + begin, bad ? 1 : 0, 0};
    }
    // the row's histograms start at zero: every slice clears its share
    for (int index = blockIdx.y * kSliceThreads + threadIdx.x; index < kRadixPasses * kRadixBins; index += layout.slices * kSliceThreads)
        mine[layout.histograms + index] = 0;
}

// The row's maximum (first index) and whether any slice saw a non-finite value; every thread gets the same.
__device__ inline Best row_best(const int32_t* mine, const SampleLayout& layout, bool* bad) {
    const ArgmaxPart* parts = reinterpret_cast<const ArgmaxPart*>(mine + layout.parts);
    Best best{-INFINITY, 0x7fffffff};
    int any_bad = 0;
    for (int index = 0; index < layout.slices; ++index) {
        const ArgmaxPart part = parts[index];
        best = better(best, Best{part.value, part.index});
        any_bad |= part.bad;
    }
    *bad = any_bad != 0;
    return best;
}

__device__ inline int radix_shift(int pass) { return pass == 0 ? 21 : (pass == 1 ? 10 : 0); }
__device__ inline int radix_bins(int pass) { return pass == 2 ? 1024 : kRadixBins; }

// The digit of pass `pass` of the remaining-th largest key among those that share the earlier digits: walks the
// row's histogram from the top. Thread t holds the counters bins - 1 - per * t downwards. All threads of the
// workgroup call it; the answer comes back in *prefix and *remaining.
__device__ inline void pick_digit(const int32_t* histogram, int pass, uint32_t* prefix, int* remaining, int* scan_scratch,
                                  uint32_t* shared_prefix, int* shared_remaining) {
    const int bins = radix_bins(pass);
    const int per = bins / kSliceThreads;      // 8 or 4
    const int top = bins - 1 - per * static_cast<int>(threadIdx.x);
    int count[8];
    int mine = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        count[j] = j < per ? histogram[top - j] : 0;
        mine += count[j];
    }
    const int above = block_exclusive_scan<int>(mine, scan_scratch);
    if (above < *remaining && *remaining <= above + mine) {
        int left = *remaining - above;
        int digit = top;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (j < per && left > count[j]) {
                left -= count[j];
                digit = top - j - 1;
            } else {
                break;
            }
        }
        *shared_prefix = *prefix | (static_cast<uint32_t>(digit) << radix_shift(pass));
        *shared_remaining = left;
    }
    __syncthreads();
    *prefix = *shared_prefix;
    *remaining = *shared_remaining;
    __syncthreads();
}

__global__ __launch_bounds__(kSliceThreads) void sample_histogram_kernel(
    const float* __restrict__ logits, const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    int32_t* __restrict__ workspace, int vocab, int pass) {
    __shared__ int histogram[kRadixBins];
    __shared__ int scan_scratch[kSliceWaves];
    __shared__ uint32_t shared_prefix;
    __shared__ int shared_remaining;
    const RowRule rule = row_rule(temperature, top_k, blockIdx.x, vocab);
    if (!rule.weighted || rule.k >= vocab) return;
    const SampleLayout layout = sample_layout(vocab);
    int32_t* mine = workspace + static_cast<int64_t>(blockIdx.x) * layout.per_row;
    const float* row = logits + static_cast<int64_t>(blockIdx.x) * vocab;
    const int lane = threadIdx.x % kWave;

    uint32_t prefix = 0, mask = 0;
    int remaining = rule.k;
    for (int earlier = 0; earlier < pass; ++earlier) {
        pick_digit(mine + layout.histograms + earlier * kRadixBins, earlier, &prefix, &remaining, scan_scratch, &shared_prefix, &shared_remaining);
        mask |= static_cast<uint32_t>(radix_bins(earlier) - 1) << radix_shift(earlier);
    }
    for (int index = threadIdx.x; index < kRadixBins; index += kSliceThreads) histogram[index] = 0;
    __syncthreads();
    const int shift = radix_shift(pass), bins = radix_bins(pass);
    const int begin = min(static_cast<int>(blockIdx.y) * layout.slice, vocab);
    const int end = min(begin + layout.slice, vocab);
    for (int base = begin; base < end; base += kSliceThreads) {
        const int index = base + threadIdx.x;
        const uint32_t key = index < end ? order_key(row[index]) : 0u;
        const bool counts = index < end && (key & mask) == prefix;
        const int bin = static_cast<int>((key >> shift) & static_cast<uint32_t>(bins - 1));
        // Logits of one row share their top bits: most lanes of a wave want the same few counters, and LDS adds
        // to one address one lane after the other. The lanes that want the first lane's counter are added by
        // that lane at once, three times over; the rest add for themselves.
        unsigned long long todo = __ballot(counts);
        for (int round = 0; round < 3 && todo != 0ull; ++round) {
            const int leader = __ffsll(static_cast<long long>(todo)) - 1;
            const int leader_bin = __shfl(bin, leader, kWave);
            const unsigned long long same = __ballot(counts && bin == leader_bin) & todo;
            if (lane == leader) atomicAdd(&histogram[leader_bin], __popcll(same));
            todo &= ~same;
        }
        if ((todo >> lane) & 1ull) atomicAdd(&histogram[bin], 1);
    }
    __syncthreads();
    for (int index = threadIdx.x; index < bins; index += kSliceThreads)
        if (histogram[index] != 0) atomicAdd(&mine[layout.histograms + pass * kRadixBins + index], histogram[index]);
}

__global__ __launch_bounds__(kSliceThreads) void sample_sums_kernel(
    const float* __restrict__ logits, const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    int32_t* __restrict__ workspace, int vocab) {
    __shared__ int scan_scratch[kSliceWaves];
    __shared__ uint32_t shared_prefix;
    __shared__ int shared_remaining;
    const RowRule rule = row_rule(temperature, top_k, blockIdx.x, vocab);
    if (!rule.weighted) return;
    const SampleLayout layout = sample_layout(vocab);
    int32_t* mine = workspace + static_cast<int64_t>(blockIdx.x) * layout.per_row;
    const float* row = logits + static_cast<int64_t>(blockIdx.x) * vocab;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    bool bad;
    const Best best = row_best(mine, layout, &bad);
    if (bad) return;

    uint32_t threshold_key = 0;   // the k-th largest key; keys above it are in, of its equals the first take_equal
    int take_equal = 0;
    if (rule.k < vocab) {
        int remaining = rule.k;
        for (int pass = 0; pass < kRadixPasses; ++pass)
            pick_digit(mine + layout.histograms + pass * kRadixBins, pass, &threshold_key, &remaining, scan_scratch, &shared_prefix, &shared_remaining);
        take_equal = remaining;
        if (blockIdx.y == 0 && threadIdx.x == 0) {
            mine[layout.select] = static_cast<int32_t>(threshold_key);
            mine[layout.select + 1] = take_equal;
        }
    }
    int begin, end;
    piece_bounds(layout, vocab, blockIdx.y, wave, &begin, &end);
    const float scaled_max = best.value / rule.tau;
    float lane_total = 0.0f;
    int lane_equal = 0;
    for (int base = begin; base < end; base += kBlockTokens) {
        float weight[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int index = base + j * kWave + lane;
            const float value = index < end ? row[index] : 0.0f;
            bool in = index < end;
            if (rule.k < vocab) {
                const uint32_t key = order_key(value);
                if (in && key == threshold_key) ++lane_equal;
                if (key <= threshold_key) in = false;
            }
            weight[j] = in ? expf(value / rule.tau - scaled_max) : 0.0f;
        }
        lane_total += (weight[0] + weight[1]) + (weight[2] + weight[3]);
    }
    const float total = wave_sum(lane_total);
    const int equal = wave_count(lane_equal);
    if (lane == 0) {
        reinterpret_cast<float*>(mine + layout.sums)[blockIdx.y * kSliceWaves + wave] = total;
        mine[layout.equals + blockIdx.y * kSliceWaves + wave] = equal;
    }
}

__global__ __launch_bounds__(kWave) void sample_draw_kernel(
    const float* __restrict__ logits, const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    const float* __restrict__ uniform, const int32_t* __restrict__ workspace, int32_t* __restrict__ out, int vocab) {
    const int row_index = blockIdx.x;
    const SampleLayout layout = sample_layout(vocab);
    const int32_t* mine = workspace + static_cast<int64_t>(row_index) * layout.per_row;
    const float* row = logits + static_cast<int64_t>(row_index) * vocab;
    const int lane = threadIdx.x;
    const RowRule rule = row_rule(temperature, top_k, row_index, vocab);
    bool bad;
    const Best best = row_best(mine, layout, &bad);
    if (bad || !rule.weighted) {
        if (lane == 0) out[row_index] = bad ? -1 : best.index;
        return;
    }
    const int k = rule.k;
    const float tau = rule.tau;
    const float scaled_max = best.value / tau;
    uint32_t threshold_key = 0;
    int take_equal = 0;
    float equal_weight = 0.0f;      // every token equal to the k-th value weighs the same
    if (k < vocab) {
        threshold_key = static_cast<uint32_t>(mine[layout.select]);
        take_equal = mine[layout.select + 1];
        equal_weight = expf(value_of_key(threshold_key) / tau - scaled_max);
    }

    // The pieces' sums in order: lane l holds pieces 4l .. 4l + 3.
    const int pieces = layout.slices * kSliceWaves;       // at most 256
    float piece_sum[4];
    int piece_equal[4];
    int lane_equal = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int piece = 4 * lane + j;
        piece_sum[j] = piece < pieces ? reinterpret_cast<const float*>(mine + layout.sums)[piece] : 0.0f;
        piece_equal[j] = (piece < pieces && k < vocab) ? mine[layout.equals + piece] : 0;
        lane_equal += piece_equal[j];
    }
    int equal_before[4];
    {
        int running = wave_inclusive_scan<int>(lane_equal) - lane_equal;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            equal_before[j] = running;
            const int taken = max(0, min(piece_equal[j], take_equal - running));
            piece_sum[j] += static_cast<float>(taken) * equal_weight;
            running += piece_equal[j];
        }
    }
    const float lane_sum = (piece_sum[0] + piece_sum[1]) + (piece_sum[2] + piece_sum[3]);
    const float inclusive = wave_inclusive_scan<float>(lane_sum);
    const float total = __shfl(inclusive, kWave - 1, kWave);
    const float exclusive_up = __shfl_up(inclusive, 1, kWave);
    const float target = uniform[row_index] * total;
    // The draw falls into the last piece that holds a selected token and begins at or below the target.
    float piece_before[4];
    int candidate = -1;
    {
        float running = lane == 0 ? 0.0f : exclusive_up;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            piece_before[j] = running;
            if (piece_sum[j] > 0.0f && running <= target) candidate = 4 * lane + j;
            running += piece_sum[j];
        }
    }
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) candidate = max(candidate, __shfl_xor(candidate, offset, kWave));
    if (candidate < 0) {      // cannot be: the piece of the maximum holds weight 1
        if (lane == 0) out[row_index] = best.index;
        return;
    }
    float before = 0.0f;
    int equal_seen = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float b = __shfl(piece_before[j], candidate / 4, kWave);
        const int e = __shfl(equal_before[j], candidate / 4, kWave);
        if (candidate % 4 == j) {
            before = b;
            equal_seen = e;
        }
    }
    int begin, end;
    piece_bounds(layout, vocab, candidate / kSliceWaves, candidate % kSliceWaves, &begin, &end);

    // The first selected token of the piece at which the running sum passes the target. A block's sum decides
    // whether to look inside it; inside, prefix sums in token order decide. Where rounding lets the target slip
    // past the last token, that last selected token is the one.
    const unsigned long long lanes_below = (1ull << lane) - 1ull;
    float running = before;
    int chosen = -1, last_selected = -1;
    for (int base = begin; base < end && chosen < 0; base += kBlockTokens) {
        float weight[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int index = base + j * kWave + lane;
            const float value = index < end ? row[index] : 0.0f;
            bool in = index < end;
            if (k < vocab) {
                const uint32_t key = order_key(value);
                const bool equal = in && key == threshold_key;
                const unsigned long long equals = __ballot(equal);
                if (key < threshold_key) in = false;
                if (equal && equal_seen + __popcll(equals & lanes_below) >= take_equal) in = false;
                equal_seen += __popcll(equals);
            }
            weight[j] = in ? expf(value / tau - scaled_max) : 0.0f;
        }
        const float block_total = wave_sum((weight[0] + weight[1]) + (weight[2] + weight[3]));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const unsigned long long selected = __ballot(weight[j] > 0.0f);
            if (selected != 0ull) last_selected = base + j * kWave + 63 - __clzll(static_cast<long long>(selected));
        }
        if (!(running + block_total > target)) {
            running += block_total;
            continue;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float within = wave_inclusive_scan<float>(weight[j]);
            const unsigned long long passed = __ballot(weight[j] > 0.0f && running + within > target);
            if (chosen < 0 && passed != 0ull) chosen = base + j * kWave + __ffsll(static_cast<long long>(passed)) - 1;
            running += __shfl(within, kWave - 1, kWave);
        }
    }
    if (chosen < 0) chosen = last_selected >= 0 ? last_selected : best.index;
    if (lane == 0) out[row_index] = chosen;
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

// The scratch of mll_argmax_static: the slices' results of its last call. One copy per GPU, held until the
// process ends. In host code this name is a stand-in for the symbol, not a device address: the address on a GPU
// comes from hipGetSymbolAddress with that GPU current, and only that address is handed to kernels.
static __device__ __align__(256) unsigned char argmax_static_scratch[MLL_ARGMAX_STATIC_MAX_PARTS * sizeof(mll::ArgmaxPart)];

namespace {

constexpr int kStaticMaxDevices = 64;
std::mutex static_scratch_mutex;
void* static_scratch_of_device[kStaticMaxDevices] = {};

// The address of argmax_static_scratch on the current GPU, asked for once per GPU; null after fail().
void* argmax_static_scratch_here() {
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kStaticMaxDevices) {
        fail("argmax_static: no current GPU, or its index is beyond 63");
        return nullptr;
    }
    std::lock_guard<std::mutex> guard(static_scratch_mutex);
    if (static_scratch_of_device[device] == nullptr) {
        void* address = nullptr;
        const hipError_t status = hipGetSymbolAddress(&address, HIP_SYMBOL(argmax_static_scratch));
        if (status != hipSuccess || address == nullptr) {
            fail(std::string("argmax_static: hipGetSymbolAddress: ") + hipGetErrorString(status));
            return nullptr;
        }
        static_scratch_of_device[device] = address;
    }
    return static_scratch_of_device[device];
}

}  // namespace

extern "C" int mll_argmax_static(const float* logits, int32_t* out, int n_rows, int vocab, hipStream_t stream) {
    MLL_REQUIRE(n_rows >= 0 && vocab > 0, "argmax_static: sizes must be positive");
    MLL_REQUIRE(logits != nullptr && out != nullptr, "argmax_static: logits and out are required");
    const int64_t parts_needed = static_cast<int64_t>(n_rows) * mll_argmax_slices(vocab);
    MLL_REQUIRE(n_rows <= 65535 && parts_needed <= MLL_ARGMAX_STATIC_MAX_PARTS,
                "argmax_static: rows x slices is " + std::to_string(parts_needed) + ", beyond the static scratch of " +
                    std::to_string(MLL_ARGMAX_STATIC_MAX_PARTS) + " (use mll_argmax with a scratch of the caller's)");
    if (n_rows == 0) return 0;
    void* parts = argmax_static_scratch_here();
    if (parts == nullptr) return 1;
    // Every slice of every row of this call is written by the first kernel before the second reads it: nothing
    // of an earlier call's contents is read, so nothing has to be cleared.
    return mll_argmax(logits, out, parts, n_rows, vocab, stream);
}

extern "C" int64_t mll_sample_workspace(int n_rows, int vocab) {
    if (n_rows <= 0 || vocab <= 0) return 0;
    return static_cast<int64_t>(n_rows) * sample_layout(vocab).per_row * 4;
}

extern "C" int mll_sample(const float* logits, const float* temperature, const int32_t* top_k,
                          const float* uniform, int32_t* out, void* workspace, int n_rows, int vocab,
                          hipStream_t stream) {
    MLL_REQUIRE(n_rows >= 0 && vocab > 0, "sample: sizes must be positive");
    MLL_REQUIRE(temperature && uniform, "sample: temperature and uniform are required");
    MLL_REQUIRE(n_rows <= 65535, "sample: more than 65535 rows");
    if (n_rows == 0) return 0;
    MLL_REQUIRE(workspace != nullptr, "sample: needs its workspace");
    const SampleLayout layout = sample_layout(vocab);
    int32_t* words = static_cast<int32_t*>(workspace);
    const dim3 grid(n_rows, layout.slices);
    sample_slices_kernel<<<grid, kSliceThreads, 0, stream>>>(logits, words, vocab);
    if (top_k != nullptr)
        for (int pass = 0; pass < kRadixPasses; ++pass)
            sample_histogram_kernel<<<grid, kSliceThreads, 0, stream>>>(logits, temperature, top_k, words, vocab, pass);
    sample_sums_kernel<<<grid, kSliceThreads, 0, stream>>>(logits, temperature, top_k, words, vocab);
    sample_draw_kernel<<<n_rows, kWave, 0, stream>>>(logits, temperature, top_k, uniform, words, out, vocab);
    return check_launch("sample");
}
