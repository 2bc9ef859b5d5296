// What this GPU reaches on the two things the engine is bound by, measured with kernels that do nothing else:
// reading memory once (the decode step's bound) and issuing v_mfma_f32_16x16x32_bf16 back to back (the prefill's).
// The benchmark quotes its fractions of the published peaks and of these.
#include "common.h"
#include "microllm_hip.h"

namespace mll {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

// Every 16 bytes of `data` are read once, by consecutive lanes; what is read is folded into one word per thread
// and written only if it has a value that random data never gives, so that the loads cannot be dropped.
__global__ __launch_bounds__(256) void read_once_kernel(const uintx4* __restrict__ data, int64_t count, unsigned* __restrict__ sink) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    uintx4 folded = uintx4{0u, 0u, 0u, 0u};
    int64_t index = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    for (; index + 3 * stride < count; index += 4 * stride) {       // four loads in flight per thread
        const uintx4 a = __builtin_nontemporal_load(data + index);
        const uintx4 b = __builtin_nontemporal_load(data + index + stride);
        const uintx4 c = __builtin_nontemporal_load(data + index + 2 * stride);
        const uintx4 d = __builtin_nontemporal_load(data + index + 3 * stride);
        folded ^= a ^ b ^ c ^ d;
    }
    for (; index < count; index += stride) folded ^= __builtin_nontemporal_load(data + index);
    const unsigned word = folded[0] ^ folded[1] ^ folded[2] ^ folded[3];
    if (word == 0x9e3779b9u) sink[0] = word;
}

// Each wave issues `iterations` rounds of 16 products into 16 accumulators of its own (no product waits for another's
// result within a round).
__global__ __launch_bounds__(256) void mfma_loop_kernel(int iterations, float* __restrict__ sink) {
    bf16x8 a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = static_cast<__bf16>(0.001f * static_cast<float>(threadIdx.x % 7 + i));
        b[i] = static_cast<__bf16>(0.002f * static_cast<float>(threadIdx.x % 5 + i));
    }
    floatx4 acc[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) acc[t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    for (int round = 0; round < iterations; ++round) {
#pragma unroll
        for (int t = 0; t < 16; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[t], 0, 0, 0);
    }
    float total = 0.0f;
#pragma unroll
    for (int t = 0; t < 16; ++t) total += acc[t][0] + acc[t][1] + acc[t][2] + acc[t][3];
    if (total == 12345.678f) sink[0] = total;
}

}  // namespace mll

using namespace mll;

extern "C" int mll_measure_read(const void* data, int64_t bytes, void* sink, int blocks, hipStream_t stream) {
    MLL_REQUIRE(bytes >= 16 && bytes % 16 == 0 && reinterpret_cast<uintptr_t>(data) % 16 == 0,
                "measure_read: give a 16-byte aligned buffer of a multiple of 16 bytes");
    MLL_REQUIRE(blocks > 0 && sink != nullptr, "measure_read: give a number of workgroups and a sink");
    read_once_kernel<<<blocks, 256, 0, stream>>>(static_cast<const uintx4*>(data), bytes / 16, static_cast<unsigned*>(sink));
    return check_launch("measure_read");
}

// Launches `blocks` workgroups of 4 waves; the flops issued are blocks * 4 * iterations * 16 * 16384.
extern "C" int mll_measure_mfma(int iterations, void* sink, int blocks, hipStream_t stream) {
    MLL_REQUIRE(iterations > 0 && blocks > 0 && sink != nullptr, "measure_mfma: give iterations, workgroups and a sink");
    mfma_loop_kernel<<<blocks, 256, 0, stream>>>(iterations, static_cast<float*>(sink));
    return check_launch("measure_mfma");
}
