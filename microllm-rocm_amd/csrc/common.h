// Shared device helpers for the gfx950 kernels: element types, wave reductions, error reporting.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cmath>
#include <cstdio>
#include <string>

namespace mll {

constexpr int kWave = 64;  // CDNA wavefront width

// Element type tags shared with the Python bindings.
enum DType : int { kF32 = 0, kBF16 = 1 };

// bfloat16 as raw bits: widening is a shift, narrowing rounds to nearest even.
struct bf16 {
    uint16_t bits;
};

__host__ __device__ inline float to_float(float value) { return value; }
__host__ __device__ inline float to_float(bf16 value) {
    union { uint32_t u; float f; } caster;
    caster.u = static_cast<uint32_t>(value.bits) << 16;
    return caster.f;
}

template <typename T> __host__ __device__ inline T from_float(float value);
template <> __host__ __device__ inline float from_float<float>(float value) { return value; }
template <> __host__ __device__ inline bf16 from_float<bf16>(float value) {
    union { uint32_t u; float f; } caster;
    caster.f = value;
    bf16 out;
    if ((caster.u & 0x7fffffffu) > 0x7f800000u) {  // NaN stays NaN
        out.bits = static_cast<uint16_t>((caster.u >> 16) | 0x0040u);
        return out;
    }
    const uint32_t rounding = 0x7fffu + ((caster.u >> 16) & 1u);
    out.bits = static_cast<uint16_t>((caster.u + rounding) >> 16);
    return out;
}

__device__ inline float wave_sum(float value) {
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) value += __shfl_xor(value, offset, kWave);
    return value;
}

__device__ inline float wave_max(float value) {
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) value = fmaxf(value, __shfl_xor(value, offset, kWave));
    return value;
}

// Sum over a block of up to 1024 threads; every thread gets the total. `scratch` holds 16 floats.
// The order of additions depends only on the block size, never on the data's place in a batch.
__device__ inline float block_sum(float value, float* scratch) {
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int waves = (blockDim.x + kWave - 1) / kWave;
    value = wave_sum(value);
    __syncthreads();  // scratch may still be read from an earlier call
    if (lane == 0) scratch[wave] = value;
    __syncthreads();
    float total = 0.0f;
    for (int index = 0; index < waves; ++index) total += scratch[index];
    return total;
}

// Host-side error text, one per thread, read through mll_last_error().
void set_error(const std::string& text);
int fail(const std::string& text);

inline int check_launch(const char* what) {
    const hipError_t status = hipGetLastError();
    if (status != hipSuccess) return fail(std::string(what) + ": " + hipGetErrorString(status));
    return 0;
}

}  // namespace mll

#define MLL_REQUIRE(condition, text)                         \
    do {                                                     \
        if (!(condition)) return ::mll::fail(text);          \
    } while (0)
