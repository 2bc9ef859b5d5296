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

// A rotation by (cos, sin) with its roundings spelled out (one product rounded, then one fused multiply-add), so
// that every kernel that rotates gives the same bits whatever the compiler would contract.
__device__ inline float rotate_first(float x1, float x2, float c, float s) { return fmaf(x1, c, -(x2 * s)); }
__device__ inline float rotate_second(float x1, float x2, float c, float s) { return fmaf(x1, s, x2 * c); }

// Waits until every load this wave has issued has arrived. The compiler waits by itself for loads into registers;
// loads from memory straight into LDS return nothing to wait for, so whoever reads that LDS calls this first (and
// then a barrier, if another wave's loads are read).
__device__ inline void wait_for_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// op over the four lanes {l, l ^ 16, l ^ 32, l ^ 48} of a wave, every one of which gets the result: two
// exchanges on the vector unit (v_permlane16_swap, v_permlane32_swap of gfx950) instead of four trips through
// LDS. op must be commutative. (The elements of the builtins' result are copied to scalars before they are
// reinterpreted: a reinterpretation of the element expression itself reads element 0 twice with this compiler.)
template <typename Op>
__device__ inline float reduce_lanes_16_apart(float value, Op op) {
    const unsigned bits = __builtin_bit_cast(unsigned, value);
    const auto rows = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
    const unsigned even = rows[0], odd = rows[1];
    value = op(__builtin_bit_cast(float, even), __builtin_bit_cast(float, odd));
    const unsigned joined = __builtin_bit_cast(unsigned, value);
    const auto halves = __builtin_amdgcn_permlane32_swap(joined, joined, false, false);
    const unsigned low = halves[0], high = halves[1];
    return op(__builtin_bit_cast(float, low), __builtin_bit_cast(float, high));
}
__device__ inline float max_lanes_16_apart(float value) {
    return reduce_lanes_16_apart(value, [](float a, float b) { return fmaxf(a, b); });
}
__device__ inline float sum_lanes_16_apart(float value) {
    return reduce_lanes_16_apart(value, [](float a, float b) { return a + b; });
}

template <typename T> __host__ __device__ inline T from_float(float value);
template <> __host__ __device__ inline float from_float<float>(float value) { return value; }
template <> __host__ __device__ inline bf16 from_float<bf16>(float value) {
    bf16 out;
#if defined(__HIP_DEVICE_COMPILE__)
    // Round to nearest even in one instruction (v_cvt_pk_bf16_f32 of gfx950); a NaN stays a NaN.
    out.bits = __builtin_bit_cast(uint16_t, static_cast<__bf16>(value));
#else
    union { uint32_t u; float f; } caster;
    caster.f = value;
    if ((caster.u & 0x7fffffffu) > 0x7f800000u) {  // NaN stays NaN
        out.bits = static_cast<uint16_t>((caster.u >> 16) | 0x0040u);
        return out;
    }
    const uint32_t rounding = 0x7fffu + ((caster.u >> 16) & 1u);
    out.bits = static_cast<uint16_t>((caster.u + rounding) >> 16);
#endif
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
