// Shared device helpers for the gfx950 math kernels (wave64 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace docc_k {

constexpr int kWave = 64;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

__device__ __forceinline__ double wave_max(double v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmax(v, __shfl_xor(v, off, kWave));
    return v;
}

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// exp(t) for t <= 0 through the hardware exp2 with a compensated argument:
// t*log2(e) is split into its rounded product and the rounding remainder, so
// the result stays within ~2 ulp down to the underflow threshold.
__device__ __forceinline__ float exp_neg(float t) {
    const float log2e_hi = 1.44269502162933349609375f;   // fp32(log2 e)
    const float log2e_lo = 1.925963033500011e-08f;       // log2 e - fp32(log2 e)
    const float ln2 = 0.693147182464599609375f;
    float hi = t * log2e_hi;
    float lo = __builtin_fmaf(t, log2e_hi, -hi) + t * log2e_lo;
    float e = __builtin_amdgcn_exp2f(hi);
    float r = __builtin_fmaf(e, lo * ln2, e);
    // below the smallest denormal the result is 0; this also keeps t = -inf
    // (whose compensation term would be inf - inf) away from the fma
    return (t < -104.0f) ? 0.0f : r;
}

// fp32 -> bf16 bits, round to nearest even, NaN kept quiet.
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t) ((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t) (u >> 16);
}

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) {
    return __builtin_bit_cast(float, (uint32_t) h << 16);
}

} // namespace docc_k
