// Shared device helpers for the gfx950 attention kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "rt_kernels.hpp"

namespace rt {

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

// bf16 bit pattern <-> f32.  Round to nearest even; NaN stays a quiet NaN.
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float x) {
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
// Two f32 -> packed bf16x2 (lo in bits 0..15).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return (uint32_t)f32_to_bf16_bits(lo) | ((uint32_t)f32_to_bf16_bits(hi) << 16);
}
__device__ __forceinline__ float bf16_lo(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t packed) { return __uint_as_float(packed & 0xffff0000u); }

// Value held by the lane 32 positions away (the other half of the wave).
__device__ __forceinline__ float other_half(float x) { return __shfl_xor(x, 32, 64); }

__device__ __forceinline__ float quiet_nan() { return __uint_as_float(0x7fc00000u); }
__device__ __forceinline__ float neg_inf() { return __uint_as_float(0xff800000u); }

}  // namespace rt
