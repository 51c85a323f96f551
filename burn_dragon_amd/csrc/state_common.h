// Device helpers shared by the state-step translation units (state_step.hip, state_deferred.hip): the RoPE
// phase of src/model/attention.rs:338-343, bf16 conversion of a stored state, the element bitmask layout.
// Internal linkage: every translation unit gets its own copy.
#pragma once

#include <hip/hip_runtime.h>

namespace {

// f32(2*PI) exactly as `2.0 * PI` evaluates with std::f32::consts::PI
// (src/model/attention.rs:343)
constexpr float kTwoPi = 6.28318530717958647692f;

__device__ __forceinline__ float rope_phase(float pos, float f) {
  const float raw = pos * f;  // contraction is off for this file: two roundings, as the reference
  return (raw - floorf(raw)) * kTwoPi;
}

__device__ __forceinline__ float softplus1(float x) { return logf(expf(x * 1.0f) + 1.0f) / 1.0f; }

__device__ __forceinline__ float bf16_to_f32(unsigned short v) {
  return __uint_as_float(static_cast<unsigned int>(v) << 16);
}
__device__ __forceinline__ unsigned short f32_to_bf16(float f) {  // round to nearest even
  unsigned int u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<unsigned short>((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<unsigned short>(u >> 16);
}

// spread the 32 bits of v to the even bit positions of a 64-bit word
__device__ __forceinline__ unsigned long long spread_bits(unsigned int v) {
  unsigned long long x = v;
  x = (x | (x << 16)) & 0x0000FFFF0000FFFFull;
  x = (x | (x << 8)) & 0x00FF00FF00FF00FFull;
  x = (x | (x << 4)) & 0x0F0F0F0F0F0F0F0Full;
  x = (x | (x << 2)) & 0x3333333333333333ull;
  x = (x | (x << 1)) & 0x5555555555555555ull;
  return x;
}

}  // namespace
