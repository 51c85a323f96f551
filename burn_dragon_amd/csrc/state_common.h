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

// two floats rounded to bf16 by the hardware conversion (v_cvt_pk_bf16_f32: nearest even, the bits of f32_to_bf16
// for every finite value), packed low | high
__device__ __forceinline__ unsigned int pack_bf16_rne(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  const f32x2_t a = {lo, hi};
  return __builtin_bit_cast(unsigned int, __builtin_convertvector(a, bf16x2_t));
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
