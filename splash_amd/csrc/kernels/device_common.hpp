// Scalar conversions, MFMA operand types and wavefront reductions shared by the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace splash::kernels {

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) int i32x4;

constexpr int kWave = 64;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// A 128-bit load of data read once (weights, KV pages): the non-temporal hint keeps it from
// displacing the activations every wave re-reads from the caches.
__device__ __forceinline__ uint4 load_stream(const uint4 *p) {
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ float half_bits_to_float(uint32_t bits) {
  return __half2float(__ushort_as_half(static_cast<unsigned short>(bits)));
}
__device__ __forceinline__ uint32_t float_to_half_bits(float v) { return __half_as_ushort(__float2half_rn(v)); }
__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits) { return __uint_as_float(bits << 16); }
// Round to nearest even; NaN stays NaN.
__device__ __forceinline__ uint32_t float_to_bf16_bits(float v) {
  uint32_t u = __float_as_uint(v);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x40u;
  u += 0x7FFFu + ((u >> 16) & 1u);
  return u >> 16;
}
__device__ __forceinline__ float round_bf16(float v) { return bf16_bits_to_float(float_to_bf16_bits(v)); }

// x / (1 + 2^(-log2(e) x)), the reference's silu (kernels/common/activation.h:8-16).
__device__ __forceinline__ float silu(float x) { return x / (1.0f + exp2f(-1.4426950408889634f * x)); }

__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

template <class T> __device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
template <class T> __device__ __forceinline__ T wave_max(T v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) { const T other = __shfl_xor(v, o, 64); v = other > v ? other : v; }
  return v;
}

} // namespace splash::kernels
