// The cached form of Gated DeltaNet recurrent layers (abi/StateCodec.h; the reference's shared/state_codec.metal and
// common/state_codec.h): int8 codes with one bf16 scale a block of 32 values, and back. A streaming kernel: a lane
// reads 16 bytes of an fp32 state (a wave 1 KiB, contiguous), the block's eight lanes share their largest magnitude
// by three cross-lane exchanges, and the lane writes its four codes as one word. 5.06 bytes move a value coded, as many
// a value restored.
#include "abi/StateCodec.h"
#include "backend/KernelRegistry.hpp"
#include "kernels/device_common.hpp"

namespace splash::kernels {
namespace {

// A value's magnitude as its bits: they order as the magnitudes do and put infinity, then NaN, above every finite one.
__device__ __forceinline__ uint32_t magnitude_bits(float v) { return __builtin_bit_cast(uint32_t, v) & 0x7FFFFFFFu; }
// The block's scale: its largest magnitude over 127 as bf16, a quiet NaN for a block that holds NaN or an infinity, so
// that every value of it restores as NaN rather than as a finite value the state never held.
__device__ __forceinline__ uint32_t block_scale_bits(uint32_t amax) {
  return amax < 0x7F800000u ? float_to_bf16_bits(__builtin_bit_cast(float, amax) * (1.0f / 127.0f)) : 0x7FC0u;
}
// rint(value / scale) within [-127, 127], the division correctly rounded: the codes IEEE arithmetic makes anywhere.
__device__ __forceinline__ uint32_t code_of(float value, float scale) {
  if (!(scale > 0.0f)) return 0u;
  const float q = fminf(fmaxf(rintf(__fdiv_rn(value, scale)), -127.0f), 127.0f);
  return uint32_t(int(q)) & 0xFFu;
}

template <bool Bf16> struct Quad;
template <> struct Quad<false> {
  static __device__ __forceinline__ void load(const uint8_t *layer, uint32_t quad, float v[4]) {
    const uint4 raw = load_stream(reinterpret_cast<const uint4 *>(layer) + quad);
    v[0] = __builtin_bit_cast(float, raw.x);
    v[1] = __builtin_bit_cast(float, raw.y);
    v[2] = __builtin_bit_cast(float, raw.z);
    v[3] = __builtin_bit_cast(float, raw.w);
  }
  static __device__ __forceinline__ void store(uint8_t *layer, uint32_t quad, const float v[4]) {
    reinterpret_cast<float4 *>(layer)[quad] = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <> struct Quad<true> {
  static __device__ __forceinline__ void load(const uint8_t *layer, uint32_t quad, float v[4]) {
    const uint2 raw = reinterpret_cast<const uint2 *>(layer)[quad];
    v[0] = bf16_bits_to_float(raw.x & 0xFFFFu);
    v[1] = bf16_bits_to_float(raw.x >> 16);
    v[2] = bf16_bits_to_float(raw.y & 0xFFFFu);
    v[3] = bf16_bits_to_float(raw.y >> 16);
  }
  static __device__ __forceinline__ void store(uint8_t *layer, uint32_t quad, const float v[4]) {
    reinterpret_cast<uint2 *>(layer)[quad] = make_uint2(float_to_bf16_bits(v[0]) | (float_to_bf16_bits(v[1]) << 16),
                                                        float_to_bf16_bits(v[2]) | (float_to_bf16_bits(v[3]) << 16));
  }
};

} // namespace

template <bool Bf16>
__global__ __launch_bounds__(256) void state_quantize(const uint8_t *__restrict__ state, uint8_t *__restrict__ codes,
                                                      StateCodecParams p) {
  const uint8_t *from = state + uint64_t(blockIdx.y) * p.state_layer_bytes;
  uint8_t *to = codes + uint64_t(blockIdx.y) * p.codes_layer_bytes;
  uint16_t *scales = reinterpret_cast<uint16_t *>(to + p.scales_offset);
  float v[STATE_CODEC_THREAD_QUADS][4];
  uint32_t quad[STATE_CODEC_THREAD_QUADS];
  // A block's eight lanes are in or out together: a layer holds whole blocks, and the lanes of one are neighbours
  // from a multiple of eight.
#pragma unroll
  for (uint32_t j = 0; j < STATE_CODEC_THREAD_QUADS; ++j) {
    quad[j] = (blockIdx.x * STATE_CODEC_THREAD_QUADS + j) * 256u + threadIdx.x;
    if (quad[j] < p.quads_per_layer) Quad<Bf16>::load(from, quad[j], v[j]);
    else v[j][0] = v[j][1] = v[j][2] = v[j][3] = 0.f;
  }
#pragma unroll
  for (uint32_t j = 0; j < STATE_CODEC_THREAD_QUADS; ++j) {
    uint32_t amax = max(max(magnitude_bits(v[j][0]), magnitude_bits(v[j][1])), max(magnitude_bits(v[j][2]), magnitude_bits(v[j][3])));
#pragma unroll
    for (int distance = 1; distance < 8; distance *= 2) amax = max(amax, uint32_t(__shfl_xor(int(amax), distance, 64)));
    const uint32_t scale = block_scale_bits(amax);
    const float wide = bf16_bits_to_float(scale);
    if (quad[j] < p.quads_per_layer) {
      reinterpret_cast<uint32_t *>(to)[quad[j]] =
          code_of(v[j][0], wide) | (code_of(v[j][1], wide) << 8) | (code_of(v[j][2], wide) << 16) | (code_of(v[j][3], wide) << 24);
      if ((threadIdx.x & 7u) == 0) scales[quad[j] / 8u] = uint16_t(scale);
    }
  }
}
SP_REGISTER_KERNEL("state_quantize", &state_quantize<false>);
SP_REGISTER_KERNEL("state_quantize_bf16_state", &state_quantize<true>);

// value = float(code) * scale, one rounding; a bf16 state rounds it again.
template <bool Bf16>
__global__ __launch_bounds__(256) void state_dequantize(const uint8_t *__restrict__ codes, uint8_t *__restrict__ state,
                                                        StateCodecParams p) {
  const uint8_t *from = codes + uint64_t(blockIdx.y) * p.codes_layer_bytes;
  uint8_t *to = state + uint64_t(blockIdx.y) * p.state_layer_bytes;
  const uint16_t *scales = reinterpret_cast<const uint16_t *>(from + p.scales_offset);
#pragma unroll
  for (uint32_t j = 0; j < STATE_CODEC_THREAD_QUADS; ++j) {
    const uint32_t quad = (blockIdx.x * STATE_CODEC_THREAD_QUADS + j) * 256u + threadIdx.x;
    if (quad >= p.quads_per_layer) continue;
    const uint32_t word = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(from) + quad);
    const float scale = bf16_bits_to_float(scales[quad / 8u]);
    float v[4];
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) v[i] = float(int(int8_t((word >> (8u * i)) & 0xFFu))) * scale;
    Quad<Bf16>::store(to, quad, v);
  }
}
SP_REGISTER_KERNEL("state_dequantize", &state_dequantize<false>);
SP_REGISTER_KERNEL("state_dequantize_bf16_state", &state_dequantize<true>);

// A cached state that keeps the running format: each layer's bytes as they are, 16 a thread.
__global__ __launch_bounds__(256) void state_copy(const uint8_t *__restrict__ from, uint8_t *__restrict__ to, StateCodecParams p) {
  const uint32_t vector = blockIdx.x * 256u + threadIdx.x;
  if (vector >= p.quads_per_layer) return;
  reinterpret_cast<uint4 *>(to + uint64_t(blockIdx.y) * p.codes_layer_bytes)[vector] =
      load_stream(reinterpret_cast<const uint4 *>(from + uint64_t(blockIdx.y) * p.state_layer_bytes) + vector);
}
SP_REGISTER_KERNEL("state_copy", &state_copy);

} // namespace splash::kernels
