// The cached form of Gated DeltaNet recurrent layers, shared by the host operator and the HIP kernels (the counterpart
// of the reference's runtime/metal/abi/StateCodec.h): a layer's values as int8 codes, row by row as the running state
// holds them, then a bf16 scale for each block of 32 consecutive values.
#pragma once
#include <stdint.h>

#define STATE_CODEC_BLOCK 32u
// A lane holds four consecutive values (16 bytes of an fp32 state), eight neighbouring lanes a block.
#define STATE_CODEC_LANE_VALUES 4u
// Quads a thread takes, a workgroup's width apart.
#define STATE_CODEC_THREAD_QUADS 2u

#if defined(__HIPCC__) || defined(__cplusplus)
constexpr inline uint64_t state_codec_scales_offset(uint32_t rows, uint32_t columns) { return uint64_t(rows) * columns; }
constexpr inline uint64_t state_codec_layer_bytes(uint32_t rows, uint32_t columns) {
  return state_codec_scales_offset(rows, columns) + uint64_t(rows) * (columns / STATE_CODEC_BLOCK) * 2u;
}
#endif

// state_quantize[_bf16_state], state_dequantize[_bf16_state]: grid (ceil(quads_per_layer / (256 * 2)), layers), 256
// threads; layer y of the running state is state_layer_bytes after the last, of the cached one codes_layer_bytes.
// state_copy: quads_per_layer counts 16-byte vectors of a layer's state, moved as they are.
struct StateCodecParams {
  uint64_t state_layer_bytes;
  uint64_t codes_layer_bytes;
  uint64_t scales_offset;
  uint32_t quads_per_layer;
  uint32_t padding;
};
#if defined(__cplusplus)
static_assert(sizeof(StateCodecParams) == 32, "state codec parameters are 32 bytes on both sides");
#endif
