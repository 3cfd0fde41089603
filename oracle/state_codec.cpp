// CPU oracle, the cached form of Gated DeltaNet recurrent layers (test infrastructure only; see oracle.h).
#include "oracle.h"
#include "common.hpp"

using namespace orc;

namespace {
constexpr uint32_t kBlock = 32;  // metal/abi/StateCodec.h:19
}

extern "C" {

uint64_t orc_state_codec_bytes(uint32_t rows, uint32_t columns) {
  // metal/abi/StateCodec.h:28-33: every value's code, row by row, then each block's bf16 scale
  return uint64_t(rows) * columns + uint64_t(rows) * (columns / kBlock) * 2;
}

// kernels/common/state_codec.h:19-35 and shared/state_codec.metal:15-47: a block's largest magnitude as bits (which put
// infinity and NaN above every finite value); its scale bf16(amax * (1 / 127)), a quiet NaN for a block that is not
// finite; a value's code rint(value / scale) within [-127, 127], the division correctly rounded, 0 when the scale is
// not positive.
int orc_state_codes(const float *values, uint32_t rows, uint32_t columns, uint8_t *image) {
  if (!rows || !columns || columns % kBlock) return -1;
  const uint64_t blocks = uint64_t(rows) * columns / kBlock, scales = uint64_t(rows) * columns;
  for (uint64_t b = 0; b < blocks; ++b) {
    const float *v = values + b * kBlock;
    uint32_t amax = 0;
    for (uint32_t i = 0; i < kBlock; ++i) {
      uint32_t bits; std::memcpy(&bits, v + i, 4);
      amax = std::max(amax, bits & 0x7FFFFFFFu);
    }
    uint16_t scale = 0x7FC0;
    if (amax < 0x7F800000u) {
      float magnitude; std::memcpy(&magnitude, &amax, 4);
      scale = f2bf(magnitude * (1.0f / 127.0f));
    }
    const float wide = bf2f(scale);
    for (uint32_t i = 0; i < kBlock; ++i) {
      int8_t code = 0;
      if (wide > 0.0f) code = int8_t(std::min(127.0f, std::max(-127.0f, std::nearbyintf(v[i] / wide))));
      image[b * kBlock + i] = uint8_t(code);
    }
    std::memcpy(image + scales + 2 * b, &scale, 2);
  }
  return 0;
}

// shared/state_codec.metal:49-62: value = float(code) * scale (one rounding; a bf16 state rounds it again).
int orc_state_values(const uint8_t *image, uint32_t rows, uint32_t columns, float *values) {
  if (!rows || !columns || columns % kBlock) return -1;
  const uint64_t count = uint64_t(rows) * columns;
  for (uint64_t i = 0; i < count; ++i) {
    uint16_t scale; std::memcpy(&scale, image + count + 2 * (i / kBlock), 2);
    values[i] = float(int8_t(image[i])) * bf2f(scale);
  }
  return 0;
}

} // extern "C"
