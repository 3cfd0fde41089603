// The cached form of Gated DeltaNet recurrent layers: the counterpart of the reference's ops::StateCodec
// (runtime/ops/StateCodec.hpp:11-49). A running state's layers are quantized into a cached state's (int8 codes, a bf16
// scale per block of 32 values: abi/StateCodec.h) and dequantized back, one dispatch over every layer.
#pragma once
#include "abi/StateCodec.h"
#include "hip/Backend.hpp"

#include <cstdint>

namespace splash::ops {

// The element type of a running state's recurrent layers (the reference's GdnStateFormat, runtime/ops/GDN.hpp). The
// decode kernels of this library keep fp32 states; the codec also takes bf16 ones.
enum class GdnStateFormat : uint8_t { Float32, BFloat16 };
constexpr uint32_t elementBytes(GdnStateFormat f) noexcept { return f == GdnStateFormat::BFloat16 ? 2 : 4; }

// A layer holds `rows` value rows (every value head's) of `columns` values (a head's key dimensions); consecutive
// layers are stateLayerBytes apart in the running state and codesLayerBytes apart in the cached one.
struct StateCodecShape final {
  uint32_t layers = 0;
  uint32_t rows = 0;
  uint32_t columns = 0;
  uint64_t stateLayerBytes = 0;
  uint64_t codesLayerBytes = 0;
  GdnStateFormat format = GdnStateFormat::Float32;

  [[nodiscard]] constexpr uint64_t stateBytes() const noexcept { return uint64_t{rows} * columns * elementBytes(format); }
  [[nodiscard]] constexpr uint64_t codesBytes() const noexcept { return state_codec_layer_bytes(rows, columns); }
  [[nodiscard]] constexpr bool valid() const noexcept {
    return layers && rows && columns && columns % STATE_CODEC_BLOCK == 0 && stateLayerBytes >= stateBytes() &&
           codesLayerBytes >= codesBytes() && stateLayerBytes % 16 == 0 && codesLayerBytes % 4 == 0 &&
           uint64_t{rows} * columns / STATE_CODEC_LANE_VALUES <= UINT32_MAX;
  }
};

class StateCodec final {
public:
  // `state` and `codes` start at the first layer.
  static void addQuantize(hip::CommandGraph &graph, hip::Buffer state, hip::Buffer codes, StateCodecShape shape);
  static void addDequantize(hip::CommandGraph &graph, hip::Buffer codes, hip::Buffer state, StateCodecShape shape);
  // Each layer's state bytes from `from`, its layers stateLayerBytes apart, to `to`, codesLayerBytes apart, as they
  // are: a cached state that keeps the running format.
  static void addCopy(hip::CommandGraph &graph, hip::Buffer from, hip::Buffer to, StateCodecShape shape);
};

} // namespace splash::ops
