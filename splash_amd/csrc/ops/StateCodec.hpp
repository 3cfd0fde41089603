// ops::StateCodec for MI355X: the int8 form in which a lane's Gated DeltaNet recurrent layers are kept when a state is
// cached. Interface after the reference's operator of the same name (runtime/ops/StateCodec.hpp:11-49); the layout of
// a coded layer is abi/StateCodec.h's. Every call records one dispatch that covers all layers of the shape.
#pragma once
#include "abi/StateCodec.h"
#include "hip/Backend.hpp"

#include <cstdint>

namespace splash::ops {

// Element type of the running state (GdnStateFormat in the reference's runtime/ops/GDN.hpp). This library's decode
// kernels write fp32 states; bf16 ones are accepted by the codec for states produced elsewhere.
enum class GdnStateFormat : uint8_t { Float32, BFloat16 };
constexpr uint32_t elementBytes(GdnStateFormat f) noexcept { return f == GdnStateFormat::BFloat16 ? 2 : 4; }

struct StateCodecShape final {
  uint32_t layers = 0;            // recurrent layers coded by one dispatch
  uint32_t rows = 0;              // value rows of a layer, all value heads together
  uint32_t columns = 0;           // values of a row: a head's key dimensions, whole blocks of 32
  uint64_t stateLayerBytes = 0;   // stride between layers in the running state (a multiple of 16)
  uint64_t codesLayerBytes = 0;   // stride between layers in the cached state (a multiple of 4)
  GdnStateFormat format = GdnStateFormat::Float32;

  [[nodiscard]] constexpr uint64_t values() const noexcept { return uint64_t{rows} * columns; }
  [[nodiscard]] constexpr uint64_t stateBytes() const noexcept { return values() * elementBytes(format); }
  [[nodiscard]] constexpr uint64_t codesBytes() const noexcept { return state_codec_layer_bytes(rows, columns); }
  [[nodiscard]] constexpr bool valid() const noexcept {
    const bool geometry = layers != 0 && rows != 0 && columns != 0 && columns % STATE_CODEC_BLOCK == 0;
    const bool strides = stateLayerBytes >= stateBytes() && codesLayerBytes >= codesBytes() && stateLayerBytes % 16 == 0 &&
                         codesLayerBytes % 4 == 0;
    return geometry && strides && values() / STATE_CODEC_LANE_VALUES <= UINT32_MAX;
  }
};

class StateCodec final {
public:
  // running state -> codes and scales; both buffers begin at layer 0.
  static void addQuantize(hip::CommandGraph &graph, hip::Buffer state, hip::Buffer codes, StateCodecShape shape);
  // codes and scales -> running state.
  static void addDequantize(hip::CommandGraph &graph, hip::Buffer codes, hip::Buffer state, StateCodecShape shape);
  // For a cache that keeps states uncoded: stateBytes() of every layer move unchanged from a buffer strided by
  // stateLayerBytes to one strided by codesLayerBytes (which must then be a multiple of 16 and hold a layer's state).
  static void addCopy(hip::CommandGraph &graph, hip::Buffer from, hip::Buffer to, StateCodecShape shape);
};

} // namespace splash::ops
