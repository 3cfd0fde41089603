#include "ops/StateCodec.hpp"

#include "ops/Linear.hpp"  // requireBytes

#include <stdexcept>
#include <string>

namespace splash::ops {
namespace {

constexpr uint32_t kThreads = 256;

// Each layer's values and codes, to the last layer's end (StateCodec.cpp:21-28 in the reference).
void requireExtents(const StateCodecShape &shape, const hip::Buffer &state, const hip::Buffer &codes) {
  if (!shape.valid()) throw std::invalid_argument("invalid state codec shape");
  requireBytes(state, uint64_t{shape.layers - 1} * shape.stateLayerBytes + shape.stateBytes(), "state codec state");
  requireBytes(codes, uint64_t{shape.layers - 1} * shape.codesLayerBytes + shape.codesBytes(), "state codec codes");
}

void add(hip::CommandGraph &graph, std::string name, hip::Buffer first, hip::Buffer second, const StateCodecShape &shape) {
  const StateCodecParams p{shape.stateLayerBytes, shape.codesLayerBytes, state_codec_scales_offset(shape.rows, shape.columns),
                           uint32_t(uint64_t{shape.rows} * shape.columns / STATE_CODEC_LANE_VALUES), 0};
  if (shape.format == GdnStateFormat::BFloat16) name += "_bf16_state";
  const uint32_t perGroup = kThreads * STATE_CODEC_THREAD_QUADS;
  graph.add(name, {std::move(first), std::move(second)}, p, {(p.quads_per_layer + perGroup - 1) / perGroup, shape.layers, 1},
            {kThreads, 1, 1});
}

} // namespace

void StateCodec::addQuantize(hip::CommandGraph &graph, hip::Buffer state, hip::Buffer codes, StateCodecShape shape) {
  requireExtents(shape, state, codes);
  add(graph, "state_quantize", std::move(state), std::move(codes), shape);
}

void StateCodec::addDequantize(hip::CommandGraph &graph, hip::Buffer codes, hip::Buffer state, StateCodecShape shape) {
  requireExtents(shape, state, codes);
  add(graph, "state_dequantize", std::move(codes), std::move(state), shape);
}

void StateCodec::addCopy(hip::CommandGraph &graph, hip::Buffer from, hip::Buffer to, StateCodecShape shape) {
  if (!shape.valid() || shape.codesLayerBytes < shape.stateBytes() || shape.codesLayerBytes % 16)
    throw std::invalid_argument("invalid state copy shape");
  requireBytes(from, uint64_t{shape.layers - 1} * shape.stateLayerBytes + shape.stateBytes(), "state copy source");
  requireBytes(to, uint64_t{shape.layers - 1} * shape.codesLayerBytes + shape.stateBytes(), "state copy destination");
  const StateCodecParams p{shape.stateLayerBytes, shape.codesLayerBytes, 0, uint32_t(shape.stateBytes() / 16), 0};
  graph.add("state_copy", {std::move(from), std::move(to)}, p, {(p.quads_per_layer + kThreads - 1) / kThreads, shape.layers, 1},
            {kThreads, 1, 1});
}

} // namespace splash::ops
