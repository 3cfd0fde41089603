#include "ops/StateCodec.hpp"

#include "ops/Linear.hpp"  // requireBytes

#include <stdexcept>
#include <string>

namespace splash::ops {
namespace {

constexpr uint32_t kBlockThreads = 256;

enum class Direction { Quantize, Dequantize };

// Bytes a buffer of `layers` layers must hold when layers are `stride` apart and the last one needs `last`.
uint64_t span(uint32_t layers, uint64_t stride, uint64_t last) { return uint64_t{layers - 1} * stride + last; }

void record(hip::CommandGraph &graph, Direction direction, const hip::Buffer &state, const hip::Buffer &codes,
            const StateCodecShape &shape) {
  if (!shape.valid()) throw std::invalid_argument("invalid state codec shape");
  requireBytes(state, span(shape.layers, shape.stateLayerBytes, shape.stateBytes()), "state codec state");
  requireBytes(codes, span(shape.layers, shape.codesLayerBytes, shape.codesBytes()), "state codec codes");
  StateCodecParams params{};
  params.state_layer_bytes = shape.stateLayerBytes;
  params.codes_layer_bytes = shape.codesLayerBytes;
  params.scales_offset = state_codec_scales_offset(shape.rows, shape.columns);
  params.quads_per_layer = uint32_t(shape.values() / STATE_CODEC_LANE_VALUES);
  const bool quantize = direction == Direction::Quantize;
  std::string kernel = quantize ? "state_quantize" : "state_dequantize";
  if (shape.format == GdnStateFormat::BFloat16) kernel += "_bf16_state";
  const uint32_t quadsPerGroup = kBlockThreads * STATE_CODEC_THREAD_QUADS;
  const uint32_t groups = (params.quads_per_layer + quadsPerGroup - 1) / quadsPerGroup;
  // The kernels take (source, destination).
  graph.add(kernel, {quantize ? state : codes, quantize ? codes : state}, params, {groups, shape.layers, 1}, {kBlockThreads, 1, 1});
}

} // namespace

void StateCodec::addQuantize(hip::CommandGraph &graph, hip::Buffer state, hip::Buffer codes, StateCodecShape shape) {
  record(graph, Direction::Quantize, state, codes, shape);
}

void StateCodec::addDequantize(hip::CommandGraph &graph, hip::Buffer codes, hip::Buffer state, StateCodecShape shape) {
  record(graph, Direction::Dequantize, state, codes, shape);
}

void StateCodec::addCopy(hip::CommandGraph &graph, hip::Buffer from, hip::Buffer to, StateCodecShape shape) {
  const uint64_t layerBytes = shape.stateBytes();
  if (!shape.valid() || shape.codesLayerBytes < layerBytes || shape.codesLayerBytes % 16)
    throw std::invalid_argument("invalid state copy shape");
  requireBytes(from, span(shape.layers, shape.stateLayerBytes, layerBytes), "state copy source");
  requireBytes(to, span(shape.layers, shape.codesLayerBytes, layerBytes), "state copy destination");
  StateCodecParams params{};
  params.state_layer_bytes = shape.stateLayerBytes;
  params.codes_layer_bytes = shape.codesLayerBytes;
  params.quads_per_layer = uint32_t(layerBytes / 16);  // 16-byte vectors here
  graph.add("state_copy", {from, to}, params, {(params.quads_per_layer + kBlockThreads - 1) / kBlockThreads, shape.layers, 1},
            {kBlockThreads, 1, 1});
}

} // namespace splash::ops
