// C shim of ops::GDN (include/splash_ops.h).
#include "capi/Guard.hpp"
#include "capi/Handles.hpp"
#include "ops/Gdn.hpp"
#include "ops/StateCodec.hpp"
#include "splash_ops.h"

using namespace splash;

namespace {
hip::Buffer B(sp_buffer *b) { return hip::Buffer::share(b); }
ops::GdnShape shapeOf(const spo_gdn_shape &s) {
  ops::GdnShape shape;
  shape.keyHeads = s.key_heads;
  shape.valueHeads = s.value_heads;
  shape.convolutionDimension = s.convolution_dimension;
  shape.packedWidth = s.packed_width;
  shape.sigmoidGate = s.sigmoid_gate != 0;
  return shape;
}
ops::GdnStateStrides stridesOf(const spo_gdn_state_strides &s) {
  return {s.convolution_layer_bytes, s.recurrent_layer_bytes, s.convolution_state_bytes};
}
} // namespace

extern "C" {

sp_status spo_gdn_layout(const spo_gdn_shape *shape, uint32_t layers, spo_gdn_state_strides *strides, uint64_t *cell_bytes,
                         uint64_t *tape_layer_bytes) {
  return capi::guard([&] {
    capi::require(shape, "shape");
    const ops::GdnShape s = shapeOf(*shape);
    if (!s.valid() || !layers) throw std::invalid_argument("invalid GDN shape");
    const ops::GdnStateStrides st = ops::GdnStateStrides::of(s, layers);
    if (strides) *strides = {st.convolutionLayerBytes, st.recurrentLayerBytes, st.convolutionStateBytes};
    if (cell_bytes) *cell_bytes = st.cellBytes(layers);
    if (tape_layer_bytes) *tape_layer_bytes = ops::gdnTapeLayerBytes(s);
  });
}

sp_status spo_gdn_add_decode(spo_graph *graph, const spo_gdn_decode_buffers *b, const spo_gdn_shape *shape, uint32_t layer,
                             const spo_gdn_state_strides *state, uint32_t tiled_heads, const spo_gdn_lane *lanes, uint32_t count) {
  return capi::guard([&] {
    capi::require(graph && b && shape && state && lanes, "graph, buffers, shape, strides or lanes");
    ops::GdnDecodeBuffers buffers{B(b->packed), B(b->convolution_weights), B(b->states), B(b->tape), B(b->decay_weights),
                                  B(b->time_bias), B(b->mixer_norm), b->float_norm != 0, B(b->hidden), B(b->tree_rows),
                                  b->hidden_table ? B(b->hidden_table) : hip::Buffer{}};
    std::vector<ops::GdnLaneStep> list;
    for (uint32_t i = 0; i < count; ++i)
      list.push_back({lanes[i].first_row, lanes[i].rows, lanes[i].pending_path, lanes[i].pending_tape, lanes[i].step_tape,
                      lanes[i].current_cell, lanes[i].next_cell});
    ops::GDN::addDecode(capi::graphOf(graph), buffers, shapeOf(*shape), layer, stridesOf(*state),
                        tiled_heads ? ops::GdnHeadOrder::Tiled : ops::GdnHeadOrder::Grouped, list);
  });
}

sp_status spo_gdn_add_fold(spo_graph *graph, sp_buffer *states, sp_buffer *tape, sp_buffer *retained_rows, uint64_t step_tape,
                           uint64_t state_cell, uint64_t fold_cell, const spo_gdn_shape *shape, uint32_t layers, uint32_t rows,
                           const spo_gdn_state_strides *state) {
  return capi::guard([&] {
    capi::require(graph && shape && state, "graph, shape or strides");
    ops::GdnFoldBuffers buffers{B(states), B(tape), B(retained_rows), step_tape, state_cell, fold_cell};
    ops::GDN::addFold(capi::graphOf(graph), buffers, shapeOf(*shape), layers, rows, stridesOf(*state));
  });
}

sp_status spo_gdn_add_prefill(spo_graph *graph, const spo_gdn_prefill_buffers *b, const spo_gdn_shape *shape, uint32_t layer,
                              uint32_t tokens, const spo_gdn_state_strides *state, uint32_t tiled_heads,
                              const spo_gdn_prefill_capture *captures, uint32_t count) {
  return capi::guard([&] {
    capi::require(graph && b && shape && state && (captures || !count), "graph, buffers, shape, strides or captures");
    ops::GdnPrefillBuffers buffers{B(b->packed), B(b->convolution_weights), B(b->states), B(b->decay_weights), B(b->time_bias),
                                   B(b->mixer_norm), b->float_norm != 0, B(b->queries), B(b->keys), B(b->values), B(b->decay),
                                   B(b->beta), B(b->recurrent_rows), B(b->hidden), b->current_cell, b->next_cell};
    std::vector<ops::GdnPrefillCapture> list;
    for (uint32_t i = 0; i < count; ++i) list.push_back({captures[i].tokens, captures[i].cell});
    ops::GDN::addPrefill(capi::graphOf(graph), buffers, shapeOf(*shape), layer, tokens, stridesOf(*state),
                         tiled_heads ? ops::GdnHeadOrder::Tiled : ops::GdnHeadOrder::Grouped, list);
  });
}

uint64_t spo_state_codec_layer_bytes(uint32_t rows, uint32_t columns) { return state_codec_layer_bytes(rows, columns); }

extern "C++" {
namespace {
ops::StateCodecShape codecShapeOf(const spo_state_codec_shape &s) {
  return {s.layers, s.rows, s.columns, s.state_layer_bytes, s.codes_layer_bytes,
          s.bf16_state ? ops::GdnStateFormat::BFloat16 : ops::GdnStateFormat::Float32};
}
} // namespace
} // extern "C++"

sp_status spo_state_codec_add_quantize(spo_graph *graph, sp_buffer *state, sp_buffer *codes, const spo_state_codec_shape *shape) {
  return capi::guard([&] {
    capi::require(graph && shape, "graph or shape");
    ops::StateCodec::addQuantize(capi::graphOf(graph), B(state), B(codes), codecShapeOf(*shape));
  });
}
sp_status spo_state_codec_add_dequantize(spo_graph *graph, sp_buffer *codes, sp_buffer *state, const spo_state_codec_shape *shape) {
  return capi::guard([&] {
    capi::require(graph && shape, "graph or shape");
    ops::StateCodec::addDequantize(capi::graphOf(graph), B(codes), B(state), codecShapeOf(*shape));
  });
}
sp_status spo_state_codec_add_copy(spo_graph *graph, sp_buffer *from, sp_buffer *to, const spo_state_codec_shape *shape) {
  return capi::guard([&] {
    capi::require(graph && shape, "graph or shape");
    ops::StateCodec::addCopy(capi::graphOf(graph), B(from), B(to), codecShapeOf(*shape));
  });
}
} // extern "C"
