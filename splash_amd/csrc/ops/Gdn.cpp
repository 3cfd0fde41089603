#include "ops/Gdn.hpp"
#include "abi/Gguf.h"
#include "abi/PagedAttention.h"  // AttentionTreeRow
#include "ops/Linear.hpp"  // requireBytes

#include <algorithm>
#include <stdexcept>

namespace splash::ops {

GdnStateStrides GdnStateStrides::of(const GdnShape &shape, uint32_t layers) noexcept {
  GdnStateStrides s;
  s.convolutionLayerBytes = uint64_t{GDN_CONVOLUTION_TAPS - 1} * shape.convolutionDimension * 2;
  s.recurrentLayerBytes = uint64_t{shape.valueHeads} * GDN_HEAD_DIMENSION * GDN_HEAD_DIMENSION * 4;
  s.convolutionStateBytes = (s.convolutionLayerBytes * layers + 255) / 256 * 256;
  return s;
}

uint64_t gdnTapeLayerBytes(const GdnShape &shape) noexcept {
  return gdn_tape_layer_bytes(shape.convolutionDimension, shape.kvWidth(), shape.valueHeads);
}

void GDN::addDecode(hip::CommandGraph &graph, const GdnDecodeBuffers &b, const GdnShape &shape, uint32_t layer,
                    const GdnStateStrides &state, GdnHeadOrder order, const std::vector<GdnLaneStep> &lanes) {
  if (!shape.valid()) throw std::invalid_argument("invalid GDN shape");
  if (!state.valid()) throw std::invalid_argument("invalid GDN state strides");
  if (lanes.empty() || lanes.size() > GDN_MAXIMUM_LANES) throw std::invalid_argument("a GDN step takes 1 to 8 lanes");
  const uint64_t tapeBytes = gdnTapeLayerBytes(shape);
  const uint64_t cellNeed = state.convolutionStateBytes + uint64_t{layer + 1} * state.recurrentLayerBytes;
  if (uint64_t{layer + 1} * state.convolutionLayerBytes > state.convolutionStateBytes)
    throw std::invalid_argument("the layer's convolution rows lie past the cell's convolution part");
  uint32_t rows = 0;
  GdnDecodeParams params{};
  params.shape = shape.params();
  params.flags = (order == GdnHeadOrder::Tiled ? GDN_TILED_HEADS : 0u) | (shape.sigmoidGate ? GDN_SIGMOID_GATE : 0u) |
                 (b.floatNorm ? GDN_FLOAT_NORM : 0u);
  params.layer = layer;
  params.lanes = uint32_t(lanes.size());
  params.conv_layer_bytes = state.convolutionLayerBytes;
  params.recurrent_layer_bytes = state.recurrentLayerBytes;
  params.convolution_state_bytes = state.convolutionStateBytes;
  for (size_t i = 0; i < lanes.size(); ++i) {
    const GdnLaneStep &l = lanes[i];
    if (!l.rows || l.rows > GDN_MAXIMUM_ROWS) throw std::invalid_argument("a lane's block holds 1 to 16 rows");
    if (l.firstRow < rows) throw std::invalid_argument("the lanes' blocks ascend and do not overlap");
    rows = l.firstRow + l.rows;
    if (l.pendingPath >> GDN_MAXIMUM_ROWS) throw std::invalid_argument("a pending path names rows of a 16-row block");
    if (l.stepTape % 16 || l.pendingTape % 16) throw std::invalid_argument("tape slots are 16-byte aligned");
    if (l.stepTape + tapeBytes > b.tape.sizeBytes() || (l.pendingPath && l.pendingTape + tapeBytes > b.tape.sizeBytes()))
      throw std::invalid_argument("a tape slot lies past the tape buffer");
    if (l.pendingPath && l.pendingTape < l.stepTape + tapeBytes && l.stepTape < l.pendingTape + tapeBytes)
      throw std::invalid_argument("a lane's pending and step tapes overlap");
    if (l.currentCell % 16 || l.nextCell % 16) throw std::invalid_argument("state cells are 16-byte aligned");
    if (l.currentCell + cellNeed > b.states.sizeBytes() || l.nextCell + cellNeed > b.states.sizeBytes())
      throw std::invalid_argument("a state cell lies past the states buffer");
    if (l.currentCell == l.nextCell) throw std::invalid_argument("a step reads and writes different cells");
    params.lane[i] = {l.firstRow, l.rows, l.pendingPath, 0, l.pendingTape, l.stepTape, l.currentCell, l.nextCell};
  }
  requireBytes(b.packed, uint64_t{rows} * shape.packedWidth * 2, "GDN packed rows");
  requireBytes(b.convolutionWeights, uint64_t{shape.convolutionDimension} * GDN_CONVOLUTION_TAPS * 2, "GDN convolution weights");
  requireBytes(b.decayWeights, uint64_t{shape.valueHeads} * 4, "GDN decay weights");
  requireBytes(b.timeBias, uint64_t{shape.valueHeads} * 2, "GDN time bias");
  requireBytes(b.mixerNorm, uint64_t{GDN_HEAD_DIMENSION} * (b.floatNorm ? 4 : 2), "GDN output norm");
  requireBytes(b.hidden, uint64_t{rows} * shape.valueHeads * GDN_HEAD_DIMENSION * 2, "GDN hidden rows");
  requireBytes(b.tree, uint64_t{rows} * sizeof(AttentionTreeRow), "GDN tree rows");
  if (b.hiddenTable) {
    requireBytes(b.hiddenTable, gguf_tables_bytes(shape.valueHeads * GDN_HEAD_DIMENSION, gguf_row_tiles(rows)), "GDN hidden table");
    params.table_tiles = gguf_row_tiles(rows);
  }
  graph.add("gdn_decode",
            {b.packed, b.convolutionWeights, b.states, b.tape, b.decayWeights, b.timeBias, b.mixerNorm, b.hidden, b.tree,
             b.hiddenTable ? b.hiddenTable : b.hidden},
            params,
            {shape.valueHeads, uint32_t(lanes.size()), 1}, {1024, 1, 1});
}

void GDN::addPrefill(hip::CommandGraph &graph, const GdnPrefillBuffers &b, const GdnShape &shape, uint32_t layer, uint32_t tokens,
                     const GdnStateStrides &state, GdnHeadOrder order, const std::vector<GdnPrefillCapture> &captures) {
  if (!shape.valid()) throw std::invalid_argument("invalid GDN shape");
  if (!state.valid()) throw std::invalid_argument("invalid GDN state strides");
  if (!tokens) throw std::invalid_argument("a GDN prompt chunk holds at least one row");
  if (uint64_t{layer + 1} * state.convolutionLayerBytes > state.convolutionStateBytes)
    throw std::invalid_argument("the layer's convolution rows lie past the cell's convolution part");
  const uint64_t cellNeed = state.convolutionStateBytes + uint64_t{layer + 1} * state.recurrentLayerBytes;
  auto requireCell = [&](uint64_t cell) {
    if (cell % 16 || cell + cellNeed > b.states.sizeBytes()) throw std::invalid_argument("a state cell lies past the states buffer or is unaligned");
  };
  requireCell(b.currentCell);
  requireCell(b.nextCell);
  uint32_t previous = 0;
  for (const GdnPrefillCapture &capture : captures) {
    if (capture.tokens <= previous || capture.tokens >= tokens)
      throw std::invalid_argument("GDN prefill captures ascend inside the chunk's rows");
    previous = capture.tokens;
    requireCell(capture.cell);
  }
  const uint64_t keyWidth = uint64_t{shape.keyHeads} * GDN_HEAD_DIMENSION, valueWidth = uint64_t{shape.valueHeads} * GDN_HEAD_DIMENSION;
  requireBytes(b.packed, uint64_t{tokens} * shape.packedWidth * 2, "GDN packed rows");
  requireBytes(b.convolutionWeights, uint64_t{shape.convolutionDimension} * GDN_CONVOLUTION_TAPS * 2, "GDN convolution weights");
  requireBytes(b.decayWeights, uint64_t{shape.valueHeads} * 4, "GDN decay weights");
  requireBytes(b.timeBias, uint64_t{shape.valueHeads} * 2, "GDN time bias");
  requireBytes(b.mixerNorm, uint64_t{GDN_HEAD_DIMENSION} * (b.floatNorm ? 4 : 2), "GDN output norm");
  requireBytes(b.queries, tokens * keyWidth * 2, "GDN query rows");
  requireBytes(b.keys, tokens * keyWidth * 2, "GDN key rows");
  requireBytes(b.values, tokens * valueWidth * 2, "GDN value rows");
  requireBytes(b.decay, uint64_t{tokens} * shape.valueHeads * 4, "GDN decay rows");
  requireBytes(b.beta, uint64_t{tokens} * shape.valueHeads * 2, "GDN beta rows");
  requireBytes(b.recurrentRows, tokens * valueWidth * 2, "GDN recurrent rows");
  requireBytes(b.hidden, tokens * valueWidth * 2, "GDN hidden rows");
  GdnPrefillParams params{};
  params.shape = shape.params();
  params.flags = (order == GdnHeadOrder::Tiled ? GDN_TILED_HEADS : 0u) | (shape.sigmoidGate ? GDN_SIGMOID_GATE : 0u) |
                 (b.floatNorm ? GDN_FLOAT_NORM : 0u);
  params.layer = layer;
  params.conv_layer_bytes = state.convolutionLayerBytes;
  params.recurrent_layer_bytes = state.recurrentLayerBytes;
  params.convolution_state_bytes = state.convolutionStateBytes;
  uint32_t begin = 0;
  uint64_t cell = b.currentCell;
  for (size_t run = 0; run <= captures.size(); ++run) {
    const bool last = run == captures.size();
    const uint32_t end = last ? tokens : captures[run].tokens;
    const uint64_t out = last ? b.nextCell : captures[run].cell;
    // a run's workgroups read rows of the cell it starts from that others of them write in the cell it leaves
    if (out == cell) throw std::invalid_argument("a GDN prefill run reads and writes different cells");
    params.first = begin;
    params.tokens = end - begin;
    params.current_cell = cell;
    params.next_cell = out;
    graph.add("gdn_prefill_prepare",
              {b.packed, b.convolutionWeights, b.states, b.decayWeights, b.timeBias, b.queries, b.keys, b.values, b.decay, b.beta}, params,
              {shape.valueHeads, (params.tokens + 3) / 4, 1}, {256, 1, 1});
    graph.add("gdn_prefill_scan", {b.queries, b.keys, b.values, b.decay, b.beta, b.states, b.recurrentRows}, params,
              {shape.valueHeads * (GDN_HEAD_DIMENSION / GDN_SCAN_STATE_ROWS), 1, 1}, {256, 1, 1});
    begin = end;
    cell = out;
  }
  params.first = 0;
  params.tokens = tokens;
  graph.add("gdn_prefill_gate", {b.recurrentRows, b.packed, b.mixerNorm, b.hidden}, params, {shape.valueHeads, (tokens + 3) / 4, 1},
            {256, 1, 1});
}

void GDN::addFold(hip::CommandGraph &graph, const GdnFoldBuffers &b, const GdnShape &shape, uint32_t layers, uint32_t rows,
                  const GdnStateStrides &state) {
  if (!shape.valid()) throw std::invalid_argument("invalid GDN shape");
  if (!state.valid() || !layers) throw std::invalid_argument("invalid GDN state strides");
  if (!rows || rows > GDN_MAXIMUM_ROWS) throw std::invalid_argument("a fold takes 1 to 16 rows");
  const uint64_t tapeBytes = gdnTapeLayerBytes(shape), cell = state.cellBytes(layers);
  if (b.stepTape % 16 || b.stepTape + tapeBytes * layers > b.tape.sizeBytes()) throw std::invalid_argument("the step's tapes lie past the tape buffer");
  if (b.stateCell % 16 || b.foldCell % 16 || b.stateCell + cell > b.states.sizeBytes() || b.foldCell + cell > b.states.sizeBytes())
    throw std::invalid_argument("a state cell lies past the states buffer");
  if (b.stateCell == b.foldCell) throw std::invalid_argument("a fold reads and writes different cells");
  requireBytes(b.retainedRows, 4, "retained rows");
  GdnFoldParams params{};
  params.shape = shape.params();
  params.rows = rows;
  params.conv_layer_bytes = state.convolutionLayerBytes;
  params.recurrent_layer_bytes = state.recurrentLayerBytes;
  params.convolution_state_bytes = state.convolutionStateBytes;
  params.step_tape = b.stepTape;
  params.tape_layer_bytes = tapeBytes;
  params.state_cell = b.stateCell;
  params.fold_cell = b.foldCell;
  graph.add("gdn_fold", {b.states, b.tape, b.retainedRows}, params, {shape.valueHeads, layers, 1}, {1024, 1, 1});
}

} // namespace splash::ops
