#include "model/DFlashDraft.hpp"

#include "ops/Glue.hpp"

#include <stdexcept>
#include <string>

namespace splash::model {
namespace {

constexpr uint32_t kRows = DRAFT_ATTENTION_QUERY_ROWS;
constexpr uint64_t kRing = draft_ring_bytes();

void requireProjection(const ops::Projection &p, uint32_t output, uint32_t input, const char *what) {
  if (p.outputSize != output || p.inputSize != input)
    throw std::invalid_argument(std::string("draft ") + what + " projection is " + std::to_string(p.outputSize) + " x " +
                                std::to_string(p.inputSize) + ", not " + std::to_string(output) + " x " + std::to_string(input));
}

void requireWeights(const DFlashDraftWeights &w) {
  const DFlashDraftLayout &l = w.layout;
  if (!l.layers || !l.hiddenSize || !l.vocabularySize || !l.intermediateSize || !l.targetLayerCount || l.hiddenSize % DRAFT_CONTEXT_GROUP)
    throw std::invalid_argument("DFlash draft layout contains a zero dimension or a hidden size that is no whole number of 64-value groups");
  if (w.layers.size() != l.layers) throw std::invalid_argument("DFlash draft weights hold another number of layers than their layout");
  for (const DFlashDraftLayerWeights &layer : w.layers) {
    requireProjection(layer.attentionDynamic, l.dynamicSize(), l.hiddenSize, "attention-dynamic");
    requireProjection(layer.qkvProjection, DRAFT_ATTENTION_QKV_WIDTH, l.hiddenSize, "qkv");
    requireProjection(layer.outputProjection, l.hiddenSize, DRAFT_ATTENTION_WIDTH, "attention-output");
    requireProjection(layer.mlpDynamic, l.dynamicSize(), l.hiddenSize, "mlp-dynamic");
    requireProjection(layer.gateProjection, l.intermediateSize, l.hiddenSize, "mlp-gate");
    requireProjection(layer.upProjection, l.intermediateSize, l.hiddenSize, "mlp-up");
    requireProjection(layer.downProjection, l.hiddenSize, l.intermediateSize, "mlp-down");
    requireProjection(layer.contextKvProjection, l.contextKvSize(), l.hiddenSize, "context k/v");
  }
  requireProjection(w.contextProjection, l.hiddenSize, l.targetHiddenSize(), "context");
  requireProjection(w.selectorProjection, DRAFT_SELECTOR_RANK, l.hiddenSize, "selector");
}

ops::DraftRings ringsOf(const hip::Buffer &rings, std::span<const DFlashLaneState> lanes, uint32_t layer, std::array<uint64_t, 8> &keys,
                        std::array<uint64_t, 8> &values) {
  for (size_t lane = 0; lane < lanes.size(); ++lane) {
    keys[lane] = lanes[lane].rings + uint64_t{layer} * 2 * kRing;
    values[lane] = keys[lane] + kRing;
  }
  return {rings, std::span<const uint64_t>(keys.data(), lanes.size()), std::span<const uint64_t>(values.data(), lanes.size())};
}

} // namespace

ops::Projection projectionRowsFrom(const ops::Projection &projection, uint32_t first) {
  if (first >= projection.outputSize) throw std::invalid_argument("a row range of a projection starts inside it");
  return projection.rows({{first, projection.outputSize - first}});
}

DFlashDraft::DFlashDraft(const DFlashDraftWeights &weights, const ops::Linear &linear, const ops::Projection &head)
    : weights_(weights), linear_(linear), head_(head) {
  requireWeights(weights);
  if (!head.outputSize || head.outputSize > weights.layout.vocabularySize || head.inputSize != weights.layout.hiddenSize ||
      head.destination != ops::FloatOutput::Float32)
    throw std::invalid_argument("the draft shares the target's vocabulary head (or a view of its rows), fp32 logits over its hidden size");
}

ops::LinearScratchSize DFlashDraft::scratchSize(uint32_t rows) const {
  ops::LinearScratchSize size;
  const auto include = [&](const ops::Projection &p) { size.include(linear_.scratchSize({p.outputSize, p.inputSize}, rows)); };
  for (const DFlashDraftLayerWeights &layer : weights_.layers)
    for (const ops::Projection *p : {&layer.attentionDynamic, &layer.qkvProjection, &layer.outputProjection, &layer.mlpDynamic,
                                     &layer.gateProjection, &layer.upProjection, &layer.downProjection, &layer.contextKvProjection})
      include(*p);
  include(weights_.contextProjection);
  include(weights_.selectorProjection);
  include(head_);
  return size;
}

void DFlashDraft::addMaskRows(hip::CommandGraph &graph, const hip::Buffer &rows, uint32_t lanes) const {
  if (!weights_.maskEmbedding) return;
  ops::DraftAttention::addMaskRows(graph, weights_.maskEmbedding, rows, weights_.layout.hiddenSize, lanes);
}

void DFlashDraft::addDecode(hip::CommandGraph &graph, const DFlashDecodeBuffers &b, std::span<const DFlashLaneState> lanes,
                            std::span<const uint32_t> cacheLengths) const {
  const auto count = static_cast<uint32_t>(cacheLengths.size());
  if (!count || count > DRAFT_ATTENTION_MAXIMUM_LANES || lanes.size() != count) throw std::invalid_argument("invalid draft decode batch");
  const DFlashDraftLayout &layout = weights_.layout;
  const uint32_t rows = count * kRows, hidden = layout.hiddenSize;
  const ops::DraftAttentionPlan plan = ops::DraftAttention::plan(layout.attentionShape(), count);
  std::array<uint64_t, 8> keys{}, values{};

  for (uint32_t index = 0; index < layout.layers; ++index) {
    const DFlashDraftLayerWeights &w = weights_.layers[index];
    const hip::Buffer &current = b.hidden[index & 1], &next = b.hidden[(index & 1) ^ 1];
    // attention: norm -> dynamic weights -> convolution -> q|k|v -> attention -> output -> convolution with the residual
    ops::PreparedInput normalized = ops::Normalization::addRmsTable(graph, current, w.inputNorm, b.normalized, b.scratch, hidden, rows);
    ops::LinearBuffers dynamic;
    dynamic.input = b.normalized;
    dynamic.output = b.dynamic;
    dynamic.scratch = b.scratch;
    dynamic.prepared = normalized;
    linear_.add(graph, dynamic, w.attentionDynamic, linear_.plan(w.attentionDynamic, rows));
    ops::DraftAttention::addConvolution(graph, {b.normalized, b.dynamic, w.attentionConvolution, current, b.convolved}, plan,
                                        ops::DraftConvolutionStage::Prepare);
    linear_.addProjection(graph, b.convolved, w.qkvProjection, b.proposalQkv, rows, b.scratch);
    ops::DraftAttention::addPrepare(graph, {b.proposalQkv, b.attention, w.queryNorm, w.keyNorm, b.ropeCos, b.ropeSin, b.queryKeys, b.queryValues},
                                    plan);
    ops::DraftAttention::addDecode(graph, {b.attention, ringsOf(b.rings, lanes, index, keys, values), b.queryKeys, b.queryValues}, cacheLengths,
                                   plan);
    linear_.addProjection(graph, b.attention, w.outputProjection, b.projected, rows, b.scratch);
    ops::DraftAttention::addConvolution(graph, {b.projected, b.dynamic, w.attentionConvolution, current, b.residual}, plan,
                                        ops::DraftConvolutionStage::Residual);
    // MLP: norm -> dynamic weights -> convolution -> SwiGLU -> down -> convolution with the residual
    normalized = ops::Normalization::addRmsTable(graph, b.residual, w.postAttentionNorm, b.normalized, b.scratch, hidden, rows);
    dynamic.prepared = normalized;
    linear_.add(graph, dynamic, w.mlpDynamic, linear_.plan(w.mlpDynamic, rows));
    ops::DraftAttention::addConvolution(graph, {b.normalized, b.dynamic, w.mlpConvolution, b.residual, b.convolved}, plan,
                                        ops::DraftConvolutionStage::Prepare);
    ops::LinearBuffers pair;
    pair.input = b.convolved;
    pair.output = b.intermediate;
    pair.scratch = b.scratch;
    linear_.add(graph, pair, w.upProjection, linear_.plan(w.upProjection, rows, ops::LinearEpilogue::GateUp), &w.gateProjection);
    linear_.addProjection(graph, b.intermediate, w.downProjection, b.projected, rows, b.scratch);
    ops::DraftAttention::addConvolution(graph, {b.projected, b.dynamic, w.mlpConvolution, b.residual, next}, plan,
                                        ops::DraftConvolutionStage::Residual);
  }
  // The final norm feeds the shared vocabulary head and then the selector's projection, which reads the table the
  // head's plan left.
  ops::PreparedInput finalHidden =
      ops::Normalization::addRmsTable(graph, b.hidden[layout.layers & 1], weights_.finalNorm, b.finalHidden, b.scratch, hidden, rows);
  ops::LinearBuffers head;
  head.input = b.finalHidden;
  head.output = b.logits;
  head.scratch = b.scratch;
  head.prepared = finalHidden;
  const ops::PreparedInput afterHead = linear_.add(graph, head, head_, linear_.plan(head_, rows));
  ops::LinearBuffers selector;
  selector.input = b.finalHidden;
  selector.output = b.selectorHidden;
  selector.scratch = b.scratch;
  selector.prepared = afterHead;
  linear_.add(graph, selector, weights_.selectorProjection, linear_.plan(weights_.selectorProjection, rows));
}

void DFlashDraft::addContextKv(hip::CommandGraph &graph, const DFlashContextBuffers &b, const DFlashLaneState &lane, uint32_t rows,
                               uint32_t startPosition) const {
  const DFlashDraftLayout &layout = weights_.layout;
  for (uint32_t index = 0; index < layout.layers; ++index) {
    linear_.addProjection(graph, b.hidden, weights_.layers[index].contextKvProjection, b.contextKv, rows, b.scratch);
    const uint64_t keys = lane.rings + uint64_t{index} * 2 * kRing;
    ops::DraftAttention::addContextPrefill(graph, b.contextKv, weights_.layers[index].keyNorm, b.ropeCos, b.ropeSin, b.rings, keys, keys + kRing,
                                           rows, startPosition, layout.attentionShape());
  }
}

void DFlashDraft::addContextPrefill(hip::CommandGraph &graph, const DFlashContextBuffers &b, const DFlashLaneState &lane, uint32_t rows,
                                    uint32_t startPosition) const {
  if (!rows || rows > ops::kMaximumDispatchRows) throw std::invalid_argument("invalid draft context prefill");
  const DFlashDraftLayout &layout = weights_.layout;
  linear_.addProjection(graph, b.capturedTargetHidden, weights_.contextProjection, b.projected, rows, b.scratch);
  ops::Normalization::addRms(graph, b.projected, weights_.hiddenNorm, b.hidden, layout.hiddenSize, rows);
  ops::DraftAttention::addWindowStore(graph, b.hidden, b.windows.slice(lane.window, layout.windowBytes()), rows, startPosition,
                                      layout.hiddenSize);
  addContextKv(graph, b, lane, rows, startPosition);
}

void DFlashDraft::addContextRebuild(hip::CommandGraph &graph, const DFlashContextBuffers &b, const DFlashLaneState &lane, uint32_t rows,
                                    uint32_t startPosition) const {
  if (!rows || rows > ops::kMaximumDispatchRows) throw std::invalid_argument("invalid draft context rebuild");
  const DFlashDraftLayout &layout = weights_.layout;
  ops::DraftAttention::addWindowLoad(graph, b.windows.slice(lane.window, layout.windowBytes()), b.hidden, rows, startPosition,
                                     layout.hiddenSize);
  addContextKv(graph, b, lane, rows, startPosition);
}

void DFlashDraft::addContextCommit(hip::CommandGraph &graph, const DFlashContextBuffers &b, std::span<const DFlashLaneState> lanes,
                                   const hip::Buffer &retainedRows, const hip::Buffer &laneRows, std::span<const uint32_t> startPositions,
                                   const ops::StepRows &step) const {
  const auto count = static_cast<uint32_t>(startPositions.size());
  if (!count || count > DRAFT_ATTENTION_MAXIMUM_LANES || step.lanes != count || lanes.size() != count)
    throw std::invalid_argument("invalid draft context batch");
  const DFlashDraftLayout &layout = weights_.layout;
  const uint32_t rows = step.rows;
  // The context projections run over the step's rows; every layer's key and value projection reads the same
  // normalized rows.
  linear_.addProjection(graph, b.capturedTargetHidden, weights_.contextProjection, b.projected, rows, b.scratch);
  ops::PreparedInput hidden = ops::Normalization::addRmsTable(graph, b.projected, weights_.hiddenNorm, b.hidden, b.scratch, layout.hiddenSize, rows);
  for (uint32_t lane = 0; lane < count; ++lane)
    ops::DraftAttention::addWindowCommit(graph, b.hidden, b.windows.slice(lanes[lane].window, layout.windowBytes()),
                                         retainedRows.slice(uint64_t{lane} * 4, 4), laneRows.slice(uint64_t{lane} * 8, 8), rows,
                                         std::min(step.laneCap, rows), startPositions[lane], layout.hiddenSize);
  std::array<uint64_t, 8> keys{}, values{};
  for (uint32_t index = 0; index < layout.layers; ++index) {
    const ops::Projection &projection = weights_.layers[index].contextKvProjection;
    ops::LinearBuffers kv;
    kv.input = b.hidden;
    kv.output = b.contextKv;
    kv.scratch = b.scratch;
    kv.prepared = hidden;
    hidden = linear_.add(graph, kv, projection, linear_.plan(projection, rows));
    ops::DraftAttention::addContextCommit(graph, b.contextKv, weights_.layers[index].keyNorm, b.ropeCos, b.ropeSin,
                                          ringsOf(b.rings, lanes, index, keys, values), retainedRows, laneRows, startPositions, step,
                                          layout.attentionShape());
  }
}

} // namespace splash::model
