#include "ops/DraftAttention.hpp"

#include "ops/Linear.hpp"  // requireBytes

#include <algorithm>
#include <stdexcept>

namespace splash::ops {
namespace {

constexpr uint32_t kRows = DRAFT_ATTENTION_QUERY_ROWS;
constexpr uint32_t kRopeRows = DRAFT_ATTENTION_ROPE_LANE_ROWS;
constexpr uint32_t kWindow = DRAFT_ATTENTION_WINDOW;
constexpr uint32_t kMaximumLanes = DRAFT_ATTENTION_MAXIMUM_LANES;
constexpr uint64_t kPartialBytes = uint64_t{DRAFT_ATTENTION_PARTIAL_FLOATS} * 4;

void requireLanes(uint32_t lanes) {
  if (!lanes || lanes > kMaximumLanes) throw std::invalid_argument("invalid draft batch width");
}
void requireCompiledShape(const DraftAttentionShape &shape) {
  if (!shape.hiddenSize || shape.hiddenSize % DRAFT_CONVOLUTION_GROUP || shape != DraftAttentionShape::of(shape.hiddenSize))
    throw std::invalid_argument("unsupported compiled draft attention shape");
}
uint64_t queryRowsBytes(const DraftAttentionPlan &plan) { return uint64_t{plan.lanes()} * kRows * DRAFT_ATTENTION_WIDTH * 2; }

// What the context writers read: the key and value rows up to `rows`, the key norm and the RoPE rows up to `ropeRows`.
void requireContextInputs(const hip::Buffer &contextKv, const hip::Buffer &keyNorm, const hip::Buffer &ropeCos,
                          const hip::Buffer &ropeSin, uint64_t rows, uint64_t ropeRows) {
  requireBytes(contextKv, rows * 2 * DRAFT_ATTENTION_KV_WIDTH * 2, "draft context K/V");
  requireBytes(keyNorm, uint64_t{DRAFT_ATTENTION_HEAD_DIMENSION} * 2, "draft key norm");
  requireBytes(ropeCos, ropeRows * DRAFT_ATTENTION_ROPE_PAIRS * 4, "draft RoPE cosine");
  requireBytes(ropeSin, ropeRows * DRAFT_ATTENTION_ROPE_PAIRS * 4, "draft RoPE sine");
}

// Lanes' rings inside the bound buffer, whole and 16-byte aligned (the kernels read 16-byte operands from them).
void requireRings(const DraftRings &rings, uint32_t lanes) {
  if (rings.keys.size() != lanes || rings.values.size() != lanes) throw std::invalid_argument("a draft step binds a key and a value ring a lane");
  const uint64_t size = rings.buffer ? rings.buffer.sizeBytes() : 0;
  for (uint32_t lane = 0; lane < lanes; ++lane)
    for (const uint64_t at : {rings.keys[lane], rings.values[lane]})
      if (at % 16 || at > size || size - at < draft_ring_bytes()) throw std::invalid_argument("a draft ring lies outside its buffer");
}

// The workgroups of a context window transfer, a wave a row and 64-value group, after checking its buffers.
hip::DispatchSize windowGroups(const hip::Buffer &context, const hip::Buffer &window, uint64_t contextRows, uint32_t rows, uint32_t width) {
  const uint64_t windowBytes = DraftAttention::contextWindowBytes(width);
  if (!rows || rows > kWindow) throw std::invalid_argument("a context window holds one ring's rows");
  requireBytes(context, contextRows * width * 2, "draft context rows");
  requireBytes(window, windowBytes, "draft context window");
  const uint64_t tasks = uint64_t{rows} * (width / DRAFT_CONTEXT_GROUP);
  return {(tasks + 3) / 4, 1, 1};
}

} // namespace

DraftAttentionWorkspace DraftAttentionPlan::workspace() const noexcept {
  const uint64_t rows = uint64_t{lanes_} * kRows;
  const uint64_t kvBytes = rows * shape_.kvHeads * shape_.headDimension * 2;
  const uint64_t partialBytes = uint64_t{lanes_} * shape_.kvHeads * DRAFT_ATTENTION_SPLITS * kPartialBytes;
  return {rows * shape_.hiddenSize * 2, rows * shape_.qkvSize * 2, rows * shape_.attentionSize * 2 + partialBytes, kvBytes, kvBytes};
}

DraftAttentionPlan DraftAttention::plan(DraftAttentionShape shape, uint32_t lanes) {
  requireLanes(lanes);
  requireCompiledShape(shape);
  return {shape, lanes};
}

void DraftAttention::addConvolution(hip::CommandGraph &graph, const DraftConvolutionBuffers &buffers, const DraftAttentionPlan &plan,
                                    DraftConvolutionStage stage) {
  const DraftAttentionShape shape = plan.shape();
  const DraftAttentionWorkspace workspace = plan.workspace();
  const uint32_t lanes = plan.lanes();
  const bool finish = stage == DraftConvolutionStage::Residual;
  requireBytes(buffers.input, workspace.convolutionBytes, "draft convolution input");
  requireBytes(buffers.output, workspace.convolutionBytes, "draft convolution output");
  if (finish) requireBytes(buffers.residual, workspace.convolutionBytes, "draft convolution residual");
  requireBytes(buffers.dynamic, uint64_t{lanes} * kRows * shape.dynamicSize * 2, "draft dynamic convolution");
  requireBytes(buffers.weights, uint64_t{DRAFT_CONVOLUTION_STAGES} * DRAFT_CONVOLUTION_TAPS * shape.hiddenSize * 2, "draft convolution weight");
  const uint64_t groups = (uint64_t{kRows} * shape.hiddenSize + 255) / 256;
  graph.add("draft_conv", {buffers.input, buffers.dynamic, buffers.weights, finish ? buffers.residual : buffers.input, buffers.output},
            DraftConvParams{finish ? 1u : 0u, shape.hiddenSize}, {groups, lanes, 1});
}

void DraftAttention::addPrepare(hip::CommandGraph &graph, const DraftPrepareBuffers &buffers, const DraftAttentionPlan &plan) {
  const DraftAttentionWorkspace workspace = plan.workspace();
  const uint32_t lanes = plan.lanes();
  requireBytes(buffers.qkv, workspace.qkvBytes, "draft q/k/v");
  requireBytes(buffers.groupedQueries, queryRowsBytes(plan), "draft grouped queries");
  requireBytes(buffers.queryKeys, workspace.queryKeysBytes, "draft query keys");
  requireBytes(buffers.queryValues, workspace.queryValuesBytes, "draft query values");
  requireBytes(buffers.queryNorm, uint64_t{DRAFT_ATTENTION_HEAD_DIMENSION} * 2, "draft query norm");
  requireBytes(buffers.keyNorm, uint64_t{DRAFT_ATTENTION_HEAD_DIMENSION} * 2, "draft key norm");
  const uint64_t ropeBytes = (uint64_t{lanes - 1} * kRopeRows + kRows) * DRAFT_ATTENTION_ROPE_PAIRS * 4;
  requireBytes(buffers.ropeCos, ropeBytes, "draft RoPE cosine");
  requireBytes(buffers.ropeSin, ropeBytes, "draft RoPE sine");
  constexpr uint32_t kTasks = kRows * (DRAFT_ATTENTION_QUERY_HEADS + DRAFT_ATTENTION_KV_HEADS);
  graph.add("draft_attention_qkv",
            {buffers.qkv, buffers.groupedQueries, buffers.queryNorm, buffers.keyNorm, buffers.ropeCos, buffers.ropeSin, buffers.queryKeys,
             buffers.queryValues},
            DraftLanesParams{lanes}, {kTasks / 8, lanes, 1}, {512, 1, 1});
}

void DraftAttention::addDecode(hip::CommandGraph &graph, const DraftDecodeAttentionBuffers &buffers, std::span<const uint32_t> cacheLengths,
                               const DraftAttentionPlan &plan) {
  const DraftAttentionWorkspace workspace = plan.workspace();
  const uint32_t lanes = plan.lanes();
  if (cacheLengths.size() != lanes) throw std::invalid_argument("invalid draft attention geometry");
  requireBytes(buffers.groupedQueries, workspace.groupedQueriesBytes, "draft grouped queries");
  requireBytes(buffers.queryKeys, workspace.queryKeysBytes, "draft query keys");
  requireBytes(buffers.queryValues, workspace.queryValuesBytes, "draft query values");
  requireRings(buffers.rings, lanes);
  DraftAttentionParams params{};
  params.lanes = lanes;
  for (uint32_t lane = 0; lane < lanes; ++lane) {
    if (cacheLengths[lane] > (1u << 20)) throw std::invalid_argument("draft attention cache length exceeds limit");
    params.cache_length[lane] = cacheLengths[lane];
    params.keys[lane] = buffers.rings.keys[lane];
    params.values[lane] = buffers.rings.values[lane];
  }
  const hip::Buffer partials = buffers.groupedQueries.slice(queryRowsBytes(plan), workspace.groupedQueriesBytes - queryRowsBytes(plan));
  graph.add("draft_attention_split", {buffers.groupedQueries, buffers.rings.buffer, buffers.queryKeys, buffers.queryValues, partials}, params,
            {DRAFT_ATTENTION_KV_HEADS, lanes, DRAFT_ATTENTION_SPLITS});
  graph.add("draft_attention_merge", {partials, buffers.groupedQueries}, DraftLanesParams{lanes}, {DRAFT_ATTENTION_KV_HEADS, lanes, 1},
            {1024, 1, 1});
}

void DraftAttention::addContextPrefill(hip::CommandGraph &graph, const hip::Buffer &contextKv, const hip::Buffer &keyNorm,
                                       const hip::Buffer &ropeCos, const hip::Buffer &ropeSin, const hip::Buffer &rings, uint64_t keys,
                                       uint64_t values, uint32_t tokens, uint32_t startPosition, DraftAttentionShape shape) {
  requireCompiledShape(shape);
  if (!tokens) throw std::invalid_argument("invalid draft context prefill geometry");
  requireContextInputs(contextKv, keyNorm, ropeCos, ropeSin, tokens, tokens);
  const uint64_t ringKeys[1] = {keys}, ringValues[1] = {values};
  requireRings({rings, ringKeys, ringValues}, 1);
  DraftContextParams params{};
  params.rows = tokens;
  params.start_position[0] = startPosition;
  params.keys[0] = keys;
  params.values[0] = values;
  // The commit's mask and lane rows are not read: the rows' buffer stands in their slots.
  graph.add("draft_context_kv", {contextKv, keyNorm, ropeCos, ropeSin, rings, contextKv, contextKv}, params,
            {uint64_t{tokens} * DRAFT_ATTENTION_KV_HEADS, 1, 1}, {64, 1, 1});
}

void DraftAttention::addContextCommit(hip::CommandGraph &graph, const hip::Buffer &contextKv, const hip::Buffer &keyNorm,
                                      const hip::Buffer &ropeCos, const hip::Buffer &ropeSin, const DraftRings &rings,
                                      const hip::Buffer &retainedRows, const hip::Buffer &laneRows,
                                      std::span<const uint32_t> startPositions, const StepRows &step, DraftAttentionShape shape) {
  const auto lanes = static_cast<uint32_t>(startPositions.size());
  requireLanes(lanes);
  requireCompiledShape(shape);
  if (step.lanes != lanes || !step.laneCap || step.laneCap > kRopeRows || step.rows < lanes || step.rows > lanes * kRopeRows)
    throw std::invalid_argument("invalid draft context commit geometry");
  // Each lane commits up to its rows of the step, at most a verify block's: its context rows among the step's, its
  // RoPE rows from its lane's first.
  requireContextInputs(contextKv, keyNorm, ropeCos, ropeSin, step.rows, uint64_t{lanes - 1} * kRopeRows + step.laneCap);
  requireBytes(retainedRows, uint64_t{lanes} * 4, "draft retained rows");
  requireBytes(laneRows, uint64_t{lanes} * sizeof(SamplingLaneRows), "draft lane rows");
  requireRings(rings, lanes);
  DraftContextParams params{};
  params.rows = step.laneCap;
  params.commit = 1;
  for (uint32_t lane = 0; lane < lanes; ++lane) {
    params.start_position[lane] = startPositions[lane];
    params.keys[lane] = rings.keys[lane];
    params.values[lane] = rings.values[lane];
  }
  graph.add("draft_context_kv", {contextKv, keyNorm, ropeCos, ropeSin, rings.buffer, retainedRows, laneRows}, params,
            {uint64_t{step.laneCap} * DRAFT_ATTENTION_KV_HEADS, lanes, 1}, {64, 1, 1});
}

uint64_t DraftAttention::contextWindowBytes(uint32_t width) {
  if (!width || width % DRAFT_CONTEXT_GROUP) throw std::invalid_argument("draft context rows are whole 64-value groups");
  return draft_context_window_bytes(width);
}

void DraftAttention::addWindowStore(hip::CommandGraph &graph, const hip::Buffer &context, const hip::Buffer &window, uint32_t rows,
                                    uint32_t startPosition, uint32_t width) {
  const hip::DispatchSize groups = windowGroups(context, window, rows, rows, width);
  graph.add("draft_context_store", {context, window, context, context}, DraftWindowParams{rows, startPosition, width, 0}, groups);
}

void DraftAttention::addWindowCommit(hip::CommandGraph &graph, const hip::Buffer &context, const hip::Buffer &window,
                                     const hip::Buffer &retained, const hip::Buffer &laneRows, uint32_t contextRows, uint32_t rows,
                                     uint32_t startPosition, uint32_t width) {
  if (!rows || rows > kRopeRows || rows > contextRows) throw std::invalid_argument("invalid draft context window commit");
  const hip::DispatchSize groups = windowGroups(context, window, contextRows, rows, width);
  requireBytes(retained, 4, "draft retained rows");
  requireBytes(laneRows, sizeof(SamplingLaneRows), "draft lane rows");
  graph.add("draft_context_store", {context, window, retained, laneRows}, DraftWindowParams{rows, startPosition, width, 1}, groups);
}

void DraftAttention::addWindowLoad(hip::CommandGraph &graph, const hip::Buffer &window, const hip::Buffer &context, uint32_t rows,
                                   uint32_t startPosition, uint32_t width) {
  const hip::DispatchSize groups = windowGroups(context, window, rows, rows, width);
  graph.add("draft_context_load", {window, context}, DraftWindowParams{rows, startPosition, width, 0}, groups);
}

void DraftAttention::addMaskRows(hip::CommandGraph &graph, const hip::Buffer &mask, const hip::Buffer &rows, uint32_t width, uint32_t lanes) {
  if (!width || !lanes || lanes > kMaximumLanes) throw std::invalid_argument("invalid draft mask rows");
  requireBytes(mask, uint64_t{width} * 2, "draft mask embedding");
  requireBytes(rows, uint64_t{lanes} * kRows * width * 2, "draft input row");
  graph.add("draft_mask_rows", {mask, rows}, DraftMaskRowsParams{width}, {(width + 255) / 256, kRows - 1, lanes});
}

} // namespace splash::ops
