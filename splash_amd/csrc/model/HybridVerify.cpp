#include "model/HybridVerify.hpp"

#include <algorithm>
#include <cmath>
#include <stdexcept>

namespace splash::model {

using hip::BufferStorage;

namespace {
// Rows one projection dispatch takes: a longer step runs its dense projections in pieces.
constexpr uint32_t kProjectionRows = ops::kMaximumDispatchRows;
template <class F> void forRowPieces(uint32_t rows, F &&piece) {
  for (uint32_t first = 0; first < rows; first += kProjectionRows) piece(first, std::min(kProjectionRows, rows - first));
}
} // namespace

HybridVerify::HybridVerify(hip::Backend &backend, HybridDimensions d, uint32_t maxLanes, uint32_t physicalPages,
                           uint32_t pageTableEntries, uint32_t prefillRows)
    : backend_(backend), dims_(d), linear_(backend.deviceInfo()), maxLanes_(maxLanes),
      lanePolicies_(backend, maxLanes, d.vocabulary) {
  if (prefillRows > ops::kMaximumChunkRows) throw std::invalid_argument("a prompt chunk holds at most 2048 rows");
  if (!d.hidden || !d.layers || !d.vocabulary || !maxLanes || maxLanes > GDN_MAXIMUM_LANES)
    throw std::invalid_argument("a hybrid verify step takes a model and 1 to 8 lanes");
  if (!d.attentionInterval || d.layers % d.attentionInterval)
    throw std::invalid_argument("the layers hold whole groups of recurrent layers and one attention layer");
  if (d.hidden % GGUF_BLOCK || d.attentionWidth() % GGUF_BLOCK || d.gdnWidth() % GGUF_BLOCK || d.vocabulary % GGUF_TILE_COLUMNS ||
      d.gdnPackedWidth % GGUF_TILE_COLUMNS || d.experts % GGUF_TILE_COLUMNS)
    throw std::invalid_argument("the model's widths hold whole super-blocks and its projections whole column tiles");
  if (!d.gdnShape().valid()) throw std::invalid_argument("invalid GDN shape");
  if (d.dense() ? (!d.denseFfn || d.denseFfn % GGUF_BLOCK) : !d.moeShape().valid())
    throw std::invalid_argument(d.dense() ? "a dense FFN holds whole super-blocks" : "invalid MoE shape");
  maxRows_ = maxLanes * ATTENTION_MAXIMUM_ROWS;
  rowCapacity_ = std::max(maxRows_, prefillRows);
  // the most rows of one window of a chunk's projections and experts, or of a step
  const uint32_t windowRows = std::min(rowCapacity_, std::max(maxRows_, kProjectionRows));
  weights_.layers.resize(d.layers);
  const ops::kv::Layout layout{d.kvHeads, d.headDimension};
  pageBytes_ = layout.bytesPerLayerPage();
  auto device = [&](uint64_t bytes, const char *label) { return backend.allocateBuffer(std::max<uint64_t>(bytes, 16), BufferStorage::Private, label); };
  auto shared = [&](uint64_t bytes, const char *label) { return backend.allocateBuffer(std::max<uint64_t>(bytes, 16), BufferStorage::Shared, label); };
  const uint64_t R = maxRows_, C = rowCapacity_;
  hidden_[0] = device(C * d.hidden * 2, "hidden 0");
  hidden_[1] = device(C * d.hidden * 2, "hidden 1");
  normalized_ = device(C * d.hidden * 2, "normalized");
  packed_ = device(C * std::max(d.qkvWidth(), d.gdnPackedWidth) * 2, "mixer input rows");
  mixed_ = device(C * std::max(d.attentionWidth(), d.gdnWidth()) * 2, "mixer output rows");
  scores_ = device(uint64_t{windowRows} * d.experts * 4, "router scores");
  logits_ = device(R * d.vocabulary * 4, "logits");
  ropeCos_ = device(C * std::max(1u, d.rotaryPairs) * 4, "rope cos");
  ropeSin_ = device(C * std::max(1u, d.rotaryPairs) * 4, "rope sin");
  inverseFrequency_ = device(std::max(1u, d.rotaryPairs) * 4, "rope inverse frequency");
  if (d.rotaryPairs) {
    std::vector<float> inv(d.rotaryPairs);
    for (uint32_t i = 0; i < d.rotaryPairs; ++i) inv[i] = float(std::pow(double(d.ropeTheta), -double(i) / d.rotaryPairs));
    inverseFrequency_.upload(inv.data(), inv.size() * 4);
  }
  inputTokens_ = shared(C * 4, "input tokens");
  treeRows_ = shared(C * sizeof(AttentionTreeRow), "tree rows");
  depths_ = shared(C * 4, "row depths");
  uniforms_ = shared(R * 8, "uniforms");
  tokens_ = shared(R * 4, "selected tokens");
  retained_ = shared(maxLanes * 4, "retained");
  acceptedCount_ = shared(maxLanes * 4, "accepted");
  retainedRows_ = shared(maxLanes * 4, "retained rows");
  pageTable_ = device(uint64_t{pageTableEntries} * 8, "page table");
  layerBytes_ = pageBytes_ * physicalPages;
  kvAll_ = device(layerBytes_ * d.attentionLayers(), "kv pools");
  for (uint32_t l = 0; l < d.attentionLayers(); ++l) kvPools_.push_back(backend.view(kvAll_, layerBytes_ * l, layerBytes_));
  // Recurrent state: two cells and two tapes a lane.
  const ops::GdnShape gdn = d.gdnShape();
  strides_ = ops::GdnStateStrides::of(gdn, d.gdnLayers());
  cellBytes_ = strides_.cellBytes(d.gdnLayers());
  tapeLayerBytes_ = ops::gdnTapeLayerBytes(gdn);
  states_ = device(cellBytes_ * 2 * maxLanes, "GDN state cells");
  tape_ = device(tapeLayerBytes_ * d.gdnLayers() * 2 * maxLanes, "GDN tapes");
  // Scratch of every dense projection at a piece's most rows.
  const uint32_t pieceRows = std::min(rowCapacity_, kProjectionRows);
  ops::LinearScratchSize size;
  for (ops::LinearMatrix m : {ops::LinearMatrix{d.qkvWidth(), d.hidden}, ops::LinearMatrix{d.hidden, d.attentionWidth()},
                              ops::LinearMatrix{d.gdnPackedWidth, d.hidden}, ops::LinearMatrix{d.hidden, d.gdnWidth()},
                              d.dense() ? ops::LinearMatrix{d.denseFfn, d.hidden} : ops::LinearMatrix{d.experts, d.hidden},
                              d.dense() ? ops::LinearMatrix{d.hidden, d.denseFfn} : ops::LinearMatrix{d.experts, d.hidden},
                              ops::LinearMatrix{d.vocabulary, d.hidden}})
    size.include(linear_.scratchSize(m, pieceRows));
  if (d.dense()) {
    intermediate_ = device(uint64_t{windowRows} * d.denseFfn * 2, "SwiGLU rows");
    ffnTable_ = device(gguf_tables_bytes(d.denseFfn, gguf_row_tiles(pieceRows)), "SwiGLU table");
  }
  scratch_.input = device(size.input, "linear table");
  scratch_.partials = device(size.partials, "linear partials");
  scratch_.counters = device(std::max<uint64_t>(size.counters, 4), "linear counters");
  mixedTable_ = device(gguf_tables_bytes(std::max(d.attentionWidth(), d.gdnWidth()), gguf_row_tiles(pieceRows)), "mixer output table");
  // Staged queries for every tile of the longest chunk; partials for the tiles of one dispatch.
  const uint64_t fusedTile = uint64_t{d.kvHeads} * (d.qHeads / std::max(1u, d.kvHeads)) * 16;
  const uint64_t staged = fusedTile * std::max(maxLanes, gguf_row_tiles(rowCapacity_));
  const uint64_t fused = fusedTile * (rowCapacity_ > maxRows_ ? ATTENTION_MAXIMUM_SEQUENCES : maxLanes);
  attentionWorkspace_.queries = device(staged * d.headDimension * 2, "staged queries");
  attentionWorkspace_.querySums = device(staged * 4, "query sums");
  attentionWorkspace_.partials = device(fused * ATTENTION_MAXIMUM_SPLITS * d.headDimension * 2, "attention partials");
  attentionWorkspace_.partialSums = device(fused * ATTENTION_MAXIMUM_SPLITS * 8, "attention partial sums");
  const ops::MoeWorkspaceSize moe = d.dense() ? ops::MoeWorkspaceSize{} : ops::MoE::workspace(d.moeShape(), windowRows);
  moeWorkspace_ = {device(moe.selected, "moe selected"),    device(moe.weights, "moe weights"),     device(moe.routeSlot, "moe route slots"),
                   device(moe.slotRow, "moe slot rows"),    device(moe.tileExpert, "moe tile experts"), device(moe.tileRows, "moe tile rows"),
                   device(moe.tileTotal, "moe tile count"), device(moe.tables, "moe tables"),       device(moe.nextTables, "moe SwiGLU tables"),
                   device(moe.intermediate, "moe SwiGLU rows"), device(moe.expertOutput, "moe expert outputs")};
  const ops::SamplingWorkspaceSize s = ops::Sampling::workspace(maxRows_);
  sampling_.logits = logits_;
  sampling_.tokens = tokens_;
  sampling_.partialValues = device(s.partialValues, "argmax values");
  sampling_.partialIndices = device(s.partialIndices, "argmax indices");
  sampling_.masses = device(s.masses, "sampling masses");
  sampling_.ranges = device(s.ranges, "sampling ranges");
  sampling_.decisions = device(s.decisions, "sampling decisions");
  sampling_.uniforms = uniforms_;
  sampling_.inputTokens = inputTokens_;
  sampling_.treeRows = treeRows_;
  // The rows a Gated DeltaNet layer's prefill passes hand each other, for the longest chunk.
  const uint64_t keyWidth = uint64_t{d.gdnKeyHeads} * GDN_HEAD_DIMENSION;
  gdnPrefill_.queries = device(C * keyWidth * 2, "GDN prefill queries");
  gdnPrefill_.keys = device(C * keyWidth * 2, "GDN prefill keys");
  gdnPrefill_.values = device(C * d.gdnWidth() * 2, "GDN prefill values");
  gdnPrefill_.decay = device(C * d.gdnValueHeads * 4, "GDN prefill decay");
  gdnPrefill_.beta = device(C * d.gdnValueHeads * 2, "GDN prefill beta");
  gdnPrefill_.recurrentRows = device(C * d.gdnWidth() * 2, "GDN prefill rows");
}

const hip::Buffer &HybridVerify::draftProbabilities() {
  if (!draft_) {
    draft_ = backend_.allocateBuffer(uint64_t{maxRows_} * dims_.vocabulary * 4, BufferStorage::Private, "draft probabilities");
    sampling_.draftProbabilities = draft_;
  }
  return draft_;
}

uint64_t HybridVerify::stepBytes(const std::vector<HybridLane> &lanes) const {
  const ops::MoeShape moe = dims_.moeShape();
  uint64_t bytes = weights_.head.weightBytes();
  for (const HybridLayer &l : weights_.layers) {
    bytes += l.mixerInput.weightBytes() + l.mixerOutput.weightBytes() + l.gateRows.weightBytes();
    if (dims_.dense()) {
      bytes += l.ffnGate.weightBytes() + l.ffnUp.weightBytes() + l.ffnDown.weightBytes();
      continue;
    }
    bytes += l.routerRows ? l.routerRows.weightBytes() : l.router.weightBytes();
    bytes += uint64_t{moe.allExperts()} * (2 * gguf_image_bytes(l.experts.format, moe.ffn, moe.hidden) +
                                           gguf_image_bytes(l.experts.downFormat, moe.hidden, moe.ffn));
  }
  uint32_t rows = 0;
  for (const HybridLane &lane : lanes) {
    bytes += uint64_t{dims_.attentionLayers()} * (uint64_t{lane.block.committed} + lane.block.rows) * (pageBytes_ / ATTENTION_PAGE_TOKENS);
    bytes += 2ull * dims_.gdnLayers() * strides_.recurrentLayerBytes;  // each state read, and written
    rows += lane.block.rows;
  }
  return bytes + 2ull * rows * dims_.vocabulary * 4;
}

ops::AttentionPlan HybridVerify::planOf(const std::vector<HybridLane> &lanes) const {
  std::vector<ops::AttentionRows> sequences;
  uint32_t rows = 0;
  for (const HybridLane &lane : lanes) {
    sequences.push_back({rows, lane.block.rows, lane.block.committed, lane.block.tableFirst});
    rows += lane.block.rows;
  }
  return ops::PagedAttention::plan({dims_.qHeads, dims_.kvHeads, dims_.headDimension, dims_.rotaryPairs, dims_.normalizeHeads,
                                    dims_.gatedAttention},
                                   sequences);
}

void HybridVerify::encodeEmbedding(hip::CommandGraph &graph, uint32_t rows) {
  ops::Embedding::add(graph, weights_.embedding, inputTokens_, hidden_[0], rows);
}

void HybridVerify::encodeLayer(hip::CommandGraph &graph, uint32_t layer, const std::vector<HybridLane> &lanes, bool inputReady,
                               bool feedsNext) {
  if (lanes.empty() || lanes.size() > maxLanes_) throw std::invalid_argument("the step takes 1 to its most lanes");
  const HybridLayer &w = weights_.layers.at(layer);
  const bool attends = dims_.attends(layer);
  const uint32_t index = dims_.mixerIndex(layer);
  uint32_t rows = 0;
  for (const HybridLane &lane : lanes) rows += lane.block.rows;
  if (rows > maxRows_) throw std::invalid_argument("more rows than the step's buffers hold");
  const hip::Buffer &residual = hidden_[0], &next = hidden_[1];
  const uint64_t hiddenBytes = uint64_t{dims_.hidden} * 2;
  const uint32_t inputWidth = w.mixerInput.outputSize, mixedWidth = w.mixerOutput.inputSize;
  if (inputWidth != (attends ? dims_.qkvWidth() : dims_.gdnPackedWidth) || mixedWidth != (attends ? dims_.attentionWidth() : dims_.gdnWidth()) ||
      w.mixerInput.inputSize != dims_.hidden || w.mixerOutput.outputSize != dims_.hidden)
    throw std::invalid_argument("the layer's projections do not fit the model");
  if (dims_.dense() ? (w.ffnGate.outputSize != dims_.denseFfn || w.ffnUp.outputSize != dims_.denseFfn || w.ffnDown.inputSize != dims_.denseFfn ||
                       w.ffnGate.inputSize != dims_.hidden || w.ffnUp.inputSize != dims_.hidden || w.ffnDown.outputSize != dims_.hidden)
                    : (w.routerRows ? (w.routerRows.outputSize != dims_.experts || w.routerRows.inputSize != dims_.hidden)
                                    : (w.router.outputSize != dims_.experts || w.router.inputSize != dims_.hidden)))
    throw std::invalid_argument("the layer's FFN does not fit the model");

  // Mixer: hidden[1] = hidden[0] + out(mixer(in(norm(hidden[0])))). With one piece of rows the mixer's last kernel
  // writes its output rows' activation table beside them.
  const bool mixerTable = rows <= kProjectionRows;
  forRowPieces(rows, [&](uint32_t first, uint32_t count) {
    const hip::Buffer normalized = rowsOf(normalized_, first, count, hiddenBytes);
    ops::LinearBuffers in;
    in.input = normalized;
    in.output = rowsOf(packed_, first, count, uint64_t{inputWidth} * 2);
    in.scratch = scratch_;
    // The layer before may have left the table of these rows, less their inverse RMS, from its combine.
    in.prepared = inputReady ? ops::PreparedInput{normalized, ops::LinearInput::TableUnscaled}
                             : ops::Normalization::addRmsTable(graph, rowsOf(residual, first, count, hiddenBytes), w.inputNorm, normalized,
                                                               scratch_, dims_.hidden, count);
    linear_.add(graph, in, w.mixerInput, linear_.plan(w.mixerInput, count));
    if (!attends && w.gateRows) {
      // beta | alpha from rows of floats: the packed row's columns after q, k, v and z
      if (inputReady) throw std::invalid_argument("float gate rows read the normalized rows, which a deferred norm does not store");
      const ops::GdnShape shape = dims_.gdnShape();
      if (w.gateRows.outputSize != 2 * shape.valueHeads || w.gateRows.inputSize != dims_.hidden)
        throw std::invalid_argument("a GDN layer's gate rows are beta then alpha, a row a value head each");
      ops::FloatProjection::add(graph, normalized, w.gateRows, in.output, count, inputWidth,
                                shape.convolutionDimension + shape.valueHeads * GDN_HEAD_DIMENSION, ops::FloatOutput::BFloat16);
    }
  });
  if (attends) {
    const ops::AttentionPlan plan = planOf(lanes);
    const ops::KvPages pages{pageTable_, kvPools_.at(index), pageBytes_};
    ops::PagedAttention::addProjection(graph, plan, {packed_, w.queryNorm, w.keyNorm, ropeCos_, ropeSin_}, attentionWorkspace_, pages);
    ops::PagedAttention::addAttention(graph, plan, attentionWorkspace_, treeRows_, pages, mixed_, mixerTable ? mixedTable_ : hip::Buffer{}, packed_);
  } else {
    std::vector<ops::GdnLaneStep> steps;
    uint32_t firstRow = 0;
    for (size_t i = 0; i < lanes.size(); ++i) {
      const HybridLane &lane = lanes[i];
      steps.push_back({firstRow, lane.block.rows, lane.pendingPath, tapeOffset(uint32_t(i), lane.parity ^ 1u, index),
                       tapeOffset(uint32_t(i), lane.parity, index), cellOffset(uint32_t(i), lane.parity), cellOffset(uint32_t(i), lane.parity ^ 1u)});
      firstRow += lane.block.rows;
    }
    ops::GdnDecodeBuffers buffers{packed_, w.convolutionWeights, states_, tape_, w.decay, w.timeBias, w.mixerNorm, w.mixerNormFloat, mixed_,
                                  treeRows_, mixerTable ? mixedTable_ : hip::Buffer{}};
    ops::GDN::addDecode(graph, buffers, dims_.gdnShape(), index, strides_,
                        tiledGdnHeads_ ? ops::GdnHeadOrder::Tiled : ops::GdnHeadOrder::Grouped, steps);
  }
  forRowPieces(rows, [&](uint32_t first, uint32_t count) {
    ops::LinearBuffers out;
    out.input = rowsOf(mixed_, first, count, uint64_t{mixedWidth} * 2);
    out.output = rowsOf(next, first, count, hiddenBytes);
    out.residual = rowsOf(residual, first, count, hiddenBytes);
    out.scratch = scratch_;
    if (mixerTable) {  // the mixer wrote the table of its output rows
      out.scratch.input = mixedTable_;
      out.prepared = {out.input, ops::LinearInput::Table16};
    }
    linear_.add(graph, out, w.mixerOutput, linear_.plan(w.mixerOutput, count, ops::LinearEpilogue::Residual));
  });

  if (dims_.dense()) {
    // FFN: hidden[0] = hidden[1] + down(silu(gate n) * up n), n = norm(hidden[1]).
    forRowPieces(rows, [&](uint32_t first, uint32_t count) {
      const hip::Buffer normalized = rowsOf(normalized_, first, count, hiddenBytes);
      const ops::PreparedInput prepared = ops::Normalization::addRmsTable(graph, rowsOf(next, first, count, hiddenBytes), w.postNorm, normalized,
                                                                          scratch_, dims_.hidden, count);
      ops::FfnBuffers ffn{normalized, rowsOf(intermediate_, first, count, uint64_t{dims_.denseFfn} * 2), scratch_, ffnTable_};
      if (feedsNext) {
        ffn.followingNorm = layer + 1 < dims_.layers ? weights_.layers[layer + 1].inputNorm : weights_.finalNorm;
        ffn.followingTable = scratch_.input;
      }
      linear_.addSwiGlu(graph, {&w.ffnGate, &w.ffnUp, &w.ffnDown}, ffn, rowsOf(next, first, count, hiddenBytes),
                        rowsOf(residual, first, count, hiddenBytes), count, prepared);
    });
    return;
  }
  // FFN: hidden[0] = hidden[1] + sum over a row's experts of weight * expert(norm(hidden[1])).
  forRowPieces(rows, [&](uint32_t first, uint32_t count) {
    const hip::Buffer normalized = rowsOf(normalized_, first, count, hiddenBytes);
    ops::LinearBuffers router;
    router.input = normalized;
    router.output = rowsOf(scores_, first, count, uint64_t{dims_.experts} * 4);
    router.scratch = scratch_;
    router.prepared = ops::Normalization::addRmsTable(graph, rowsOf(next, first, count, hiddenBytes), w.postNorm, normalized, scratch_,
                                                      dims_.hidden, count);
    if (w.routerRows)
      ops::FloatProjection::add(graph, normalized, w.routerRows, router.output, count, dims_.experts, 0, ops::FloatOutput::Float32);
    else
      linear_.add(graph, router, w.router, linear_.plan(w.router, count));
  });
  const ops::MoeShape moe = dims_.moeShape();
  ops::MoE::addRouting(graph, scores_, dims_.experts, moeWorkspace_, moe, rows, normalized_, w.sharedScalarGate);
  ops::MoeFollowingNorm following;
  if (feedsNext) {
    following.weight = layer + 1 < dims_.layers ? weights_.layers[layer + 1].inputNorm : weights_.finalNorm;
    following.table = scratch_.input;
  }
  ops::MoE::addRouted(graph, normalized_, next, residual, w.experts, moeWorkspace_, moe, rows, following);
}

void HybridVerify::encodeHead(hip::CommandGraph &graph, uint32_t rows, bool inputReady) {
  const uint64_t hiddenBytes = uint64_t{dims_.hidden} * 2;
  forRowPieces(rows, [&](uint32_t first, uint32_t count) {
    const hip::Buffer normalized = rowsOf(normalized_, first, count, hiddenBytes);
    ops::LinearBuffers head;
    head.input = normalized;
    head.output = rowsOf(logits_, first, count, uint64_t{dims_.vocabulary} * 4);
    head.scratch = scratch_;
    head.prepared = inputReady ? ops::PreparedInput{normalized, ops::LinearInput::TableUnscaled}
                               : ops::Normalization::addRmsTable(graph, rowsOf(hidden_[0], first, count, hiddenBytes), weights_.finalNorm,
                                                                 normalized, scratch_, dims_.hidden, count);
    linear_.add(graph, head, weights_.head, linear_.plan(weights_.head, count));
  });
}

void HybridVerify::setCapture(std::vector<uint32_t> layers, hip::Buffer destination) {
  for (size_t i = 0; i < layers.size(); ++i)
    if (layers[i] >= dims_.layers || (i && layers[i] <= layers[i - 1])) throw std::invalid_argument("captured layers are the model's, ascending");
  if (!layers.empty())
    ops::requireBytes(destination, uint64_t{std::max(maxRows_, rowCapacity_)} * layers.size() * dims_.hidden * 2, "captured target hidden rows");
  captureLayers_ = std::move(layers);
  captured_ = std::move(destination);
}

void HybridVerify::encodeCapture(hip::CommandGraph &graph, uint32_t layer, uint32_t rows) const {
  for (size_t slot = 0; slot < captureLayers_.size(); ++slot)
    if (captureLayers_[slot] == layer)
      ops::RowCopy::add(graph, hidden_[0], {0, dims_.hidden, 0}, captured_,
                        {0, uint32_t(captureLayers_.size()) * dims_.hidden, uint32_t(slot) * dims_.hidden}, rows, dims_.hidden);
}

void HybridVerify::encode(hip::CommandGraph &graph, const std::vector<HybridLane> &lanes, bool commit) {
  if (lanes.empty() || lanes.size() > maxLanes_) throw std::invalid_argument("the step takes 1 to its most lanes");
  std::vector<ops::LaneRows> laneRows;
  std::vector<ops::RopeSequence> rope;
  std::vector<ops::SamplingPolicy> policies;
  std::vector<uint32_t> remaining;
  uint32_t rows = 0;
  bool samples = false;
  for (const HybridLane &lane : lanes) {
    laneRows.push_back({rows, lane.block.rows});
    rope.push_back({rows, lane.block.rows, lane.block.committed});
    policies.push_back(lane.block.policy);
    remaining.push_back(lane.block.remaining);
    samples = samples || lane.block.policy.samples();
    rows += lane.block.rows;
  }
  if (samples) (void)draftProbabilities();
  if (dims_.rotaryPairs)
    ops::RoPE::addTreeTables(graph, inverseFrequency_, depths_, ropeCos_, ropeSin_, dims_.rotaryPairs, rope);
  encodeEmbedding(graph, rows);
  // One piece of rows: a layer's combine can write the table the next layer's (or the head's) first projection reads.
  bool feeds = rows <= kProjectionRows && dims_.hidden % GGUF_BLOCK == 0;
  if (dims_.dense())
    for (const HybridLayer &l : weights_.layers) feeds = feeds && linear_.normsRows(l.ffnDown, rows);
  // float gate rows read the normalized rows themselves, which a layer fed by the combine before it never stores
  for (const HybridLayer &l : weights_.layers) feeds = feeds && !l.gateRows;
  for (uint32_t layer = 0; layer < dims_.layers; ++layer) {
    encodeLayer(graph, layer, lanes, feeds && layer > 0, feeds);
    encodeCapture(graph, layer, rows);
  }
  encodeHead(graph, rows, feeds);
  // a lane's penalties rewrite its rows of the head's fresh logits before anything selects from them
  const bool penalized = lanePolicies_.apply(policies);
  ops::SamplingBuffers selection = sampling_;
  if (lanePolicies_.anyConstrained(lanes.size())) {
    selection.tokenMask = lanePolicies_.tokenMask(maxRows_);
    selection.maskWords = lanePolicies_.maskWords();
  }
  if (penalized) ops::Sampling::addPenalties(graph, selection, dims_.vocabulary, dims_.vocabulary, laneRows, policies, lanePolicies_.table());
  ops::Sampling::addVerify(graph, selection, dims_.vocabulary, dims_.vocabulary, laneRows, policies, lanePolicies_.stopTokens());
  const ops::AcceptanceBuffers acceptance{inputTokens_, treeRows_, tokens_, retained_, acceptedCount_, retainedRows_};
  ops::Sampling::addAcceptance(graph, acceptance, laneRows, remaining, lanePolicies_.stopTokens());
  // a step that commits counts the tokens its penalized lanes keep, for the next step's penalties
  if (penalized && commit)
    ops::Sampling::addPenaltyCount(graph, acceptance, dims_.vocabulary, laneRows, lanePolicies_.penalized(lanes.size()), lanePolicies_.table());
  if (commit && dims_.attentionLayers())
    ops::PagedAttention::addPathCommit(graph, planOf(lanes), retainedRows_, {pageTable_, kvAll_, pageBytes_}, dims_.attentionLayers(),
                                       layerBytes_);
}

// A layer of a prompt chunk: every window's mixer input rows, the mixer over all the chunk's rows, then every window's
// output projection and FFN. No projection defers its norm here: a window starts with a norm pass.
void HybridVerify::encodePrefillLayer(hip::CommandGraph &graph, uint32_t layer, const ops::AttentionChunkPlan &plan, uint32_t tokens,
                                      uint64_t currentCell, uint64_t nextCell) {
  const HybridLayer &w = weights_.layers.at(layer);
  const bool attends = dims_.attends(layer);
  const uint32_t index = dims_.mixerIndex(layer);
  const hip::Buffer &residual = hidden_[0], &next = hidden_[1];
  const uint64_t hiddenBytes = uint64_t{dims_.hidden} * 2;
  const uint32_t inputWidth = w.mixerInput.outputSize, mixedWidth = w.mixerOutput.inputSize;
  if (inputWidth != (attends ? dims_.qkvWidth() : dims_.gdnPackedWidth) || mixedWidth != (attends ? dims_.attentionWidth() : dims_.gdnWidth()))
    throw std::invalid_argument("the layer's projections do not fit the model");
  forRowPieces(tokens, [&](uint32_t first, uint32_t count) {
    const hip::Buffer normalized = rowsOf(normalized_, first, count, hiddenBytes);
    ops::LinearBuffers in;
    in.input = normalized;
    in.output = rowsOf(packed_, first, count, uint64_t{inputWidth} * 2);
    in.scratch = scratch_;
    in.prepared = ops::Normalization::addRmsTable(graph, rowsOf(residual, first, count, hiddenBytes), w.inputNorm, normalized, scratch_,
                                                  dims_.hidden, count);
    linear_.add(graph, in, w.mixerInput, linear_.plan(w.mixerInput, count));
    if (!attends && w.gateRows) {
      const ops::GdnShape shape = dims_.gdnShape();
      ops::FloatProjection::add(graph, normalized, w.gateRows, in.output, count, inputWidth,
                                shape.convolutionDimension + shape.valueHeads * GDN_HEAD_DIMENSION, ops::FloatOutput::BFloat16);
    }
  });
  if (attends) {
    const ops::KvPages pages{pageTable_, kvPools_.at(index), pageBytes_};
    ops::PagedAttention::addChunkProjection(graph, plan, {packed_, w.queryNorm, w.keyNorm, ropeCos_, ropeSin_}, attentionWorkspace_, pages);
    ops::PagedAttention::addChunkAttention(graph, plan, attentionWorkspace_, treeRows_, pages, mixed_, {}, packed_);
  } else {
    ops::GdnPrefillBuffers buffers = gdnPrefill_;
    buffers.packed = packed_;
    buffers.convolutionWeights = w.convolutionWeights;
    buffers.states = states_;
    buffers.decayWeights = w.decay;
    buffers.timeBias = w.timeBias;
    buffers.mixerNorm = w.mixerNorm;
    buffers.floatNorm = w.mixerNormFloat;
    buffers.hidden = mixed_;
    buffers.currentCell = currentCell;
    buffers.nextCell = nextCell;
    ops::GDN::addPrefill(graph, buffers, dims_.gdnShape(), index, tokens, strides_,
                         tiledGdnHeads_ ? ops::GdnHeadOrder::Tiled : ops::GdnHeadOrder::Grouped);
  }
  const ops::MoeShape moe = dims_.moeShape();
  forRowPieces(tokens, [&](uint32_t first, uint32_t count) {
    const hip::Buffer nextRows = rowsOf(next, first, count, hiddenBytes), residualRows = rowsOf(residual, first, count, hiddenBytes);
    const hip::Buffer normalized = rowsOf(normalized_, first, count, hiddenBytes);
    ops::LinearBuffers out;
    out.input = rowsOf(mixed_, first, count, uint64_t{mixedWidth} * 2);
    out.output = nextRows;
    out.residual = residualRows;
    out.scratch = scratch_;
    linear_.add(graph, out, w.mixerOutput, linear_.plan(w.mixerOutput, count, ops::LinearEpilogue::Residual));
    const ops::PreparedInput prepared = ops::Normalization::addRmsTable(graph, nextRows, w.postNorm, normalized, scratch_, dims_.hidden, count);
    if (dims_.dense()) {
      const ops::FfnBuffers ffn{normalized, intermediate_, scratch_, ffnTable_};
      linear_.addSwiGlu(graph, {&w.ffnGate, &w.ffnUp, &w.ffnDown}, ffn, nextRows, residualRows, count, prepared);
      return;
    }
    if (w.routerRows) {
      ops::FloatProjection::add(graph, normalized, w.routerRows, scores_, count, dims_.experts, 0, ops::FloatOutput::Float32);
    } else {
      ops::LinearBuffers router;
      router.input = normalized;
      router.output = scores_;
      router.scratch = scratch_;
      router.prepared = prepared;
      linear_.add(graph, router, w.router, linear_.plan(w.router, count));
    }
    ops::MoE::addRouting(graph, scores_, dims_.experts, moeWorkspace_, moe, count, normalized, w.sharedScalarGate);
    ops::MoE::addRouted(graph, normalized, nextRows, residualRows, w.experts, moeWorkspace_, moe, count, {});
  });
}

void HybridVerify::encodePrefill(hip::CommandGraph &graph, uint32_t lane, uint32_t tableFirst, uint32_t committed, uint32_t tokens,
                                 uint32_t parity, uint32_t firstLayer, uint32_t layerCount) {
  if (!tokens || tokens > rowCapacity_) throw std::invalid_argument("a prompt chunk takes 1 to the driver's most prefill rows");
  if (lane >= maxLanes_) throw std::invalid_argument("no such lane");
  if (firstLayer >= dims_.layers || layerCount > dims_.layers - firstLayer) throw std::invalid_argument("no such layers");
  const ops::AttentionChunkPlan plan = ops::PagedAttention::planChunks(
      {dims_.qHeads, dims_.kvHeads, dims_.headDimension, dims_.rotaryPairs, dims_.normalizeHeads, dims_.gatedAttention},
      {{0, tokens, committed, tableFirst}});
  if (firstLayer == 0) {
    if (dims_.rotaryPairs) {
      // the RoPE tables eight blocks a dispatch, each dispatch over its own rows of the depths and tables
      const uint32_t span = ATTENTION_MAXIMUM_SEQUENCES * ATTENTION_MAXIMUM_ROWS;
      const uint64_t tableBytes = uint64_t{dims_.rotaryPairs} * 4;
      for (uint32_t first = 0; first < tokens; first += span) {
        const uint32_t count = std::min(span, tokens - first);
        std::vector<ops::RopeSequence> rope;
        for (uint32_t at = 0; at < count; at += ATTENTION_MAXIMUM_ROWS)
          rope.push_back({at, std::min<uint32_t>(ATTENTION_MAXIMUM_ROWS, count - at), committed + first + at});
        ops::RoPE::addTreeTables(graph, inverseFrequency_, rowsOf(depths_, first, count, 4), rowsOf(ropeCos_, first, count, tableBytes),
                                 rowsOf(ropeSin_, first, count, tableBytes), dims_.rotaryPairs, rope);
      }
    }
    encodeEmbedding(graph, tokens);
  }
  const uint32_t end = layerCount ? firstLayer + layerCount : dims_.layers;
  for (uint32_t layer = firstLayer; layer < end; ++layer) {
    encodePrefillLayer(graph, layer, plan, tokens, cellOffset(lane, parity), cellOffset(lane, parity ^ 1u));
    encodeCapture(graph, layer, tokens);
  }
}

} // namespace splash::model
