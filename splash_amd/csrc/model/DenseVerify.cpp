#include "model/DenseVerify.hpp"

#include <algorithm>
#include <cmath>
#include <stdexcept>

namespace splash::model {

using hip::BufferStorage;

namespace {
// A long chunk's projections run in windows of this many rows (whole 64-row pieces of the activation tables).
constexpr uint32_t kWindowRows = ops::kMaximumDispatchRows;
// Rows [first, first + count) of a buffer of rows of `rowBytes` bytes.
hip::Buffer rowsOf(const hip::Buffer &buffer, uint32_t first, uint32_t count, uint64_t rowBytes) {
  return buffer.slice(first * rowBytes, count * rowBytes);
}
// The activation tables (k inputs a row) of rows [first, first + count) of the tables of a chunk's rows: 64-row
// pieces lie one after the other, and `first` is a multiple of 64.
hip::Buffer tablesOf(const hip::Buffer &tables, uint32_t k, uint32_t first, uint32_t count) {
  return tables.slice(uint64_t{first / GGUF_MAXIMUM_ROWS} * gguf_table_bytes(k, GGUF_PIECE_TILES), gguf_tables_bytes(k, gguf_row_tiles(count)));
}
} // namespace

DenseVerify::DenseVerify(hip::Backend &backend, DenseDimensions d, uint32_t maxLanes, uint32_t physicalPages,
                         uint32_t pageTableEntries, uint32_t prefillRows)
    : backend_(backend), dims_(d), linear_(backend.deviceInfo()), maxLanes_(maxLanes),
      lanePolicies_(backend, maxLanes, d.vocabulary) {
  if (prefillRows > ops::kMaximumChunkRows) throw std::invalid_argument("a prompt chunk holds at most 2048 rows");
  if (!d.hidden || !d.layers || !d.vocabulary || !d.ffn || !maxLanes || maxLanes > ATTENTION_MAXIMUM_SEQUENCES)
    throw std::invalid_argument("a dense verify step takes a model and 1 to 8 lanes");
  if (d.hidden % GGUF_BLOCK || d.ffn % GGUF_BLOCK || d.attentionWidth() % GGUF_BLOCK || d.vocabulary % GGUF_TILE_COLUMNS)
    throw std::invalid_argument("the model's widths hold whole super-blocks and its vocabulary whole column tiles");
  maxRows_ = maxLanes * ATTENTION_MAXIMUM_ROWS;
  rowCapacity_ = std::max(maxRows_, prefillRows);
  const uint32_t windowRows = std::min(rowCapacity_, std::max(maxRows_, kWindowRows));  // the most rows of one projection dispatch
  weights_.layers.resize(d.layers);
  const ops::kv::Layout layout{d.kvHeads, d.headDimension};
  pageBytes_ = layout.bytesPerLayerPage();
  auto device = [&](uint64_t bytes, const char *label) { return backend.allocateBuffer(std::max<uint64_t>(bytes, 16), BufferStorage::Private, label); };
  auto shared = [&](uint64_t bytes, const char *label) { return backend.allocateBuffer(std::max<uint64_t>(bytes, 16), BufferStorage::Shared, label); };
  const uint64_t R = maxRows_, C = rowCapacity_;
  hidden_[0] = device(C * d.hidden * 2, "hidden 0");
  hidden_[1] = device(C * d.hidden * 2, "hidden 1");
  normalized_ = device(C * d.hidden * 2, "normalized");
  qkv_ = device(C * d.qkvWidth() * 2, "qkv");
  attention_ = device(C * d.attentionWidth() * 2, "attention output");
  intermediate_ = device(uint64_t{windowRows} * d.ffn * 2, "ffn intermediate");
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
  // One allocation holds every layer's pool, layerBytes_ apart, so one dispatch commits them all.
  layerBytes_ = pageBytes_ * physicalPages;
  kvAll_ = device(layerBytes_ * d.layers, "kv pools");
  kvPools_.reserve(d.layers);
  for (uint32_t l = 0; l < d.layers; ++l) kvPools_.push_back(backend.view(kvAll_, layerBytes_ * l, layerBytes_));
  // Scratch of every projection of the step at its most rows.
  ops::LinearScratchSize size;
  for (ops::LinearMatrix m : {ops::LinearMatrix{d.qkvWidth(), d.hidden}, ops::LinearMatrix{d.hidden, d.attentionWidth()},
                              ops::LinearMatrix{d.ffn, d.hidden}, ops::LinearMatrix{d.hidden, d.ffn},
                              ops::LinearMatrix{d.vocabulary, d.hidden}})
    size.include(linear_.scratchSize(m, windowRows));
  // the table of a chunk's normalized rows holds every window's: a layer's last projection leaves it for the next layer
  size.input = std::max<uint64_t>(size.input, gguf_tables_bytes(d.hidden, gguf_row_tiles(rowCapacity_)));
  // a q|k|v projection that prepares its attention block keeps partials whatever its plan's parts
  for (uint32_t rows : {16u, 32u, 64u})
    for (uint32_t format : {GGUF_FMT_Q4K, GGUF_FMT_Q6K})
      for (bool several : {false, true})
        if (!several || d.qkvWidth() % 64 == 0)
          size.include(ops::Linear::attentionScratchSize(linear_.plan(
              ops::LinearWorkload{{d.qkvWidth(), d.hidden}, std::min(rows, maxRows_), ops::LinearEpilogue::None, format, several})));
  scratch_.input = device(size.input, "linear table");
  scratch_.partials = device(size.partials, "linear partials");
  scratch_.counters = device(std::max<uint64_t>(size.counters, 4), "linear counters");
  // The attention merge and the gate/up pass write the table of the projection after them here.
  nextTable_ = device(gguf_tables_bytes(std::max(d.attentionWidth(), d.ffn), gguf_row_tiles(windowRows)), "linear table 2");
  if (rowCapacity_ > maxRows_)
    chunkAttentionTable_ = device(gguf_tables_bytes(d.attentionWidth(), gguf_row_tiles(rowCapacity_)), "chunk attention table");
  // Chained projections each keep a table, partials and counters of their own.
  chainTables_[0] = device(gguf_table_bytes(d.hidden, gguf_row_tiles(maxRows_)), "gate/up table");
  chainTables_[1] = device(gguf_table_bytes(d.ffn, gguf_row_tiles(maxRows_)), "down table");
  for (ops::LinearScratch &link : chainScratch_) {
    link.partials = device(size.partials, "chained partials");
    link.counters = device(std::max<uint64_t>(size.counters, 4), "chained counters");
  }
  chainProgress_ = device(GGUF_CHAIN_PROGRESS_WORDS * 4, "chain progress");
  chainProgress_.fill(0, GGUF_CHAIN_PROGRESS_WORDS * 4);
  // Attention workspace for the most splits any sequence may take.
  // Staged queries for every tile of the longest chunk; partials for the tiles of one dispatch.
  const uint64_t fusedTile = uint64_t{d.kvHeads} * (d.qHeads / d.kvHeads) * 16;
  const uint64_t staged = fusedTile * std::max(maxLanes, gguf_row_tiles(rowCapacity_));
  const uint64_t fused = fusedTile * (rowCapacity_ > maxRows_ ? ATTENTION_MAXIMUM_SEQUENCES : maxLanes);
  maxSplits_ = ATTENTION_MAXIMUM_SPLITS;
  attentionWorkspace_.queries = device(staged * d.headDimension * 2, "staged queries");
  attentionWorkspace_.querySums = device(staged * 4, "query sums");
  attentionWorkspace_.partials = device(fused * maxSplits_ * d.headDimension * 2, "attention partials");
  attentionWorkspace_.partialSums = device(fused * maxSplits_ * 8, "attention partial sums");
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
}

const hip::Buffer &DenseVerify::draftProbabilities() {
  if (!draft_) {
    draft_ = backend_.allocateBuffer(uint64_t{maxRows_} * dims_.vocabulary * 4, BufferStorage::Private, "draft probabilities");
    sampling_.draftProbabilities = draft_;
  }
  return draft_;
}

const hip::Buffer &DenseVerify::candidateChildren(uint32_t which) {
  if (!children_.candidateIds) {
    const uint64_t R = maxRows_;
    auto shared = [&](uint64_t bytes, const char *label) { return backend_.allocateBuffer(bytes, BufferStorage::Shared, label); };
    children_.candidateIds = shared(R * SAMPLING_CANDIDATES * 4, "candidate ids");
    children_.candidateProbabilities = shared(R * SAMPLING_CANDIDATES * 4, "candidate probabilities");
    children_.candidateDraws = shared(R * SAMPLING_TREE_CHILDREN, "drawn children");
    children_.childUniforms = shared(R * SAMPLING_TREE_CHILDREN * 4, "child uniforms");
    // no children drawn until a draft says so: such rows draw from their whole distribution
    std::vector<uint8_t> none(R * SAMPLING_TREE_CHILDREN, uint8_t(SAMPLING_NO_DRAW));
    children_.candidateDraws.upload(none.data(), none.size());
  }
  switch (which) {
  case 0: return children_.candidateIds;
  case 1: return children_.candidateProbabilities;
  case 2: return children_.candidateDraws;
  case 3: return children_.childUniforms;
  default: throw std::invalid_argument("no such candidate buffer");
  }
}

uint64_t DenseVerify::stepBytes(const std::vector<VerifyLane> &lanes) const {
  uint64_t bytes = weights_.head.weightBytes();
  for (const DenseLayer &l : weights_.layers)
    bytes += l.qkv.weightBytes() + l.output.weightBytes() + l.gate.weightBytes() + l.up.weightBytes() + l.down.weightBytes();
  uint32_t rows = 0;
  for (const VerifyLane &lane : lanes) {
    bytes += uint64_t{dims_.layers} * (uint64_t{lane.committed} + lane.rows) * (pageBytes_ / ATTENTION_PAGE_TOKENS);
    rows += lane.rows;
  }
  return bytes + 2ull * rows * dims_.vocabulary * 4;  // logits written, then read by acceptance
}

void DenseVerify::encodeEmbedding(hip::CommandGraph &graph, uint32_t rows) {
  ops::Embedding::add(graph, weights_.embedding, inputTokens_, hidden_[0], rows);
}

void DenseVerify::encodeLayer(hip::CommandGraph &graph, uint32_t layer, const ops::AttentionPlan &plan, uint32_t rows,
                              bool inputReady, bool feedsNext) {
  const DenseLayer &w = weights_.layers.at(layer);
  const hip::Buffer &residual = hidden_[0], &next = hidden_[1];
  // Attention block: hidden[1] = hidden[0] + o(attention(qkv(norm(hidden[0])))).
  // A table a residual projection's epilogue wrote stands for the normalized rows, which are then
  // never stored; their inverse RMS is applied by the projection that reads the table.
  const ops::PreparedInput ready{normalized_, ops::LinearInput::TableUnscaled};
  ops::PreparedInput prepared =
      inputReady ? ready : ops::Normalization::addRmsTable(graph, residual, w.inputNorm, normalized_, scratch_, dims_.hidden, rows);
  ops::LinearBuffers qkv;
  qkv.input = normalized_;
  qkv.output = qkv_;
  qkv.scratch = scratch_;
  qkv.prepared = prepared;
  const ops::LinearPlan qkvPlan = linear_.plan(w.qkv, rows);
  const ops::KvPages pages{pageTable_, kvPools_.at(layer), pageBytes_};
  ops::AttentionProjectionBuffers projection{qkv_, w.queryNorm, w.keyNorm, ropeCos_, ropeSin_};
  const ops::LinearScratchSize fusedNeed = ops::Linear::attentionScratchSize(qkvPlan);
  if (fusedPrepare_ && ops::PagedAttention::fusesProjection(plan, w.qkv, qkvPlan) &&
      scratch_.partials.sizeBytes() >= fusedNeed.partials && scratch_.counters.sizeBytes() >= fusedNeed.counters) {
    ops::PagedAttention::addFusedProjection(graph, linear_, qkv, w.qkv, qkvPlan, plan, projection, attentionWorkspace_, pages);
  } else {
    linear_.add(graph, qkv, w.qkv, qkvPlan);
    ops::PagedAttention::addProjection(graph, plan, projection, attentionWorkspace_, pages);
  }
  ops::PagedAttention::addAttention(graph, plan, attentionWorkspace_, treeRows_, pages, attention_, nextTable_);
  // The output projection adds the residual and, where its shape allows, norms the sum into the
  // gate/up pass's table; the down projection does the same for the layer (or head) after it.
  const bool outputNorms = linear_.normsRows(w.output, rows);
  ops::LinearBuffers output;
  output.input = attention_;
  output.output = next;
  output.residual = residual;
  output.scratch = scratch_;
  output.scratch.input = nextTable_;
  output.prepared = {attention_, ops::LinearInput::Table16};
  if (outputNorms) {
    output.normWeight = w.postNorm;
    output.nextTable = scratch_.input;
  }
  linear_.add(graph, output, w.output,
              linear_.plan(w.output, rows, outputNorms ? ops::LinearEpilogue::ResidualNorm : ops::LinearEpilogue::Residual));
  // FFN block: hidden[0] = hidden[1] + down(silu(gate n) * up n), n = norm(hidden[1]).
  prepared = outputNorms ? ready : ops::Normalization::addRmsTable(graph, next, w.postNorm, normalized_, scratch_, dims_.hidden, rows);
  ops::FfnBuffers ffn{normalized_, intermediate_, scratch_, nextTable_};
  if (feedsNext) {
    ffn.followingNorm = layer + 1 < dims_.layers ? weights_.layers[layer + 1].inputNorm : weights_.finalNorm;
    ffn.followingTable = scratch_.input;
  }
  linear_.addSwiGlu(graph, {&w.gate, &w.up, &w.down}, ffn, next, residual, rows, prepared);
}

void DenseVerify::setCapture(std::vector<uint32_t> layers, hip::Buffer destination) {
  for (size_t i = 0; i < layers.size(); ++i)
    if (layers[i] >= dims_.layers || (i && layers[i] <= layers[i - 1])) throw std::invalid_argument("captured layers are the model's, ascending");
  if (!layers.empty())
    ops::requireBytes(destination, uint64_t{std::max(maxRows_, rowCapacity_)} * layers.size() * dims_.hidden * 2, "captured target hidden rows");
  captureLayers_ = std::move(layers);
  captured_ = std::move(destination);
}

void DenseVerify::encodeCapture(hip::CommandGraph &graph, uint32_t layer, uint32_t rows) const {
  for (size_t slot = 0; slot < captureLayers_.size(); ++slot)
    if (captureLayers_[slot] == layer)
      ops::RowCopy::add(graph, hidden_[0], {0, dims_.hidden, 0}, captured_,
                        {0, uint32_t(captureLayers_.size()) * dims_.hidden, uint32_t(slot) * dims_.hidden}, rows, dims_.hidden);
}

bool DenseVerify::chains(uint32_t rows) const noexcept {
  if (!chained_ || !captureLayers_.empty() || rows > ops::kMaximumDecodeTileRows || !layersFeedNext(rows)) return false;
  for (const DenseLayer &l : weights_.layers)
    if (!linear_.normsRows(l.output, rows)) return false;
  return true;
}

uint32_t DenseVerify::takeChainStatus() {
  if (!encodedChains_) return 0;
  uint32_t status = 0;
  chainProgress_.download(&status, 4, GGUF_CHAIN_LINKS * 4);
  if (status) chainProgress_.fill(0, GGUF_CHAIN_PROGRESS_WORDS * 4);
  return status;
}

// The layers with their projections chained: the first layer's q|k|v on its own, then a layer's head norms, RoPE and
// cache store, its attention, and one dispatch of its output projection, gate/up pair, down projection and the q|k|v
// projection of the layer after it (after the last layer, the LM head).
void DenseVerify::encodeChainedLayers(hip::CommandGraph &graph, const ops::AttentionPlan &plan, uint32_t rows) {
  const hip::Buffer &tableQkv = scratch_.input, &tableOutput = nextTable_, &tableGateUp = chainTables_[0], &tableDown = chainTables_[1];
  const ops::PreparedInput ready{normalized_, ops::LinearInput::TableUnscaled};
  auto scratchOf = [&](uint32_t link, const hip::Buffer &table) {
    ops::LinearScratch scratch = chainScratch_[link];
    scratch.input = table;
    return scratch;
  };
  {
    const DenseLayer &first = weights_.layers.front();
    ops::LinearBuffers qkv;
    qkv.input = normalized_;
    qkv.output = qkv_;
    qkv.scratch = scratch_;
    qkv.prepared = ops::Normalization::addRmsTable(graph, hidden_[0], first.inputNorm, normalized_, scratch_, dims_.hidden, rows);
    linear_.add(graph, qkv, first.qkv, linear_.plan(first.qkv, rows));
  }
  for (uint32_t layer = 0; layer < dims_.layers; ++layer) {
    const DenseLayer &w = weights_.layers[layer];
    const bool lastLayer = layer + 1 == dims_.layers;
    const ops::KvPages pages{pageTable_, kvPools_.at(layer), pageBytes_};
    ops::AttentionProjectionBuffers projection{qkv_, w.queryNorm, w.keyNorm, ropeCos_, ropeSin_};
    ops::PagedAttention::addProjection(graph, plan, projection, attentionWorkspace_, pages);
    ops::PagedAttention::addAttention(graph, plan, attentionWorkspace_, treeRows_, pages, attention_, tableOutput);
    std::vector<ops::ChainedProjection> links;
    ops::LinearBuffers output;
    output.input = attention_;
    output.output = hidden_[1];
    output.residual = hidden_[0];
    output.scratch = scratchOf(0, tableOutput);
    output.prepared = {attention_, ops::LinearInput::Table16};
    output.normWeight = w.postNorm;
    output.nextTable = tableGateUp;
    links.push_back({output, &w.output, linear_.plan(w.output, rows, ops::LinearEpilogue::ResidualNorm)});
    ops::LinearBuffers pair;
    pair.input = normalized_;
    pair.output = intermediate_;
    pair.scratch = scratchOf(1, tableGateUp);
    pair.prepared = ready;
    pair.nextTable = tableDown;
    links.push_back({pair, &w.up, linear_.plan(w.up, rows, ops::LinearEpilogue::GateUp), &w.gate});
    ops::LinearBuffers down;
    down.input = intermediate_;
    down.output = hidden_[0];
    down.residual = hidden_[1];
    down.scratch = scratchOf(2, tableDown);
    down.prepared = {intermediate_, ops::LinearInput::Table16};
    down.normWeight = lastLayer ? weights_.finalNorm : weights_.layers[layer + 1].inputNorm;
    down.nextTable = tableQkv;
    links.push_back({down, &w.down, linear_.plan(w.down, rows, ops::LinearEpilogue::ResidualNorm)});
    const ops::Projection &following = lastLayer ? weights_.head : weights_.layers[layer + 1].qkv;
    ops::LinearBuffers next;
    next.input = normalized_;
    next.output = lastLayer ? logits_ : qkv_;
    next.scratch = scratchOf(3, tableQkv);
    next.prepared = ready;
    links.push_back({next, &following, linear_.plan(following, rows)});
    linear_.addChain(graph, std::move(links), chainProgress_);
  }
  encodedChains_ = true;
}

bool DenseVerify::layersFeedNext(uint32_t rows) const noexcept {
  for (const DenseLayer &l : weights_.layers)
    if (!linear_.normsRows(l.down, rows)) return false;
  return true;
}

void DenseVerify::encodeHead(hip::CommandGraph &graph, uint32_t rows, bool inputReady) {
  const ops::PreparedInput prepared =
      inputReady ? ops::PreparedInput{normalized_, ops::LinearInput::TableUnscaled}
                 : ops::Normalization::addRmsTable(graph, hidden_[0], weights_.finalNorm, normalized_, scratch_, dims_.hidden, rows);
  ops::LinearBuffers head;
  head.input = normalized_;
  head.output = logits_;
  head.scratch = scratch_;
  head.prepared = prepared;
  linear_.add(graph, head, weights_.head, linear_.plan(weights_.head, rows));
}

void DenseVerify::setStagedPrefill(bool staged) {
  if (staged && !prefillTable_) {
    if (rowCapacity_ <= maxRows_) throw std::invalid_argument("the driver was created without room for a long prompt chunk");
    const uint32_t widest = std::max({dims_.hidden, dims_.attentionWidth(), dims_.ffn});
    prefillTable_ = backend_.allocateBuffer(ops::Linear::prefillTableBytes(widest, rowCapacity_), BufferStorage::Private, "prefill tables");
    const uint64_t ffnBytes = uint64_t{rowCapacity_} * dims_.ffn * 2;
    gateRows_ = backend_.allocateBuffer(ffnBytes, BufferStorage::Private, "prefill gate rows");
    upRows_ = backend_.allocateBuffer(ffnBytes, BufferStorage::Private, "prefill up rows");
    swigluRows_ = backend_.allocateBuffer(ffnBytes, BufferStorage::Private, "prefill SwiGLU rows");
  }
  stagedPrefill_ = staged;
}

// A layer of a long chunk under the staged rule: each projection one pass of the prefill tile over all the rows.
void DenseVerify::encodeStagedChunkLayer(hip::CommandGraph &graph, uint32_t layer, const ops::AttentionChunkPlan &plan, uint32_t tokens) {
  const DenseLayer &w = weights_.layers.at(layer);
  const hip::Buffer &residual = hidden_[0], &next = hidden_[1];
  ops::Normalization::addRms(graph, residual, w.inputNorm, normalized_, dims_.hidden, tokens);
  ops::Linear::addPrefill(graph, normalized_, w.qkv, qkv_, {}, prefillTable_, tokens);
  const ops::KvPages pages{pageTable_, kvPools_.at(layer), pageBytes_};
  ops::PagedAttention::addChunkProjection(graph, plan, {qkv_, w.queryNorm, w.keyNorm, ropeCos_, ropeSin_}, attentionWorkspace_, pages);
  ops::PagedAttention::addChunkAttention(graph, plan, attentionWorkspace_, treeRows_, pages, attention_);
  ops::Linear::addPrefill(graph, attention_, w.output, next, residual, prefillTable_, tokens);
  ops::Normalization::addRms(graph, next, w.postNorm, normalized_, dims_.hidden, tokens);
  ops::Linear::addPrefill(graph, normalized_, w.gate, gateRows_, {}, prefillTable_, tokens);
  ops::Linear::addPrefill(graph, normalized_, w.up, upRows_, {}, prefillTable_, tokens);
  ops::SwiGlu::add(graph, gateRows_, upRows_, swigluRows_, uint64_t{tokens} * dims_.ffn);
  ops::Linear::addPrefill(graph, swigluRows_, w.down, residual, next, prefillTable_, tokens);
}

// A layer of a long chunk: every window's q|k|v rows, the chunked attention over all of them, then every window's output
// projection and SwiGLU. Each window's projections and tables are the ones encodeLayer gives a step of its rows.
void DenseVerify::encodeChunkLayer(hip::CommandGraph &graph, uint32_t layer, const ops::AttentionChunkPlan &plan, uint32_t tokens,
                                   bool inputReady, bool feedsNext) {
  const DenseLayer &w = weights_.layers.at(layer);
  const uint64_t hiddenBytes = uint64_t{dims_.hidden} * 2;
  struct Window {
    uint32_t first, rows;
    hip::Buffer residual, next, normalized, qkv, attention;
    ops::LinearScratch scratch;  // the driver's partials and counters, the window's own tables of normalized rows
  };
  std::vector<Window> windows;
  for (uint32_t first = 0; first < tokens; first += kWindowRows) {
    Window v;
    v.first = first;
    v.rows = std::min(kWindowRows, tokens - first);
    v.residual = rowsOf(hidden_[0], first, v.rows, hiddenBytes);
    v.next = rowsOf(hidden_[1], first, v.rows, hiddenBytes);
    v.normalized = rowsOf(normalized_, first, v.rows, hiddenBytes);
    v.qkv = rowsOf(qkv_, first, v.rows, uint64_t{dims_.qkvWidth()} * 2);
    v.attention = rowsOf(attention_, first, v.rows, uint64_t{dims_.attentionWidth()} * 2);
    v.scratch = scratch_;
    v.scratch.input = tablesOf(scratch_.input, dims_.hidden, first, v.rows);
    windows.push_back(std::move(v));
  }
  for (const Window &v : windows) {
    const ops::PreparedInput prepared =
        inputReady ? ops::PreparedInput{v.normalized, ops::LinearInput::TableUnscaled}
                   : ops::Normalization::addRmsTable(graph, v.residual, w.inputNorm, v.normalized, v.scratch, dims_.hidden, v.rows);
    ops::LinearBuffers qkv;
    qkv.input = v.normalized;
    qkv.output = v.qkv;
    qkv.scratch = v.scratch;
    qkv.prepared = prepared;
    linear_.add(graph, qkv, w.qkv, linear_.plan(w.qkv, v.rows));
  }
  const ops::KvPages pages{pageTable_, kvPools_.at(layer), pageBytes_};
  ops::PagedAttention::addChunkProjection(graph, plan, {qkv_, w.queryNorm, w.keyNorm, ropeCos_, ropeSin_}, attentionWorkspace_, pages);
  ops::PagedAttention::addChunkAttention(graph, plan, attentionWorkspace_, treeRows_, pages, attention_, chunkAttentionTable_);
  for (const Window &v : windows) {
    const ops::PreparedInput ready{v.normalized, ops::LinearInput::TableUnscaled};
    const bool outputNorms = linear_.normsRows(w.output, v.rows);
    ops::LinearBuffers output;
    output.input = v.attention;
    output.output = v.next;
    output.residual = v.residual;
    output.scratch = v.scratch;
    output.scratch.input = tablesOf(chunkAttentionTable_, dims_.attentionWidth(), v.first, v.rows);
    output.prepared = {v.attention, ops::LinearInput::Table16};
    if (outputNorms) {
      output.normWeight = w.postNorm;
      output.nextTable = v.scratch.input;
    }
    linear_.add(graph, output, w.output,
                linear_.plan(w.output, v.rows, outputNorms ? ops::LinearEpilogue::ResidualNorm : ops::LinearEpilogue::Residual));
    const ops::PreparedInput prepared =
        outputNorms ? ready : ops::Normalization::addRmsTable(graph, v.next, w.postNorm, v.normalized, v.scratch, dims_.hidden, v.rows);
    ops::FfnBuffers ffn{v.normalized, intermediate_, v.scratch, nextTable_};
    if (feedsNext) {
      ffn.followingNorm = layer + 1 < dims_.layers ? weights_.layers[layer + 1].inputNorm : weights_.finalNorm;
      ffn.followingTable = v.scratch.input;
    }
    linear_.addSwiGlu(graph, {&w.gate, &w.up, &w.down}, ffn, v.next, v.residual, v.rows, prepared);
  }
}

void DenseVerify::encodePrefill(hip::CommandGraph &graph, uint32_t tableFirst, uint32_t committed, uint32_t tokens) {
  if (!tokens || tokens > rowCapacity_) throw std::invalid_argument("a prompt chunk takes 1 to the driver's most prefill rows");
  if (tokens > maxRows_) {
    const ops::AttentionGeometry geometry{dims_.qHeads, dims_.kvHeads, dims_.headDimension, dims_.rotaryPairs, dims_.normalizeHeads};
    const ops::AttentionChunkPlan plan = ops::PagedAttention::planChunks(geometry, {{0, tokens, committed, tableFirst}});
    if (dims_.rotaryPairs) {
      // the RoPE tables eight blocks a dispatch, each dispatch over its own rows of the depths and tables
      const uint32_t span = ATTENTION_MAXIMUM_SEQUENCES * ATTENTION_MAXIMUM_ROWS;
      for (uint32_t first = 0; first < tokens; first += span) {
        const uint32_t count = std::min(span, tokens - first);
        std::vector<ops::RopeSequence> rope;
        for (uint32_t at = 0; at < count; at += ATTENTION_MAXIMUM_ROWS)
          rope.push_back({at, std::min<uint32_t>(ATTENTION_MAXIMUM_ROWS, count - at), committed + first + at});
        const uint64_t tableBytes = uint64_t{dims_.rotaryPairs} * 4;
        ops::RoPE::addTreeTables(graph, inverseFrequency_, rowsOf(depths_, first, count, 4), rowsOf(ropeCos_, first, count, tableBytes),
                                 rowsOf(ropeSin_, first, count, tableBytes), dims_.rotaryPairs, rope);
      }
    }
    encodeEmbedding(graph, tokens);
    // every window is a step's worth of rows at most, so what holds for one holds for all
    const bool feeds = layersFeedNext(std::min(tokens, kWindowRows));
    for (uint32_t layer = 0; layer < dims_.layers; ++layer) {
      if (stagedPrefill_) encodeStagedChunkLayer(graph, layer, plan, tokens);
      else encodeChunkLayer(graph, layer, plan, tokens, feeds && layer > 0, feeds && layer + 1 < dims_.layers);
      encodeCapture(graph, layer, tokens);
    }
    return;
  }
  std::vector<ops::AttentionRows> sequences;
  std::vector<ops::RopeSequence> rope;
  for (uint32_t first = 0; first < tokens; first += ATTENTION_MAXIMUM_ROWS) {
    const uint32_t rows = std::min<uint32_t>(ATTENTION_MAXIMUM_ROWS, tokens - first);
    sequences.push_back({first, rows, committed + first, tableFirst});
    rope.push_back({first, rows, committed + first});
  }
  const ops::AttentionGeometry geometry{dims_.qHeads, dims_.kvHeads, dims_.headDimension, dims_.rotaryPairs, dims_.normalizeHeads};
  const ops::AttentionPlan plan = ops::PagedAttention::plan(geometry, sequences);
  if (dims_.rotaryPairs)
    ops::RoPE::addTreeTables(graph, inverseFrequency_, depths_, ropeCos_, ropeSin_, dims_.rotaryPairs, rope);
  encodeEmbedding(graph, tokens);
  const bool feeds = layersFeedNext(tokens);
  for (uint32_t layer = 0; layer < dims_.layers; ++layer) {
    encodeLayer(graph, layer, plan, tokens, feeds && layer > 0, feeds && layer + 1 < dims_.layers);
    encodeCapture(graph, layer, tokens);
  }
}

void DenseVerify::encode(hip::CommandGraph &graph, const std::vector<VerifyLane> &lanes, bool commit) {
  if (lanes.empty() || lanes.size() > maxLanes_) throw std::invalid_argument("the step takes 1 to its most lanes");
  std::vector<ops::AttentionRows> sequences;
  std::vector<ops::LaneRows> laneRows;
  std::vector<ops::RopeSequence> rope;
  std::vector<ops::SamplingPolicy> policies;
  std::vector<uint32_t> remaining;
  uint32_t rows = 0;
  bool samples = false;
  for (const VerifyLane &lane : lanes) {
    sequences.push_back({rows, lane.rows, lane.committed, lane.tableFirst});
    laneRows.push_back({rows, lane.rows});
    rope.push_back({rows, lane.rows, lane.committed});
    policies.push_back(lane.policy);
    remaining.push_back(lane.remaining);
    samples = samples || lane.policy.samples();
    rows += lane.rows;
  }
  const ops::AttentionGeometry geometry{dims_.qHeads, dims_.kvHeads, dims_.headDimension, dims_.rotaryPairs, dims_.normalizeHeads};
  const ops::AttentionPlan plan = ops::PagedAttention::plan(geometry, sequences);
  if (samples && !testChildren_) (void)draftProbabilities();
  if (dims_.rotaryPairs)
    ops::RoPE::addTreeTables(graph, inverseFrequency_, depths_, ropeCos_, ropeSin_, dims_.rotaryPairs, rope);
  encodeEmbedding(graph, rows);
  if (chains(rows)) {
    encodeChainedLayers(graph, plan, rows);
  } else {
    const bool feeds = layersFeedNext(rows);
    for (uint32_t layer = 0; layer < dims_.layers; ++layer) {
      encodeLayer(graph, layer, plan, rows, feeds && layer > 0, feeds);
      encodeCapture(graph, layer, rows);
    }
    encodeHead(graph, rows, feeds);
  }
  // the sampled lanes' test is the step's choice (setTestChildren), not a property of which buffers were ever fetched
  ops::SamplingBuffers sampling = sampling_;
  if (testChildren_) {
    sampling.candidateIds = children_.candidateIds;
    sampling.candidateProbabilities = children_.candidateProbabilities;
    sampling.candidateDraws = children_.candidateDraws;
    sampling.childUniforms = children_.childUniforms;
  }
  // a lane's penalties rewrite its rows of the head's fresh logits before anything selects from them
  const bool penalized = lanePolicies_.apply(policies);
  if (lanePolicies_.anyConstrained(lanes.size())) {
    sampling.tokenMask = lanePolicies_.tokenMask(maxRows_);
    sampling.maskWords = lanePolicies_.maskWords();
  }
  if (penalized) ops::Sampling::addPenalties(graph, sampling, dims_.vocabulary, dims_.vocabulary, laneRows, policies, lanePolicies_.table());
  ops::Sampling::addVerify(graph, sampling, dims_.vocabulary, dims_.vocabulary, laneRows, policies, lanePolicies_.stopTokens());
  const ops::AcceptanceBuffers acceptance{inputTokens_, treeRows_, tokens_, retained_, acceptedCount_, retainedRows_};
  ops::Sampling::addAcceptance(graph, acceptance, laneRows, remaining, lanePolicies_.stopTokens());
  // a step that commits counts the tokens its penalized lanes keep, for the next step's penalties
  if (penalized && commit)
    ops::Sampling::addPenaltyCount(graph, acceptance, dims_.vocabulary, laneRows, lanePolicies_.penalized(lanes.size()), lanePolicies_.table());
  if (commit)
    ops::PagedAttention::addPathCommit(graph, plan, retainedRows_, {pageTable_, kvAll_, pageBytes_}, dims_.layers, layerBytes_);
}

} // namespace splash::model
