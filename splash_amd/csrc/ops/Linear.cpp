#include "ops/Linear.hpp"

#include <algorithm>
#include <array>
#include <stdexcept>

namespace splash::ops {

void requireBytes(const hip::Buffer &buffer, uint64_t bytes, const char *what) {
  if (!buffer) throw std::invalid_argument(std::string(what) + " buffer is missing");
  if (buffer.sizeBytes() < bytes) throw std::invalid_argument(std::string(what) + " buffer is too small");
}

namespace {

const char *epilogueSuffix(LinearEpilogue epilogue, FloatOutput destination, bool table = false) {
  if (epilogue == LinearEpilogue::GateUp && table) return "_gt";
  switch (epilogue) {
  case LinearEpilogue::None: return destination == FloatOutput::Float32 ? "_a_f32" : "_a";
  case LinearEpilogue::Residual: return "_r";
  case LinearEpilogue::GateUp: return "_g";
  case LinearEpilogue::ResidualNorm: return "_rn";
  }
  return "_a";
}

// Wave work units of a dispatch: one column tile each; a gate/up pair holds the tiles of both tensors.
uint32_t unitsOf(uint32_t columns, LinearEpilogue epilogue) {
  const uint32_t tiles = columns / GGUF_TILE_COLUMNS;
  return epilogue == LinearEpilogue::GateUp ? 2 * tiles : tiles;
}
constexpr uint32_t kWavesAcross = 4;  // waves, and so units, of a workgroup
uint32_t groupsOf(uint32_t columns, LinearEpilogue epilogue) { return (unitsOf(columns, epilogue) + kWavesAcross - 1) / kWavesAcross; }

void requireSegments(const Projection &p, LinearMatrix matrix) {
  if (p.outputSize != matrix.outputSize || p.inputSize != matrix.inputSize)
    throw std::invalid_argument("block projection does not match its plan's matrix");
  const std::vector<QuantizedSegment> &segments = p.blocks().segments;
  if (segments.empty() || segments.size() > GGUF_MAXIMUM_SEGMENTS)
    throw std::invalid_argument("a block projection dispatch takes one to three segments");
  for (const QuantizedSegment &s : segments) {
    if (s.outputSize % GGUF_TILE_COLUMNS || s.inputSize % GGUF_BLOCK)
      throw std::invalid_argument("block segments hold whole 16-column tiles of whole 256-input super-blocks");
    requireBytes(s.image, gguf_image_bytes(s.formatId, s.outputSize, s.inputSize), "block weight image");
  }
}

} // namespace

LinearWorkload workloadOf(const Projection &projection, uint32_t rows, LinearEpilogue epilogue) {
  LinearWorkload w{{projection.outputSize, projection.inputSize}, rows, epilogue};
  const std::vector<QuantizedSegment> &segments = projection.blocks().segments;
  if (!segments.empty()) w.formatId = segments.front().formatId;
  for (const QuantizedSegment &s : segments) {
    w.severalFormats |= s.formatId != segments.front().formatId;
    if (gguf_record_bytes(s.formatId) > gguf_record_bytes(w.formatId)) w.formatId = s.formatId;
  }
  return w;
}

LinearPlan::LinearPlan(LinearWorkload workload, LinearConfig config, FloatOutput destination)
    : workload_(workload), config_(config), destination_(destination) {
  requireConfiguration();
}

void LinearPlan::requireConfiguration() const {
  const auto [n, k] = workload_.matrix;
  if (!workload_.rows || workload_.rows > kMaximumDispatchRows)
    throw std::invalid_argument("the block tile runs plans of 1 to 64 rows");
  if (!n || n % GGUF_TILE_COLUMNS || !k || k % GGUF_BLOCK)
    throw std::invalid_argument("block projections take whole 16-column tiles and 256-input super-blocks");
  const LinearConfig &c = config_;
  if (!c.validSplits() || c.splits > k / GGUF_BLOCK)
    throw std::invalid_argument("block splits take at least one super-block each");
  if (c.wholeGroups > groupsOf(n, workload_.epilogue)) throw std::invalid_argument("more whole workgroups than the projection has");
  if (destination_ == FloatOutput::Float32 && workload_.epilogue != LinearEpilogue::None)
    throw std::invalid_argument("only a plain block plan writes fp32");
  if (workload_.severalFormats && c.tile != LinearTile::GgufColumn &&
      (workload_.epilogue != LinearEpilogue::None || destination_ != FloatOutput::BFloat16 || c.wholeGroups || n % 64))
    throw std::invalid_argument("segments of several formats take a plain bf16 plan whose workgroups all partition K");
  if (c.tile == LinearTile::GgufColumn &&
      (workload_.rows > GGUF_COLUMN_ROWS || c.splits != 1 || c.wholeGroups || workload_.epilogue == LinearEpilogue::ResidualNorm))
    throw std::invalid_argument("the column tile takes up to two rows, unsplit, and does not norm its rows");
  if (c.tile == LinearTile::GgufStaged &&
      (workload_.severalFormats || (workload_.epilogue != LinearEpilogue::None && workload_.epilogue != LinearEpilogue::Residual)))
    throw std::invalid_argument("the staged rule takes plain and residual plans of one format");
}

LinearScratchSize LinearPlan::scratchSize() const noexcept {
  const auto [n, k] = workload_.matrix;
  const uint32_t tiles = gguf_row_tiles(workload_.rows);
  LinearScratchSize size;
  size.input = gguf_tables_bytes(k, tiles);
  if (config_.splits > 1) {
    // [split][unit][row tile][4][64 lanes] fp32 partials over whole workgroups, and one counter per workgroup.
    // of the partitioned workgroups only
    const uint64_t groups = std::max<uint64_t>(1, groupsOf(n, workload_.epilogue) - config_.wholeGroups);
    // a piece of the dispatch's rows keeps its own, as many as a whole piece takes
    // (the kernel's row tiles: 1, 2 or 4, which may be more than the rows fill)
    const uint32_t pieces = rowPieces(workload_.rows), pieceTiles = storageRows() / GGUF_ROW_TILE;
    size.partials = uint64_t{pieces} * config_.splits * groups * kWavesAcross * pieceTiles * 256u * sizeof(float);
    size.counters = uint64_t{pieces} * groups * sizeof(uint32_t);
  }
  return size;
}

Linear::Linear(const sp_device_info &device) noexcept {
  if (device.compute_units) calibration_.computeUnits = device.compute_units;
}

LinearPlan Linear::plan(LinearWorkload workload, LinearConfig config, FloatOutput destination) {
  return LinearPlan(workload, config, destination);
}

LinearPlan Linear::plan(LinearWorkload w, FloatOutput destination) const {
  // Fill the device: partition K across workgroups (fp32 partials, summed in split order by the
  // last arriver) until the dispatch holds groupsPerUnit workgroups per compute unit or a
  // workgroup's range is down to minimumBlocksPerWave super-blocks.
  const uint32_t blocks = w.matrix.inputSize / GGUF_BLOCK;
  const uint32_t groups = std::max(1u, groupsOf(w.matrix.outputSize, w.epilogue));
  const uint32_t wanted =
      calibration_.computeUnits * (w.formatId == GGUF_FMT_Q6K ? calibration_.groupsPerUnitQ6K : calibration_.groupsPerUnit);
  uint32_t most = std::min(LinearConfig::kMaximumSplits, std::max(1u, blocks / calibration_.minimumBlocksPerWave));
  // A projection of a few column tiles (a router) leaves most of the device idle however short its
  // ranges: it partitions K down to single super-blocks.
  if (groups * most * 4 < calibration_.computeUnits) most = std::min(LinearConfig::kMaximumSplits, blocks);
  LinearConfig config;
  const uint32_t units = calibration_.computeUnits;
  if (!w.severalFormats && groups >= 2 * units && groups % units) {
    // Enough workgroups to fill the device without partitioning, but a remainder that would leave
    // most units idle at the end: the whole rounds run unsplit and the remainder is partitioned
    // into about one piece per unit, dispatched last.
    config.wholeGroups = groups - groups % units;
    config.splits = std::clamp((units + (groups % units) / 2) / (groups % units), 1u, most);
    if (config.splits == 1) config.wholeGroups = 0;
  } else {
    // Rounded down: one workgroup past a full round costs a second round.
    config.splits = std::clamp(wanted / groups, 1u, most);
  }
  return LinearPlan(w, config, destination);
}

LinearPlan Linear::plan(const Projection &projection, uint32_t rows, LinearEpilogue epilogue) const {
  return plan(workloadOf(projection, rows, epilogue), epilogue == LinearEpilogue::None ? projection.destination : FloatOutput::BFloat16);
}

LinearScratchSize Linear::scratchSize(LinearMatrix matrix, uint32_t rows) const {
  LinearScratchSize size;
  for (LinearEpilogue e : {LinearEpilogue::None, LinearEpilogue::Residual, LinearEpilogue::GateUp})
    size.include(plan(LinearWorkload{matrix, rows, e}).scratchSize());
  if (matrix.outputSize % GGUF_BLOCK == 0)
    size.include(plan(LinearWorkload{matrix, rows, LinearEpilogue::ResidualNorm}).scratchSize());
  // segments of several formats partition every workgroup, however many the matrix has
  if (matrix.outputSize % 64 == 0)
    for (uint32_t format : {GGUF_FMT_Q4K, GGUF_FMT_Q6K})
      size.include(plan(LinearWorkload{matrix, rows, LinearEpilogue::None, format, true}).scratchSize());
  return size;
}

void Linear::addPrepare(hip::CommandGraph &graph, const hip::Buffer &input, const LinearScratch &scratch, uint32_t width,
                        uint32_t rows) {
  if (!rows || rows > kMaximumDispatchRows) throw std::invalid_argument("a block projection takes 1 to 256 rows");
  if (!width || width % GGUF_BLOCK) throw std::invalid_argument("block projections take whole 256-input super-blocks");
  const uint32_t tiles = gguf_row_tiles(rows);
  requireBytes(input, uint64_t{rows} * width * 2, "projection input");
  requireBytes(scratch.input, gguf_tables_bytes(width, tiles), "projection table");
  graph.add("gguf_prepare_table", {input, scratch.input}, GgufPrepareParams{width, rows, tiles, width},
            {width / 32, tiles, 1}, {64, 1, 1});
}

// One validated projection dispatch: what Linear::add hands the graph, and what a chain holds of each link.
struct Linear::Resolved {
  std::string kernel;
  std::array<hip::Buffer, 8> buffers;
  GgufDecodeParams params{};
  uint32_t items = 0, pieces = 1, groups = 0;
  uint32_t format = 0, epilogue = 0;
  bool mixed = false, prepared = false;
  PreparedInput after;
};

PreparedInput Linear::add(hip::CommandGraph &graph, LinearBuffers b, const Projection &p, const LinearPlan &plan,
                          const Projection *gate) const {
  const LinearWorkload w = plan.workload();
  if (plan.configuration().tile == LinearTile::GgufColumn) return addColumn(graph, std::move(b), p, plan, gate);
  const hip::Buffer input = b.input, table = b.scratch.input;
  const Resolved r = resolve(std::move(b), p, plan, gate);
  if (!r.prepared) addPrepare(graph, input, LinearScratch{table, {}, {}}, w.matrix.inputSize, w.rows);
  graph.add(r.kernel, {r.buffers.begin(), r.buffers.end()}, r.params, {r.items, r.pieces, 1}, {256, 1, 1});
  return r.after;
}

// The column tile: a dispatch a tensor, each of its own format, over the rows as they are (the reference's
// Linear::addGgufColumn, LinearGguf.cpp:508-520).
PreparedInput Linear::addColumn(hip::CommandGraph &graph, LinearBuffers b, const Projection &p, const LinearPlan &plan,
                                const Projection *gate) const {
  const LinearWorkload w = plan.workload();
  const auto [n, k] = w.matrix;
  requireSegments(p, w.matrix);
  const bool gateUp = w.epilogue == LinearEpilogue::GateUp, residual = w.epilogue == LinearEpilogue::Residual;
  if (gateUp != (gate != nullptr)) throw std::invalid_argument("a block gate/up plan takes a gate projection, no other does");
  if (gate) {
    requireSegments(*gate, w.matrix);
    if (p.blocks().segments.size() != 1 || gate->blocks().segments.size() != 1 ||
        gate->blocks().segments.front().formatId != p.blocks().segments.front().formatId)
      throw std::invalid_argument("a one-pass block gate/up takes single tensors of one format");
  }
  const bool float32 = plan.destination() == FloatOutput::Float32;
  requireBytes(b.input, uint64_t{w.rows} * k * 2, "projection input");
  requireBytes(b.output, uint64_t{w.rows} * n * (float32 ? 4 : 2), "projection output");
  if (residual) requireBytes(b.residual, uint64_t{w.rows} * n * 2, "projection residual");
  for (const QuantizedSegment &s : p.blocks().segments) {
    GgufColumnParams params{};
    params.rows = w.rows;
    params.input_size = k;
    params.out_stride = n;
    params.out_offset = s.columnOffset;
    const hip::Buffer &image = gate ? gate->blocks().segments.front().image : s.image;
    graph.add(std::string("gguf_column_") + s.name() + (gateUp ? "_g" : residual ? "_r" : float32 ? "_a_f32" : "_a"),
              {image, s.image, b.input, b.output, residual ? b.residual : b.output}, params, {s.outputSize / GGUF_TILE_COLUMNS, 1, 1},
              {512, 1, 1});
  }
  return {b.input, LinearInput::Plain};
}

Linear::Resolved Linear::resolve(LinearBuffers b, const Projection &p, const LinearPlan &plan, const Projection *gate) const {
  const LinearWorkload w = plan.workload();
  const LinearConfig c = plan.configuration();
  const auto [n, k] = w.matrix;
  // Everything is checked before anything is added.
  requireSegments(p, w.matrix);
  const bool mixed = workloadOf(p, w.rows, w.epilogue).severalFormats;
  if (mixed != w.severalFormats) throw std::invalid_argument("the plan is not of this projection's formats");
  if (mixed)
    for (const QuantizedSegment &s : p.blocks().segments)
      if (s.outputSize % 64) throw std::invalid_argument("segments of several formats hold whole 64-column workgroups");
  const bool gateUp = w.epilogue == LinearEpilogue::GateUp;
  if (gateUp != (gate != nullptr)) throw std::invalid_argument("a block gate/up plan takes a gate projection, no other does");
  if (gate) {
    requireSegments(*gate, w.matrix);
    if (p.blocks().segments.size() != 1 || gate->blocks().segments.size() != 1 ||
        gate->blocks().segments.front().formatId != p.blocks().segments.front().formatId)
      throw std::invalid_argument("a one-pass block gate/up takes single tensors of one format");
  }
  const uint32_t tiles = gguf_row_tiles(w.rows);
  const uint64_t outBytes = plan.destination() == FloatOutput::Float32 ? 4 : 2;
  requireBytes(b.output, uint64_t{w.rows} * n * outBytes, "projection output");
  const bool norms = w.epilogue == LinearEpilogue::ResidualNorm;
  if (w.epilogue == LinearEpilogue::Residual || norms) requireBytes(b.residual, uint64_t{w.rows} * n * 2, "projection residual");
  const LinearScratchSize need = plan.scratchSize();
  requireBytes(b.scratch.input, need.input, "projection table");
  if (c.splits > 1) {
    requireBytes(b.scratch.partials, need.partials, "projection partials");
    requireBytes(b.scratch.counters, need.counters, "projection counters");
  }
  if (norms) {
    if (p.blocks().segments.size() != 1) throw std::invalid_argument("a projection that norms its rows is one tensor");
    if (n % GGUF_BLOCK) throw std::invalid_argument("a table epilogue takes whole super-blocks of output columns");
    requireBytes(b.normWeight, uint64_t{n} * 2, "norm weight");
    requireBytes(b.nextTable, gguf_tables_bytes(n, gguf_row_tiles(w.rows)), "next projection table");
    if (b.nextTable.sameView(b.scratch.input)) throw std::invalid_argument("the next projection's table is not the plan's own");
  }
  const bool writesTable = gateUp && bool(b.nextTable);
  if (b.nextTable && !gateUp && !norms) throw std::invalid_argument("only a gate/up or a norming plan writes the next projection's table");
  if (writesTable) {
    if (n % GGUF_BLOCK) throw std::invalid_argument("a table epilogue takes whole super-blocks of output columns");
    requireBytes(b.nextTable, gguf_tables_bytes(n, tiles), "next projection table");
    if (b.nextTable.sameView(b.scratch.input)) throw std::invalid_argument("the next projection's table is not the plan's own");
  }
  const bool prepared = b.prepared.layout != LinearInput::Plain && b.prepared.source && b.input &&
                        b.prepared.source.sameView(b.input);
  if (!prepared) requireBytes(b.input, uint64_t{w.rows} * k * 2, "projection input");

  GgufDecodeParams params{};
  params.input_size = k;
  params.rows = w.rows;
  params.splits = c.splits;
  params.whole_groups = c.wholeGroups;
  params.out_stride = n;
  std::array<hip::Buffer, 3> images;
  const std::vector<QuantizedSegment> &segments = p.blocks().segments;
  if (gateUp) {
    images = {gate->blocks().segments.front().image, segments.front().image, segments.front().image};
    params.cols[0] = n;
    params.offset[0] = 0;
  } else {
    for (size_t s = 0; s < 3; ++s) {
      const QuantizedSegment &segment = segments[std::min(s, segments.size() - 1)];
      images[s] = segment.image;
      if (s < segments.size()) {
        params.cols[s] = segment.outputSize;
        params.offset[s] = segment.columnOffset;
        if (mixed) params.formats[s] = segment.formatId;
      }
    }
  }
  params.units = unitsOf(n, w.epilogue);
  params.deferred_scale = prepared && b.prepared.layout == LinearInput::TableUnscaled;
  // Unused bindings still name a buffer: the table stands in for them.
  const hip::Buffer &spare = b.scratch.input;
  const bool staged = c.tile == LinearTile::GgufStaged;
  const std::string name = std::string(staged ? "gguf_staged_" : "gguf_decode_") + (mixed ? "mixed" : segments.front().name()) + "_m" +
                           std::to_string(plan.storageRows()) + epilogueSuffix(w.epilogue, plan.destination(), writesTable);
  if (norms) {
    images[1] = b.normWeight;
    images[2] = b.nextTable;
  }
  Resolved r;
  r.kernel = name;
  r.buffers = {images[0], images[1], images[2], b.scratch.input, b.output,
               w.epilogue == LinearEpilogue::Residual || norms ? b.residual : writesTable ? b.nextTable : spare,
               c.splits > 1 ? b.scratch.partials : spare, c.splits > 1 ? b.scratch.counters : spare};
  r.params = params;
  r.groups = groupsOf(n, w.epilogue);
  r.items = c.wholeGroups + (r.groups - c.wholeGroups) * c.splits;
  r.pieces = rowPieces(w.rows);
  r.format = segments.front().formatId;
  r.epilogue = norms ? GGUF_EPILOGUE_RESIDUAL_NORM
               : gateUp ? (writesTable ? GGUF_EPILOGUE_GATE_UP_TABLE : GGUF_EPILOGUE_GATE_UP)
               : w.epilogue == LinearEpilogue::Residual ? GGUF_EPILOGUE_RESIDUAL
               : plan.destination() == FloatOutput::Float32 ? GGUF_EPILOGUE_PLAIN_F32 : GGUF_EPILOGUE_PLAIN;
  r.mixed = mixed;
  r.prepared = prepared;
  r.after = {b.input, prepared ? b.prepared.layout : LinearInput::Table16};
  (void)tiles;
  return r;
}

void Linear::addChain(hip::CommandGraph &graph, std::vector<ChainedProjection> links, const hip::Buffer &progress) const {
  if (links.empty() || links.size() > GGUF_CHAIN_LINKS) throw std::invalid_argument("a chain holds one to four projections");
  requireBytes(progress, GGUF_CHAIN_PROGRESS_WORDS * 4, "chain progress");
  GgufChainParams chain{};
  chain.links = uint32_t(links.size());
  chain.spin_limit = calibration_.chainSpinLimit;
  std::vector<hip::Buffer> buffers;
  std::vector<Resolved> resolved;
  const uint32_t storage = links.front().plan.storageRows();
  uint32_t items = 0;
  for (size_t i = 0; i < links.size(); ++i) {
    ChainedProjection &link = links[i];
    if (!link.projection) throw std::invalid_argument("a chain link names its projection");
    if (link.plan.storageRows() != storage || rowPieces(link.plan.workload().rows) != 1)
      throw std::invalid_argument("a chain's projections share one tile height of up to 64 rows");
    if (link.plan.configuration().tile != LinearTile::GgufMfma) throw std::invalid_argument("chained projections run the register rule");
    resolved.push_back(resolve(link.buffers, *link.projection, link.plan, link.gate));
    const Resolved &r = resolved.back();
    if (!r.prepared) throw std::invalid_argument("a chained projection reads a table that is already there or that the link before it writes");
    if (r.epilogue == GGUF_EPILOGUE_RESIDUAL || r.epilogue == GGUF_EPILOGUE_GATE_UP)
      throw std::invalid_argument("a chained projection is plain, a gate/up pair that writes the next table, or a residual one that norms its rows");
    // a link's table, partials and counters are its own, and nothing the dispatch has read is written later
    for (size_t j = 0; j < i; ++j) {
      const LinearBuffers &other = links[j].buffers;
      if (other.scratch.input.sameView(link.buffers.scratch.input)) throw std::invalid_argument("chained projections read tables of their own");
      if (link.plan.configuration().splits > 1 && links[j].plan.configuration().splits > 1 &&
          (other.scratch.partials.sameView(link.buffers.scratch.partials) || other.scratch.counters.sameView(link.buffers.scratch.counters)))
        throw std::invalid_argument("chained projections keep partials and counters of their own");
      if (link.buffers.nextTable && link.buffers.nextTable.sameView(other.scratch.input))
        throw std::invalid_argument("a chained projection writes no table an earlier link read");
    }
    GgufChainLink &out = chain.link[i];
    out.p = r.params;
    out.first_item = items;
    out.format = r.format;
    out.epilogue = r.epilogue;
    out.mixed = r.mixed;
    out.groups = r.groups;
    items += r.items;
    buffers.insert(buffers.end(), r.buffers.begin(), r.buffers.end());
  }
  // links past the last bind the first one's buffers and take no workgroup
  for (size_t i = links.size(); i < GGUF_CHAIN_LINKS; ++i) {
    chain.link[i].first_item = items;
    buffers.insert(buffers.end(), resolved.front().buffers.begin(), resolved.front().buffers.end());
  }
  buffers.push_back(progress);
  graph.add("gguf_decode_chain_m" + std::to_string(storage), std::move(buffers), chain, {items, 1, 1}, {256, 1, 1});
}

bool Linear::preparesAttention(const Projection &p, const LinearPlan &plan, const AttentionParams &a) noexcept {
  const LinearWorkload w = plan.workload();
  const uint32_t D = a.head_dim;
  if (w.epilogue != LinearEpilogue::None || plan.destination() != FloatOutput::BFloat16) return false;
  if (rowPieces(w.rows) != 1 || plan.configuration().wholeGroups || plan.configuration().tile != LinearTile::GgufMfma) return false;
  if ((D != 64 && D != 128) || a.gated || a.int8_queries || !a.kv_heads) return false;
  if (w.matrix.outputSize != (a.q_heads + 2 * a.kv_heads) * D || a.qkv_stride != w.matrix.outputSize) return false;
  if (!a.sequences || a.sequences > ATTENTION_MAXIMUM_SEQUENCES) return false;
  for (uint32_t s = 0; s < a.sequences; ++s)
    if (uint64_t{a.sequence[s].first_row} + a.sequence[s].rows > w.rows) return false;
  for (const QuantizedSegment &s : p.blocks().segments)
    if (s.outputSize % D || s.columnOffset % D) return false;
  return true;
}

LinearScratchSize Linear::attentionScratchSize(const LinearPlan &plan) noexcept {
  // [part][workgroup][4 waves][row tile][4][64 lanes] fp32 sums, and a counter a head (at most one a workgroup)
  const LinearWorkload w = plan.workload();
  const uint64_t groups = groupsOf(w.matrix.outputSize, w.epilogue), pieceTiles = plan.storageRows() / GGUF_ROW_TILE;
  LinearScratchSize size = plan.scratchSize();
  size.partials = plan.configuration().splits * groups * kWavesAcross * pieceTiles * 256u * sizeof(float);
  size.counters = groups * sizeof(uint32_t);
  return size;
}

PreparedInput Linear::addWithAttention(hip::CommandGraph &graph, LinearBuffers b, const Projection &p, const LinearPlan &plan,
                                       const AttentionPrepareBindings &attention) const {
  const LinearWorkload w = plan.workload();
  const AttentionParams &a = attention.params;
  const hip::Buffer input = b.input, table = b.scratch.input, partials = b.scratch.partials, counters = b.scratch.counters;
  const Resolved r = resolve(std::move(b), p, plan, nullptr);
  if (!preparesAttention(p, plan, a)) throw std::invalid_argument("no fused kernel prepares this attention block from this projection");
  const LinearScratchSize need = attentionScratchSize(plan);
  requireBytes(partials, need.partials, "projection partials");
  requireBytes(counters, need.counters, "projection counters");
  const uint32_t rows = w.rows, D = a.head_dim;
  if (a.normalize) {
    requireBytes(attention.queryNorm, D * 2, "query norm weight");
    requireBytes(attention.keyNorm, D * 2, "key norm weight");
  }
  if (a.rotary_pairs) {
    requireBytes(attention.ropeCos, uint64_t{rows} * a.rotary_pairs * 4, "RoPE cosine table");
    requireBytes(attention.ropeSin, uint64_t{rows} * a.rotary_pairs * 4, "RoPE sine table");
  }
  const uint64_t fused = uint64_t{a.sequences} * a.q_heads * 16;
  requireBytes(attention.queries, fused * D * 2, "staged queries");
  requireBytes(attention.querySums, fused * 4, "staged query sums");
  if (!attention.pageTable || !attention.pool) throw std::invalid_argument("the fused projection stores into the layer's pages");
  if (!r.prepared) addPrepare(graph, input, LinearScratch{table, {}, {}}, w.matrix.inputSize, rows);
  const hip::Buffer &spare = table;
  const std::string name = std::string("gguf_decode_qkv_") + (r.mixed ? "mixed" : p.blocks().segments.front().name()) + "_m" +
                           std::to_string(plan.storageRows());
  graph.add(name,
            {r.buffers[0], r.buffers[1], r.buffers[2], r.buffers[3], r.buffers[4], partials, counters,
             a.normalize ? attention.queryNorm : spare, a.normalize ? attention.keyNorm : spare,
             a.rotary_pairs ? attention.ropeCos : spare, a.rotary_pairs ? attention.ropeSin : spare, attention.queries,
             attention.querySums, attention.pageTable, attention.pool},
            GgufQkvParams{r.params, a}, {r.items, 1, 1}, {256, 1, 1});
  return r.after;
}

uint64_t Linear::prefillTableBytes(uint32_t inputSize, uint32_t rows) noexcept {
  return gguf_tables_bytes(inputSize, gguf_row_tiles(rows));
}

namespace {
hip::Buffer viewOf(const hip::Buffer &base, uint64_t offset, uint64_t length) {
  sp_buffer *raw = nullptr;
  hip::throwStatus(sp_buffer_view(base.handle(), offset, length, &raw));
  return hip::Buffer::adopt(raw);
}
} // namespace

void Linear::addPrefill(hip::CommandGraph &graph, const hip::Buffer &input, const Projection &p, const hip::Buffer &output,
                        const hip::Buffer &residual, const hip::Buffer &table, uint32_t rows) {
  const uint32_t n = p.outputSize, k = p.inputSize;
  if (!rows || rows > kMaximumPrefillRows) throw std::invalid_argument("a prefill chunk takes 1 to 16384 rows");
  requireSegments(p, {n, k});
  for (const QuantizedSegment &s : p.blocks().segments)
    if (s.outputSize % 128 || s.columnOffset % 16) throw std::invalid_argument("a prefill projection's tensors hold whole 128-column workgroups");
  const bool float32 = p.destination == FloatOutput::Float32;
  if (float32 && residual) throw std::invalid_argument("only a plain prefill projection writes fp32");
  requireBytes(input, uint64_t{rows} * k * 2, "projection input");
  requireBytes(output, uint64_t{rows} * n * (float32 ? 4 : 2), "projection output");
  if (residual) requireBytes(residual, uint64_t{rows} * n * 2, "projection residual");
  requireBytes(table, prefillTableBytes(k, rows), "projection tables");
  // the rows' tables, 256 rows (four 64-row pieces) a pass
  const uint64_t pieceBytes = gguf_table_bytes(k, GGUF_PIECE_TILES);
  for (uint32_t first = 0; first < rows; first += kMaximumDispatchRows) {
    const uint32_t count = std::min(kMaximumDispatchRows, rows - first);
    const uint64_t tableAt = uint64_t{first / GGUF_MAXIMUM_ROWS} * pieceBytes;
    addPrepare(graph, viewOf(input, uint64_t{first} * k * 2, uint64_t{count} * k * 2),
               LinearScratch{viewOf(table, tableAt, gguf_tables_bytes(k, gguf_row_tiles(count))), {}, {}}, k, count);
  }
  for (const QuantizedSegment &s : p.blocks().segments) {
    GgufPrefillParams params{};
    params.input_size = k;
    params.rows = rows;
    params.columns = s.outputSize;
    params.out_stride = n;
    params.out_offset = s.columnOffset;
    graph.add(std::string("gguf_prefill_") + s.name() + (residual ? "_r" : float32 ? "_a_f32" : "_a"),
              {s.image, table, output, residual ? residual : output}, params, {s.outputSize / 128, (rows + 127) / 128, 1}, {256, 1, 1});
  }
}

void Linear::addProjection(hip::CommandGraph &graph, hip::Buffer input, const Projection &projection, hip::Buffer output,
                           uint32_t rows, LinearScratch scratch) const {
  LinearBuffers buffers;
  buffers.input = std::move(input);
  buffers.output = std::move(output);
  buffers.scratch = std::move(scratch);
  add(graph, std::move(buffers), projection, plan(projection, rows));
}

void Linear::addResidualProjection(hip::CommandGraph &graph, hip::Buffer input, const Projection &projection,
                                   hip::Buffer residual, hip::Buffer output, uint32_t rows, LinearScratch scratch) const {
  LinearBuffers buffers;
  buffers.input = std::move(input);
  buffers.output = std::move(output);
  buffers.residual = std::move(residual);
  buffers.scratch = std::move(scratch);
  add(graph, std::move(buffers), projection, plan(projection, rows, LinearEpilogue::Residual));
}

bool Linear::normsRows(const Projection &projection, uint32_t rows) const noexcept {
  return rows && rows <= kMaximumDispatchRows && projection.blocks().segments.size() == 1 &&
         projection.outputSize % GGUF_BLOCK == 0;
}

void Linear::addSwiGlu(hip::CommandGraph &graph, const SwiGluProjections &ffn, const FfnBuffers &b, hip::Buffer residual,
                       hip::Buffer output, uint32_t rows, PreparedInput normalized) const {
  if (!ffn.gate || !ffn.up || !ffn.down) throw std::invalid_argument("a SwiGLU takes gate, up and down projections");
  LinearBuffers pair;
  pair.input = b.normalized;
  pair.output = b.intermediate;
  pair.scratch = b.scratch;
  pair.prepared = std::move(normalized);
  const LinearPlan pairPlan = plan(*ffn.up, rows, LinearEpilogue::GateUp);
  LinearBuffers down;
  down.input = b.intermediate;
  down.output = std::move(output);
  down.residual = std::move(residual);
  down.scratch = b.scratch;
  if (b.nextTable) {
    pair.nextTable = b.nextTable;
    down.scratch.input = b.nextTable;
    down.prepared = {b.intermediate, LinearInput::Table16};
  }
  const bool norms = bool(b.followingNorm);
  if (norms) {
    down.normWeight = b.followingNorm;
    down.nextTable = b.followingTable;
  }
  const LinearPlan downPlan = plan(*ffn.down, rows, norms ? LinearEpilogue::ResidualNorm : LinearEpilogue::Residual);
  add(graph, std::move(pair), *ffn.up, pairPlan, ffn.gate);
  add(graph, std::move(down), *ffn.down, downPlan);
}

} // namespace splash::ops
