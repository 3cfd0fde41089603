#include "ops/PagedAttention.hpp"
#include "ops/Linear.hpp"  // requireBytes

#include <algorithm>
#include <stdexcept>
#include <string>

namespace splash::ops {

AttentionSplits attentionSplits(uint64_t tokens) noexcept {
  // About 64 splits of a long history, whole 64-token steps each (a page holds whole steps, so no
  // step straddles two pages): with 8 KV heads that is two workgroups per compute unit whatever the
  // length; a split holds at least four steps (a page's worth), below which its fixed cost outweighs it.
  const uint64_t steps = std::max<uint64_t>(1, (tokens + ATTENTION_STEP_TOKENS - 1) / ATTENTION_STEP_TOKENS);
  AttentionSplits s;
  constexpr uint64_t kSplits = 64;
  s.stepsPerSplit = uint32_t(std::max<uint64_t>(4, (steps + kSplits - 1) / kSplits));
  s.splits = uint32_t((steps + s.stepsPerSplit - 1) / s.stepsPerSplit);
  return s;
}

namespace {
std::string kernelSuffix(const AttentionGeometry &g) { return "_d" + std::to_string(g.headDimension); }
bool compiled(const AttentionGeometry &g) {
  return (g.headDimension == 128 && (g.group() == 8 || g.group() == 4)) || (g.headDimension == 64 && g.group() == 2);
}
uint32_t totalRows(const std::vector<AttentionRows> &sequences) {
  uint32_t rows = 0;
  for (const AttentionRows &s : sequences) rows = std::max(rows, s.firstRow + s.rows);
  return rows;
}
void requirePages(const AttentionPlan &plan, const KvPages &pages) {
  const uint64_t need = plan.geometry().layout().bytesPerLayerPage();
  if (pages.pageBytes < need || pages.pageBytes % 16) throw std::invalid_argument("KV page stride is smaller than a page or unaligned");
  if (!pages.pool || pages.pool.sizeBytes() < pages.pageBytes) throw std::invalid_argument("KV pool buffer is too small");
  uint64_t entries = 0;
  for (const AttentionRows &s : plan.sequences())
    entries = std::max<uint64_t>(entries, uint64_t{s.tableFirst} + kv::Layout::pagesFor(uint64_t{s.committed} + s.rows));
  requireBytes(pages.pageTable, entries * 8, "KV page table");
}
} // namespace

AttentionWorkspaceSize AttentionPlan::workspace() const noexcept {
  const uint64_t fused = uint64_t{sequences_.size()} * geometry_.kvHeads * geometry_.group() * 16;
  AttentionWorkspaceSize size;
  size.queries = fused * geometry_.headDimension * 2;
  size.querySums = fused * 4;
  size.partials = fused * splits_ * geometry_.headDimension * 2;
  size.partialSums = fused * splits_ * 8;
  return size;
}

AttentionParams AttentionPlan::params(uint64_t pageBytes) const noexcept {
  AttentionParams p{};
  p.q_heads = geometry_.qHeads;
  p.kv_heads = geometry_.kvHeads;
  p.head_dim = geometry_.headDimension;
  p.rotary_pairs = geometry_.rotaryPairs;
  p.normalize = geometry_.normalize;
  p.qkv_stride = geometry_.packedWidth();
  p.gated = geometry_.gated;
  p.int8_queries = geometry_.int8Queries;
  p.splits = splits_;
  p.sequences = uint32_t(sequences_.size());
  p.page_bytes = pageBytes;
  for (size_t i = 0; i < sequences_.size(); ++i)
    p.sequence[i] = {sequences_[i].firstRow, sequences_[i].committed, sequences_[i].tableFirst, uint16_t(sequences_[i].rows),
                     uint16_t(partition_[i].stepsPerSplit)};
  return p;
}

AttentionPlan PagedAttention::plan(const AttentionGeometry &geometry, std::vector<AttentionRows> sequences) {
  if (!geometry.kvHeads || geometry.qHeads % geometry.kvHeads || !compiled(geometry))
    throw std::invalid_argument("no attention kernel for this head geometry");
  if (2 * geometry.rotaryPairs > geometry.headDimension) throw std::invalid_argument("the rotated pairs are dimensions of the head");
  if (sequences.empty() || sequences.size() > ATTENTION_MAXIMUM_SEQUENCES)
    throw std::invalid_argument("an attention dispatch takes 1 to 8 sequences");
  AttentionPlan plan;
  plan.geometry_ = geometry;
  for (const AttentionRows &s : sequences) {
    if (!s.rows || s.rows > ATTENTION_MAXIMUM_ROWS) throw std::invalid_argument("a sequence's verify block holds 1 to 16 rows");
    const AttentionSplits part = attentionSplits(uint64_t{s.committed} + s.rows);
    if (part.splits > ATTENTION_MAXIMUM_SPLITS || part.stepsPerSplit > 0xFFFF)
      throw std::invalid_argument("the sequence is longer than the attention kernels split");
    plan.partition_.push_back(part);
    plan.splits_ = std::max(plan.splits_, part.splits);
  }
  plan.sequences_ = std::move(sequences);
  return plan;
}

void PagedAttention::addProjection(hip::CommandGraph &graph, const AttentionPlan &plan, const AttentionProjectionBuffers &b,
                                   const AttentionWorkspace &w, const KvPages &pages) {
  const AttentionGeometry &g = plan.geometry();
  const uint32_t rows = totalRows(plan.sequences());
  requireBytes(b.qkv, uint64_t{rows} * g.packedWidth() * 2, "attention qkv");
  if (g.normalize) {
    requireBytes(b.queryNorm, g.headDimension * 2, "query norm weight");
    requireBytes(b.keyNorm, g.headDimension * 2, "key norm weight");
  }
  if (g.rotaryPairs) {
    requireBytes(b.ropeCos, uint64_t{rows} * g.rotaryPairs * 4, "RoPE cosine table");
    requireBytes(b.ropeSin, uint64_t{rows} * g.rotaryPairs * 4, "RoPE sine table");
  }
  const AttentionWorkspaceSize need = plan.workspace();
  requireBytes(w.queries, need.queries, "staged queries");
  requireBytes(w.querySums, need.querySums, "staged query sums");
  requirePages(plan, pages);
  // Unused bindings still name a buffer.
  const hip::Buffer &spare = b.qkv;
  graph.add("attention_q8_qkv" + kernelSuffix(g),
            {b.qkv, g.normalize ? b.queryNorm : spare, g.normalize ? b.keyNorm : spare, g.rotaryPairs ? b.ropeCos : spare,
             g.rotaryPairs ? b.ropeSin : spare, w.queries, w.querySums, pages.pageTable, pages.pool},
            plan.params(pages.pageBytes), {g.qHeads + g.kvHeads, ATTENTION_MAXIMUM_ROWS, plan.sequences().size()},
            {g.headDimension, 1, 1});
}

bool PagedAttention::fusesProjection(const AttentionPlan &plan, const Projection &projection, const LinearPlan &linearPlan) noexcept {
  return linearPlan.workload().rows == totalRows(plan.sequences()) && Linear::preparesAttention(projection, linearPlan, plan.params(0));
}

PreparedInput PagedAttention::addFusedProjection(hip::CommandGraph &graph, const Linear &linear, LinearBuffers linearBuffers,
                                                 const Projection &projection, const LinearPlan &linearPlan, const AttentionPlan &plan,
                                                 const AttentionProjectionBuffers &b, const AttentionWorkspace &w, const KvPages &pages) {
  if (!fusesProjection(plan, projection, linearPlan)) throw std::invalid_argument("no fused kernel prepares this attention block from this projection");
  if (!b.qkv.sameView(linearBuffers.output)) throw std::invalid_argument("the fused projection writes the block's packed rows");
  const AttentionWorkspaceSize need = plan.workspace();
  requireBytes(w.queries, need.queries, "staged queries");
  requireBytes(w.querySums, need.querySums, "staged query sums");
  requirePages(plan, pages);
  return linear.addWithAttention(graph, std::move(linearBuffers), projection, linearPlan,
                                 AttentionPrepareBindings{b.queryNorm, b.keyNorm, b.ropeCos, b.ropeSin, w.queries, w.querySums,
                                                          pages.pageTable, pages.pool, plan.params(pages.pageBytes)});
}

void PagedAttention::addAttention(hip::CommandGraph &graph, const AttentionPlan &plan, const AttentionWorkspace &w,
                                  const hip::Buffer &treeRows, const KvPages &pages, const hip::Buffer &output,
                                  const hip::Buffer &outputTable, const hip::Buffer &packed, uint32_t tableRows) {
  const AttentionGeometry &g = plan.geometry();
  const uint32_t rows = totalRows(plan.sequences());
  if (tableRows && tableRows < rows) throw std::invalid_argument("the output table holds the dispatch's rows");
  const AttentionWorkspaceSize need = plan.workspace();
  requireBytes(w.queries, need.queries, "staged queries");
  requireBytes(w.querySums, need.querySums, "staged query sums");
  requireBytes(w.partials, need.partials, "attention partials");
  requireBytes(w.partialSums, need.partialSums, "attention partial sums");
  requireBytes(treeRows, uint64_t{rows} * sizeof(AttentionTreeRow), "verify tree rows");
  requireBytes(output, uint64_t{rows} * g.qHeads * g.headDimension * 2, "attention output");
  if (g.gated) requireBytes(packed, uint64_t{rows} * g.packedWidth() * 2, "attention qkv (the gates)");
  requirePages(plan, pages);
  AttentionParams params = plan.params(pages.pageBytes);
  const uint32_t width = g.qHeads * g.headDimension;
  if (outputTable) {
    if (width % GGUF_BLOCK) throw std::invalid_argument("an attention output table holds whole super-blocks");
    params.table_tiles = gguf_row_tiles(tableRows ? tableRows : rows);
    requireBytes(outputTable, gguf_tables_bytes(width, params.table_tiles), "attention output table");
  }
  graph.add(std::string(g.int8Queries ? "attention_q8q_split" : "attention_q8_split") + kernelSuffix(g) + "_g" + std::to_string(g.group()),
            {w.queries, w.querySums, treeRows, pages.pageTable, pages.pool, w.partials, w.partialSums}, params,
            {g.kvHeads, plan.splits(), plan.sequences().size()}, {256, 1, 1});
  graph.add("attention_reduce" + kernelSuffix(g) + (outputTable ? "_t" : ""),
            {w.partials, w.partialSums, output, outputTable ? outputTable : output, g.gated ? packed : output}, params,
            {g.qHeads, ATTENTION_MAXIMUM_ROWS, plan.sequences().size()}, {256, 1, 1});
}

AttentionWorkspaceSize AttentionChunkPlan::workspace() const noexcept {
  AttentionWorkspaceSize size;
  for (const AttentionPlan &plan : dispatches_) {
    const AttentionWorkspaceSize one = plan.workspace();
    size.queries += one.queries;
    size.querySums += one.querySums;
    size.partials = std::max(size.partials, one.partials);
    size.partialSums = std::max(size.partialSums, one.partialSums);
  }
  return size;
}

AttentionChunkPlan PagedAttention::planChunks(const AttentionGeometry &geometry, const std::vector<AttentionChunk> &chunks) {
  if (chunks.empty()) throw std::invalid_argument("a chunked attention takes at least one chunk");
  std::vector<AttentionRows> tiles;
  AttentionChunkPlan plan;
  plan.geometry_ = geometry;
  for (const AttentionChunk &chunk : chunks) {
    if (!chunk.tokens || chunk.tokens > kMaximumChunkRows) throw std::invalid_argument("a prompt chunk holds 1 to 2048 rows");
    if (chunk.firstRow < plan.rows_) throw std::invalid_argument("the chunks' rows ascend and do not overlap");
    for (uint32_t first = 0; first < chunk.tokens; first += ATTENTION_MAXIMUM_ROWS)
      tiles.push_back({chunk.firstRow + first, std::min<uint32_t>(ATTENTION_MAXIMUM_ROWS, chunk.tokens - first), chunk.committed + first,
                       chunk.tableFirst});
    plan.rows_ = chunk.firstRow + chunk.tokens;
  }
  plan.tiles_ = uint32_t(tiles.size());
  for (size_t first = 0; first < tiles.size(); first += ATTENTION_MAXIMUM_SEQUENCES)
    plan.dispatches_.push_back(PagedAttention::plan(
        geometry, {tiles.begin() + first, tiles.begin() + std::min(tiles.size(), first + ATTENTION_MAXIMUM_SEQUENCES)}));
  return plan;
}

namespace {
// Dispatch d's part of a chunk plan's workspace: its tiles' staged queries after those of the dispatches before it.
AttentionWorkspace workspaceOf(const AttentionChunkPlan &plan, const AttentionWorkspace &all, size_t d) {
  uint64_t queries = 0, sums = 0;
  for (size_t i = 0; i < d; ++i) {
    const AttentionWorkspaceSize before = plan.dispatches()[i].workspace();
    queries += before.queries;
    sums += before.querySums;
  }
  const AttentionWorkspaceSize mine = plan.dispatches()[d].workspace();
  AttentionWorkspace w = all;
  w.queries = all.queries.slice(queries, mine.queries);
  w.querySums = all.querySums.slice(sums, mine.querySums);
  return w;
}
void requireChunkWorkspace(const AttentionChunkPlan &plan, const AttentionWorkspace &w, bool attends) {
  const AttentionWorkspaceSize need = plan.workspace();
  requireBytes(w.queries, need.queries, "staged queries");
  requireBytes(w.querySums, need.querySums, "staged query sums");
  if (attends) {
    requireBytes(w.partials, need.partials, "attention partials");
    requireBytes(w.partialSums, need.partialSums, "attention partial sums");
  }
}
} // namespace

void PagedAttention::addChunkProjection(hip::CommandGraph &graph, const AttentionChunkPlan &plan, const AttentionProjectionBuffers &buffers,
                                        const AttentionWorkspace &workspace, const KvPages &pages) {
  requireChunkWorkspace(plan, workspace, false);
  for (size_t d = 0; d < plan.dispatches().size(); ++d)
    addProjection(graph, plan.dispatches()[d], buffers, workspaceOf(plan, workspace, d), pages);
}

void PagedAttention::addChunkAttention(hip::CommandGraph &graph, const AttentionChunkPlan &plan, const AttentionWorkspace &workspace,
                                       const hip::Buffer &treeRows, const KvPages &pages, const hip::Buffer &output,
                                       const hip::Buffer &outputTable, const hip::Buffer &packed) {
  requireChunkWorkspace(plan, workspace, true);
  // every dispatch writes its rows of the one table of all the rows
  if (outputTable)
    requireBytes(outputTable, gguf_tables_bytes(plan.geometry().qHeads * plan.geometry().headDimension, gguf_row_tiles(plan.rows())),
                 "attention output table");
  for (size_t d = 0; d < plan.dispatches().size(); ++d)
    addAttention(graph, plan.dispatches()[d], workspaceOf(plan, workspace, d), treeRows, pages, output, outputTable, packed, plan.rows());
}

void PagedAttention::addPathCommit(hip::CommandGraph &graph, const AttentionPlan &plan, const hip::Buffer &retained,
                                   const KvPages &pages, uint32_t layers, uint64_t layerBytes) {
  const AttentionGeometry &g = plan.geometry();
  requireBytes(retained, plan.sequences().size() * 4, "retained rows");
  requirePages(plan, pages);
  if (!layers || (layers > 1 && (layerBytes < pages.pageBytes || pages.pool.sizeBytes() < layerBytes * layers)))
    throw std::invalid_argument("KV pool buffer does not hold the layers' pools");
  const AttentionParams full = plan.params(pages.pageBytes);
  AttentionCommitParams params{};
  params.kv_heads = g.kvHeads;
  params.head_dim = g.headDimension;
  params.sequences = full.sequences;
  params.layers = layers;
  params.page_bytes = pages.pageBytes;
  params.layer_bytes = layerBytes;
  for (uint32_t i = 0; i < full.sequences; ++i) params.sequence[i] = full.sequence[i];
  graph.add("attention_q8_commit" + kernelSuffix(g), {retained, pages.pageTable, pages.pool}, params,
            {g.kvHeads, plan.sequences().size(), layers}, {g.headDimension, 1, 1});
}

} // namespace splash::ops
