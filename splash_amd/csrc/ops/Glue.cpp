#include "ops/Glue.hpp"

#include <string>

#include <stdexcept>

namespace splash::ops {

namespace {
void requireNorm(const hip::Buffer &input, const hip::Buffer &weight, const hip::Buffer &output, uint32_t width, uint32_t rows) {
  if (!width || !rows) throw std::invalid_argument("a norm takes rows of a width");
  requireBytes(input, uint64_t{rows} * width * 2, "norm input");
  requireBytes(weight, uint64_t{width} * 2, "norm weight");
  requireBytes(output, uint64_t{rows} * width * 2, "norm output");
}
} // namespace

void Normalization::addRms(hip::CommandGraph &graph, const hip::Buffer &input, const hip::Buffer &weight, const hip::Buffer &output,
                           uint32_t width, uint32_t rows) {
  requireNorm(input, weight, output, width, rows);
  graph.add("norm_rms", {input, weight, output}, NormParams{width, rows, 0, 0}, {rows, 1, 1}, {256, 1, 1});
}

PreparedInput Normalization::addRmsTable(hip::CommandGraph &graph, const hip::Buffer &input, const hip::Buffer &weight,
                                         const hip::Buffer &output, const LinearScratch &scratch, uint32_t width, uint32_t rows) {
  requireNorm(input, weight, output, width, rows);
  if (width % GGUF_BLOCK || rows > kMaximumDispatchRows)
    throw std::invalid_argument("the activation table takes up to 256 rows of whole 256-input super-blocks");
  const uint32_t tiles = gguf_row_tiles(rows);
  requireBytes(scratch.input, gguf_tables_bytes(width, tiles), "projection table");
  graph.add("norm_rms_table16", {input, weight, output, scratch.input}, NormParams{width, rows, tiles, 0},
            {tiles * GGUF_ROW_TILE, 1, 1}, {256, 1, 1});
  return {output, LinearInput::Table16};
}

void Embedding::add(hip::CommandGraph &graph, const EmbeddingTable &table, const hip::Buffer &tokens, const hip::Buffer &output,
                    uint32_t rows) {
  if (!gguf_native_bytes(table.formatId)) throw std::invalid_argument("no token gather for this table format");
  if (!rows || !table.hidden || table.hidden % GGUF_BLOCK || !table.vocabulary)
    throw std::invalid_argument("a token table holds whole native blocks");
  requireBytes(table.rows, uint64_t{table.vocabulary} * (table.hidden / GGUF_BLOCK) * gguf_native_bytes(table.formatId), "token table");
  requireBytes(tokens, uint64_t{rows} * 4, "input tokens");
  requireBytes(output, uint64_t{rows} * table.hidden * 2, "embedding output");
  graph.add(std::string("gguf_embed_") + gguf_format_name(table.formatId), {table.rows, tokens, output},
            GgufEmbedParams{rows, table.vocabulary, table.hidden}, {rows, table.hidden / GGUF_BLOCK, 1}, {64, 1, 1});
}

void FloatProjection::add(hip::CommandGraph &graph, const hip::Buffer &input, const FloatRows &w, const hip::Buffer &output, uint32_t rows,
                          uint32_t outStride, uint32_t outOffset, FloatOutput type) {
  if (!rows || !w.inputSize || w.inputSize % 8 || !w.outputSize || uint64_t{outOffset} + w.outputSize > outStride)
    throw std::invalid_argument("invalid float projection");
  requireBytes(w.rows, w.weightBytes(), "float projection weight");
  requireBytes(input, uint64_t{rows} * w.inputSize * 2, "float projection input");
  const uint64_t element = type == FloatOutput::Float32 ? 4 : 2;
  requireBytes(output, (uint64_t{rows - 1} * outStride + outOffset + w.outputSize) * element, "float projection output");
  graph.add(std::string("gguf_float_") + (w.bfloat16 ? "bf16" : "f32") + (type == FloatOutput::Float32 ? "_f32" : "_bf16"),
            {input, w.rows, output}, GgufFloatParams{rows, w.inputSize, w.outputSize, outStride, outOffset, {}},
            {(w.outputSize + 15) / 16, (rows + 15) / 16, 1}, {256, 1, 1});
}

void RoPE::addTreeTables(hip::CommandGraph &graph, const hip::Buffer &inverseFrequency, const hip::Buffer &depth,
                         const hip::Buffer &cosines, const hip::Buffer &sines, uint32_t pairs,
                         const std::vector<RopeSequence> &sequences) {
  if (!pairs || pairs > 1024) throw std::invalid_argument("RoPE tables take 1 to 1024 pairs");
  if (sequences.empty() || sequences.size() > 8) throw std::invalid_argument("RoPE tables take 1 to 8 sequences");
  RopeTreeParams params{};
  params.pairs = pairs;
  params.sequences = uint32_t(sequences.size());
  for (size_t i = 0; i < sequences.size(); ++i) {
    params.first_row[i] = sequences[i].firstRow;
    params.row_count[i] = sequences[i].rows;
    params.anchor[i] = sequences[i].anchor;
    params.rows = std::max(params.rows, sequences[i].firstRow + sequences[i].rows);
  }
  requireBytes(inverseFrequency, uint64_t{pairs} * 4, "RoPE inverse frequencies");
  requireBytes(depth, uint64_t{params.rows} * 4, "row depths");
  requireBytes(cosines, uint64_t{params.rows} * pairs * 4, "RoPE cosine table");
  requireBytes(sines, uint64_t{params.rows} * pairs * 4, "RoPE sine table");
  graph.add("rope_build_tree_tables", {inverseFrequency, depth, cosines, sines}, params, {params.rows, 1, 1}, {pairs, 1, 1});
}

void SwiGlu::add(hip::CommandGraph &graph, const hip::Buffer &gate, const hip::Buffer &up, const hip::Buffer &output, uint64_t count) {
  if (!count || count % 8) throw std::invalid_argument("a SwiGLU pass takes whole vectors of eight values");
  requireBytes(gate, count * 2, "SwiGLU gate rows");
  requireBytes(up, count * 2, "SwiGLU up rows");
  requireBytes(output, count * 2, "SwiGLU rows");
  graph.add("swiglu_rows", {gate, up, output}, SwiGluRowsParams{count}, {(count / 8 + 255) / 256, 1, 1}, {256, 1, 1});
}

void RowCopy::add(hip::CommandGraph &graph, const hip::Buffer &source, RowRegion from, const hip::Buffer &destination, RowRegion to,
                  uint32_t rows, uint32_t width) {
  if (!rows || !width || from.column + uint64_t{width} > from.stride || to.column + uint64_t{width} > to.stride)
    throw std::invalid_argument("invalid row copy");
  auto regionBytes = [&](RowRegion r) { return ((uint64_t{r.row} + rows - 1) * r.stride + r.column + width) * 2; };
  requireBytes(source, regionBytes(from), "row copy source");
  requireBytes(destination, regionBytes(to), "row copy destination");
  graph.add("copy_rows_bf16", {source, destination},
            RowCopyParams{rows, width, from.row, from.stride, from.column, to.row, to.stride, to.column},
            {uint32_t((uint64_t{rows} * width + 255) / 256), 1, 1}, {256, 1, 1});
}

} // namespace splash::ops
