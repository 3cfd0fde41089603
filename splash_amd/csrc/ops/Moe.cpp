#include "ops/Moe.hpp"
#include "ops/Linear.hpp"  // requireBytes

#include <stdexcept>
#include <string>

namespace splash::ops {

namespace {
constexpr uint32_t kMaximumRows = 256;  // rows of a step: eight lanes of sixteen and room to spare
void requireShape(const MoeShape &shape, uint32_t rows) {
  if (!shape.valid()) throw std::invalid_argument("invalid MoE shape");
  if (!rows || rows > kMaximumRows) throw std::invalid_argument("a MoE step takes 1 to 256 rows");
  // The grouping kernel's bit matrix, a row an expert and a bit a route, lives in one workgroup's LDS.
  if (uint64_t{shape.allExperts()} * ((uint64_t{rows} * shape.routesPerRow() + 31) / 32) > MOE_GROUP_WORDS)
    throw std::invalid_argument("too many experts for that many routes: experts * ceil(rows * routes a row / 32) is at most 16384");
}
const char *formatName(uint32_t format) {
  if (!gguf_record_bytes(format)) throw std::invalid_argument("no routed expert kernel for this format");
  return gguf_format_name(format);
}
} // namespace

MoeWorkspaceSize MoE::workspace(const MoeShape &shape, uint32_t rows) {
  requireShape(shape, rows);
  const uint64_t routes = uint64_t{rows} * shape.routesPerRow(), tiles = moe_maximum_tiles(uint32_t(routes), shape.allExperts()),
                 slots = tiles * MOE_TILE_ROWS;
  MoeWorkspaceSize s;
  s.selected = routes * 4;
  s.weights = routes * 4;
  s.routeSlot = routes * 4;
  s.slotRow = slots * 4;
  s.tileExpert = s.tileRows = tiles * 4;
  s.tileTotal = 16;
  s.tables = tiles * gguf_table_bytes(shape.hidden, 1);
  s.nextTables = tiles * gguf_table_bytes(shape.ffn, 1);
  s.intermediate = slots * shape.ffn * 2;
  s.expertOutput = slots * shape.hidden * 2;
  return s;
}

void MoE::addRouting(hip::CommandGraph &graph, const hip::Buffer &scores, uint32_t scoreStride, const MoeWorkspace &w,
                     const MoeShape &shape, uint32_t rows, const hip::Buffer &input, const hip::Buffer &sharedScalarGate) {
  requireShape(shape, rows);
  if (shape.sharedGate) {
    requireBytes(input, uint64_t{rows} * shape.hidden * 2, "router input rows");
    requireBytes(sharedScalarGate, uint64_t{shape.hidden} * 4, "shared expert gate");
  }
  if (scoreStride < shape.experts) throw std::invalid_argument("a row of scores holds every expert's");
  const MoeWorkspaceSize need = workspace(shape, rows);
  requireBytes(scores, (uint64_t{rows - 1} * scoreStride + shape.experts) * 4, "router scores");
  requireBytes(w.selected, need.selected, "selected experts");
  requireBytes(w.weights, need.weights, "routing weights");
  requireBytes(w.routeSlot, need.routeSlot, "route slots");
  requireBytes(w.slotRow, need.slotRow, "slot rows");
  requireBytes(w.tileExpert, need.tileExpert, "tile experts");
  requireBytes(w.tileRows, need.tileRows, "tile rows");
  requireBytes(w.tileTotal, 4, "tile count");
  const uint32_t routes = rows * shape.routesPerRow();
  graph.add("moe_route_select", {scores, shape.sharedGate ? input : scores, shape.sharedGate ? sharedScalarGate : scores, w.selected, w.weights},
            MoeRouteParams{rows, shape.experts, shape.topK, scoreStride, shape.sharedSlices, shape.sharedGate, shape.hidden, shape.sigmoidRouter}, {rows, 1, 1},
            {64, 1, 1});
  // The grouping and the combine take the shared slices as further experts and routes of a row.
  graph.add("moe_group_routes", {w.selected, w.routeSlot, w.slotRow, w.tileExpert, w.tileRows, w.tileTotal},
            MoeGroupParams{routes, shape.allExperts(), shape.routesPerRow(), moe_maximum_tiles(routes, shape.allExperts())}, {1, 1, 1},
            {1024, 1, 1});
}

void MoE::addRouted(hip::CommandGraph &graph, const hip::Buffer &normalized, const hip::Buffer &residual, const hip::Buffer &output,
                    const MoeExperts &experts, const MoeWorkspace &w, const MoeShape &shape, uint32_t rows,
                    const MoeFollowingNorm &following) {
  requireShape(shape, rows);
  const bool writesTable = bool(following.table);
  if (writesTable) {
    if (shape.hidden % GGUF_BLOCK) throw std::invalid_argument("a table epilogue takes whole super-blocks of columns");
    requireBytes(following.weight, uint64_t{shape.hidden} * 2, "norm weight");
    requireBytes(following.table, gguf_tables_bytes(shape.hidden, gguf_row_tiles(rows)), "next projection table");
  }
  const MoeWorkspaceSize need = workspace(shape, rows);
  const uint32_t routes = rows * shape.routesPerRow(), tiles = moe_maximum_tiles(routes, shape.allExperts());
  const std::string pairKernel = std::string("gguf_moe_decode_") + formatName(experts.format) + "_gt";
  const std::string downKernel = std::string("gguf_moe_decode_") + formatName(experts.downFormat) + "_a";
  const uint64_t pairBytes = gguf_image_bytes(experts.format, shape.ffn, shape.hidden);
  const uint64_t downBytes = gguf_image_bytes(experts.downFormat, shape.hidden, shape.ffn);
  requireBytes(normalized, uint64_t{rows} * shape.hidden * 2, "normalized rows");
  requireBytes(residual, uint64_t{rows} * shape.hidden * 2, "residual rows");
  requireBytes(output, uint64_t{rows} * shape.hidden * 2, "MoE output");
  requireBytes(experts.gate, pairBytes * shape.allExperts(), "expert gate images");
  requireBytes(experts.up, pairBytes * shape.allExperts(), "expert up images");
  requireBytes(experts.down, downBytes * shape.allExperts(), "expert down images");
  requireBytes(w.routeSlot, need.routeSlot, "route slots");
  requireBytes(w.slotRow, need.slotRow, "slot rows");
  requireBytes(w.tileExpert, need.tileExpert, "tile experts");
  requireBytes(w.tileRows, need.tileRows, "tile rows");
  requireBytes(w.tileTotal, 4, "tile count");
  requireBytes(w.weights, need.weights, "routing weights");
  requireBytes(w.tables, need.tables, "tile tables");
  requireBytes(w.nextTables, need.nextTables, "tile SwiGLU tables");
  requireBytes(w.intermediate, need.intermediate, "tile SwiGLU rows");
  requireBytes(w.expertOutput, need.expertOutput, "expert outputs");

  const uint64_t tableBytes = gguf_table_bytes(shape.hidden, 1), nextBytes = gguf_table_bytes(shape.ffn, 1);
  graph.add("moe_gather_table", {normalized, w.slotRow, w.tileTotal, w.tables}, MoeGatherParams{shape.hidden, tiles, tableBytes},
            {shape.hidden / 32, tiles, 1}, {64, 1, 1});
  GgufMoeParams pair{};
  pair.decode.input_size = shape.hidden;
  pair.decode.splits = 1;
  pair.decode.out_stride = shape.ffn;
  pair.decode.cols[0] = shape.ffn;
  pair.decode.units = 2 * (shape.ffn / GGUF_TILE_COLUMNS);
  pair.expert_bytes = pairBytes;
  pair.table_bytes = tableBytes;
  pair.next_table_bytes = nextBytes;
  pair.out_row_bytes = shape.ffn * 2;
  graph.add(pairKernel, {experts.gate, experts.up, w.tables, w.intermediate, w.nextTables, w.tileExpert, w.tileRows, w.tileTotal}, pair,
            {pair.decode.units / 4, tiles, 1}, {256, 1, 1});
  GgufMoeParams down{};
  down.decode.input_size = shape.ffn;
  down.decode.splits = 1;
  down.decode.out_stride = shape.hidden;
  down.decode.cols[0] = shape.hidden;
  down.decode.units = shape.hidden / GGUF_TILE_COLUMNS;
  down.expert_bytes = downBytes;
  down.table_bytes = nextBytes;
  down.next_table_bytes = 0;
  down.out_row_bytes = shape.hidden * 2;
  graph.add(downKernel, {experts.down, experts.down, w.nextTables, w.expertOutput, w.nextTables, w.tileExpert, w.tileRows, w.tileTotal}, down,
            {(down.decode.units + 3) / 4, tiles, 1}, {256, 1, 1});
  graph.add("moe_combine",
            {w.expertOutput, w.routeSlot, w.weights, residual, output, writesTable ? following.weight : output,
             writesTable ? following.table : output},
            MoeCombineParams{rows, shape.hidden, shape.routesPerRow(), writesTable ? gguf_row_tiles(rows) : 0u},
            {rows, (shape.hidden + 255) / 256, 1}, {256, 1, 1});
}

} // namespace splash::ops
