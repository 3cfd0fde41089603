// C shim of ops::MoE (include/splash_ops.h).
#include "capi/Guard.hpp"
#include "capi/Handles.hpp"
#include "ops/Moe.hpp"
#include "splash_ops.h"

using namespace splash;

namespace {
hip::Buffer B(sp_buffer *b) { return hip::Buffer::share(b); }
ops::MoeShape shapeOf(const spo_moe_shape &s) { return {s.hidden, s.ffn, s.experts, s.top_k, s.shared_slices, s.shared_gate != 0, s.sigmoid_router != 0}; }
ops::MoeWorkspace workspaceOf(const spo_moe_workspace &w) {
  return {B(w.selected), B(w.weights), B(w.route_slot), B(w.slot_row), B(w.tile_expert), B(w.tile_rows), B(w.tile_total), B(w.tables),
          B(w.next_tables), B(w.intermediate), B(w.expert_output)};
}
} // namespace

extern "C" {

sp_status spo_moe_workspace_sizes(const spo_moe_shape *shape, uint32_t rows, uint64_t sizes[11]) {
  return capi::guard([&] {
    capi::require(shape && sizes, "shape or result");
    const ops::MoeWorkspaceSize s = ops::MoE::workspace(shapeOf(*shape), rows);
    const uint64_t all[11] = {s.selected, s.weights, s.routeSlot, s.slotRow, s.tileExpert, s.tileRows, s.tileTotal, s.tables, s.nextTables,
                              s.intermediate, s.expertOutput};
    for (int i = 0; i < 11; ++i) sizes[i] = all[i];
  });
}

sp_status spo_moe_add_routing(spo_graph *graph, sp_buffer *scores, uint32_t score_stride, const spo_moe_workspace *workspace,
                              const spo_moe_shape *shape, uint32_t rows, sp_buffer *input, sp_buffer *shared_scalar_gate) {
  return capi::guard([&] {
    capi::require(graph && workspace && shape, "graph, workspace or shape");
    ops::MoE::addRouting(capi::graphOf(graph), B(scores), score_stride, workspaceOf(*workspace), shapeOf(*shape), rows,
                         input ? B(input) : hip::Buffer{}, shared_scalar_gate ? B(shared_scalar_gate) : hip::Buffer{});
  });
}

sp_status spo_moe_add_routed(spo_graph *graph, sp_buffer *normalized, sp_buffer *residual, sp_buffer *output, sp_buffer *gate_images,
                             sp_buffer *up_images, sp_buffer *down_images, uint32_t format, uint32_t down_format,
                             const spo_moe_workspace *workspace, const spo_moe_shape *shape, uint32_t rows) {
  return capi::guard([&] {
    capi::require(graph && workspace && shape, "graph, workspace or shape");
    ops::MoE::addRouted(capi::graphOf(graph), B(normalized), B(residual), B(output),
                        ops::MoeExperts{B(gate_images), B(up_images), B(down_images), format, down_format}, workspaceOf(*workspace),
                        shapeOf(*shape), rows);
  });
}

sp_status spo_moe_add_routed_norm(spo_graph *graph, sp_buffer *normalized, sp_buffer *residual, sp_buffer *output,
                                  sp_buffer *gate_images, sp_buffer *up_images, sp_buffer *down_images, uint32_t format,
                                  uint32_t down_format, const spo_moe_workspace *workspace, const spo_moe_shape *shape,
                                  uint32_t rows, sp_buffer *norm_weight, sp_buffer *next_table) {
  return capi::guard([&] {
    capi::require(graph && workspace && shape && norm_weight && next_table, "graph, workspace, shape, norm weight or table");
    ops::MoE::addRouted(capi::graphOf(graph), B(normalized), B(residual), B(output),
                        ops::MoeExperts{B(gate_images), B(up_images), B(down_images), format, down_format}, workspaceOf(*workspace),
                        shapeOf(*shape), rows, ops::MoeFollowingNorm{B(norm_weight), B(next_table)});
  });
}

} // extern "C"
