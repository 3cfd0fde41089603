// ops::MoE of the reference (runtime/ops/MoE.hpp:403-410, MoE.cpp:143-287) for the verify step:
// top-k routing of a block's rows, grouping of the routes by expert, the routed experts' SwiGLU
// and down projections on the grouped tiles, and the weighted sum back onto the residual stream.
#pragma once
#include "abi/Moe.h"
#include "hip/Backend.hpp"

namespace splash::ops {

struct MoeShape final {
  uint32_t hidden = 0, ffn = 0, experts = 0, topK = 0;
  // The shared expert is sharedSlices experts every row visits after its routed ones, ids experts to
  // experts + sharedSlices - 1, each of the routed experts' width (a shared expert sharedSlices times that wide is
  // their sum); with sharedGate each slice's weight is the sigmoid of the row's product with the block's scalar gate,
  // else 1 (the reference's MoeShape, runtime/ops/MoE.hpp:50-63). Their images follow the routed experts' in the
  // same buffers, in the same formats.
  uint32_t sharedSlices = 0;
  bool sharedGate = false;
  // The routed experts' weights: the softmax of the selected scores, or each one's sigmoid over the sum of theirs
  // (the reference's MoeRouter, moe.metal:21, :96-110).
  bool sigmoidRouter = false;
  [[nodiscard]] uint32_t routesPerRow() const noexcept { return topK + sharedSlices; }
  [[nodiscard]] uint32_t allExperts() const noexcept { return experts + sharedSlices; }
  [[nodiscard]] bool valid() const noexcept {
    return hidden && hidden % GGUF_BLOCK == 0 && ffn && ffn % GGUF_BLOCK == 0 && experts && allExperts() <= MOE_MAXIMUM_EXPERTS && topK &&
           routesPerRow() <= MOE_MAXIMUM_TOP && topK <= experts && sharedSlices <= 64 && (sharedSlices || !sharedGate);
  }
};
// Every expert's re-tiled image of a tensor, expert e at e * gguf_image_bytes(format, rows, inputs).
struct MoeExperts final {
  hip::Buffer gate, up, down;
  uint32_t format = GGUF_FMT_Q4K;      // of gate and up
  uint32_t downFormat = GGUF_FMT_Q4K;
};
// Bytes of the workspace buffers, in the order of MoeWorkspace's fields.
struct MoeWorkspaceSize final {
  uint64_t selected = 0, weights = 0, routeSlot = 0, slotRow = 0, tileExpert = 0, tileRows = 0, tileTotal = 0, tables = 0,
           nextTables = 0, intermediate = 0, expertOutput = 0;
};
struct MoeWorkspace final {
  hip::Buffer selected;      // uint32 [rows][topK]: the experts by rank
  hip::Buffer weights;       // fp32 [rows][topK]
  hip::Buffer routeSlot;     // uint32 [rows * topK]
  hip::Buffer slotRow;       // uint32 [maximum tiles * 16]
  hip::Buffer tileExpert, tileRows, tileTotal;
  hip::Buffer tables;        // the tiles' activation tables of the normalized rows
  hip::Buffer nextTables;    // and of the SwiGLU rows
  hip::Buffer intermediate;  // bf16 [slot][ffn]
  hip::Buffer expertOutput;  // bf16 [slot][hidden]
};

struct MoeFollowingNorm final {
  hip::Buffer weight;  // bf16 [hidden]
  hip::Buffer table;   // gguf_tables_bytes(hidden, row tiles)
};

class MoE final {
public:
  [[nodiscard]] static MoeWorkspaceSize workspace(const MoeShape &shape, uint32_t rows);
  // Selects and weighs each row's experts from its fp32 router scores ([rows][scoreStride]), appends the shape's shared
  // slices to every row's routes and groups the routes. `input` (the normalized rows, bf16 [rows][hidden]) and
  // `sharedScalarGate` (fp32 [hidden]) only for a gated shared expert (MoE.hpp:410-416 in the reference).
  static void addRouting(hip::CommandGraph &graph, const hip::Buffer &scores, uint32_t scoreStride, const MoeWorkspace &workspace,
                         const MoeShape &shape, uint32_t rows, const hip::Buffer &input = {}, const hip::Buffer &sharedScalarGate = {});
  // output = bf16(residual + sum over a row's routes of weight * down(silu(gate x) * up x)) of its experts, x = normalized.
  // `following` (optional): the output rows also leave as the activation table of the projection after their RMS
  // norm under following.weight, as a LinearEpilogue::ResidualNorm plan writes it (that projection reads it as
  // LinearInput::TableUnscaled).
  static void addRouted(hip::CommandGraph &graph, const hip::Buffer &normalized, const hip::Buffer &residual, const hip::Buffer &output,
                        const MoeExperts &experts, const MoeWorkspace &workspace, const MoeShape &shape, uint32_t rows,
                        const MoeFollowingNorm &following = {});
};

} // namespace splash::ops
