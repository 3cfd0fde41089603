// ops::GDN of the reference (runtime/ops/GDN.hpp:16-203, GDN.cpp:225-330) for the verify step: the
// decode step of up to eight lanes with its tape, the fold of a step's accepted rows alone, and the prompt
// chunk that builds the state a lane's first step starts from (GDN.hpp:75-104, :166-181), over kernels/gdn.hip.
#pragma once
#include "abi/Gdn.h"
#include "hip/Backend.hpp"

#include <vector>

namespace splash::ops {

struct GdnShape final {
  uint32_t keyHeads = 0, valueHeads = 0;
  uint32_t headDimension = GDN_HEAD_DIMENSION;
  uint32_t convolutionDimension = 0;
  uint32_t packedWidth = 0;
  bool sigmoidGate = false;
  [[nodiscard]] bool valid() const noexcept {
    return keyHeads && valueHeads && valueHeads % keyHeads == 0 && headDimension == GDN_HEAD_DIMENSION &&
           convolutionDimension == (2ull * keyHeads + valueHeads) * headDimension &&
           packedWidth >= convolutionDimension + uint64_t{valueHeads} * headDimension + 2ull * valueHeads;
  }
  [[nodiscard]] uint32_t kvWidth() const noexcept { return (keyHeads + valueHeads) * headDimension; }
  [[nodiscard]] GdnShapeParams params() const noexcept { return {keyHeads, valueHeads, convolutionDimension, packedWidth}; }
};
enum class GdnHeadOrder : uint8_t { Grouped, Tiled };

// A state cell's strides (GDN.hpp:63-73): fp32 recurrent states only.
struct GdnStateStrides final {
  uint64_t convolutionLayerBytes = 0, recurrentLayerBytes = 0, convolutionStateBytes = 0;
  [[nodiscard]] bool valid() const noexcept { return convolutionLayerBytes && recurrentLayerBytes && convolutionStateBytes; }
  // The strides of a cell of `layers` layers, and its size.
  static GdnStateStrides of(const GdnShape &shape, uint32_t layers) noexcept;
  [[nodiscard]] uint64_t cellBytes(uint32_t layers) const noexcept { return convolutionStateBytes + layers * recurrentLayerBytes; }
};
[[nodiscard]] uint64_t gdnTapeLayerBytes(const GdnShape &shape) noexcept;

// One lane of a step: its block of the step's rows, its tape slots (byte offsets of this layer's
// tapes in the tape buffer), the path of its previous step's rows its state does not hold yet, and
// its cells (byte offsets in the states buffer).
struct GdnLaneStep final {
  uint32_t firstRow = 0, rows = 0;
  uint32_t pendingPath = 0;
  uint64_t pendingTape = 0, stepTape = 0;
  uint64_t currentCell = 0, nextCell = 0;
};

struct GdnDecodeBuffers final {
  hip::Buffer packed;              // bf16 [rows][packedWidth]
  hip::Buffer convolutionWeights;  // bf16 [convolutionDimension][4]
  hip::Buffer states;              // the lanes' cells
  hip::Buffer tape;
  hip::Buffer decayWeights;        // fp32 [valueHeads]: a_scale
  hip::Buffer timeBias;            // bf16 [valueHeads]: dt_bias
  hip::Buffer mixerNorm;           // bf16 or fp32 [128]
  bool floatNorm = false;
  hip::Buffer hidden;              // bf16 [rows][valueHeads * 128]
  // The step's rows' places in their blocks' trees (AttentionTreeRow, a row each): every row reads the
  // state before the block along its own path, and its convolution reads its path's tokens (GDN.hpp:143-147).
  hip::Buffer tree;
  // Optional: the hidden rows also leave as the activation table (gguf_tables_bytes(valueHeads * 128, row tiles)) of
  // the projection that reads them, so no table pass runs before it.
  hip::Buffer hiddenTable{};
};
struct GdnFoldBuffers final {
  hip::Buffer states;
  hip::Buffer tape;
  hip::Buffer retainedRows;  // uint32: the row mask the step's acceptance wrote
  uint64_t stepTape = 0;     // the step's first layer's tape
  uint64_t stateCell = 0;    // the cell the step wrote
  uint64_t foldCell = 0;     // the cell the fold writes
};

// A prompt chunk of one lane and layer (GDN.hpp:75-93): the chunk's packed rows, the lane's cells, and the
// buffers of rows the three passes hand to each other. A chunk's rows all enter the state; nothing is taped.
struct GdnPrefillBuffers final {
  hip::Buffer packed;              // bf16 [tokens][packedWidth]
  hip::Buffer convolutionWeights;  // bf16 [convolutionDimension][4]
  hip::Buffer states;              // the cells
  hip::Buffer decayWeights;        // fp32 [valueHeads]
  hip::Buffer timeBias;            // bf16 [valueHeads]
  hip::Buffer mixerNorm;           // bf16 or fp32 [128]
  bool floatNorm = false;
  hip::Buffer queries, keys;       // bf16 [tokens][keyHeads * 128]: normalized, scaled
  hip::Buffer values;              // bf16 [tokens][valueHeads * 128]
  hip::Buffer decay;               // fp32 [tokens][valueHeads]
  hip::Buffer beta;                // bf16 [tokens][valueHeads]
  hip::Buffer recurrentRows;       // bf16 [tokens][valueHeads * 128]: the scan's outputs before the gated norm
  hip::Buffer hidden;              // bf16 [tokens][valueHeads * 128]
  uint64_t currentCell = 0;        // the cell the chunk starts from
  uint64_t nextCell = 0;           // the cell after its last row
};
// A state a chunk leaves on the way (GDN.hpp:95-104): the cell after its first `tokens` rows, convolution carry and
// recurrent state as a chunk ending there would leave them. What a cached state codes (ops::StateCodec) is such a cell.
struct GdnPrefillCapture final {
  uint32_t tokens = 0;
  uint64_t cell = 0;
};

class GDN final {
public:
  // A chunk of `tokens` rows of one lane, in runs that end at the captures (ascending, inside the rows): each run is
  // a prepare and a scan dispatch that continue from the cell the run before wrote, and one gate dispatch covers all
  // rows (GDN.cpp:176-222). The scan is sequential, so the runs compute bit for bit what one run computes.
  static void addPrefill(hip::CommandGraph &graph, const GdnPrefillBuffers &buffers, const GdnShape &shape, uint32_t layer,
                         uint32_t tokens, const GdnStateStrides &state, GdnHeadOrder order,
                         const std::vector<GdnPrefillCapture> &captures = {});
  // The step of 1 to 8 lanes of one layer.
  static void addDecode(hip::CommandGraph &graph, const GdnDecodeBuffers &buffers, const GdnShape &shape, uint32_t layer,
                        const GdnStateStrides &state, GdnHeadOrder order, const std::vector<GdnLaneStep> &lanes);
  // The state after the first `rows` rows of the path a lane retained of a step, in each of `layers` layers.
  static void addFold(hip::CommandGraph &graph, const GdnFoldBuffers &buffers, const GdnShape &shape, uint32_t layers, uint32_t rows,
                      const GdnStateStrides &state);
};

} // namespace splash::ops
