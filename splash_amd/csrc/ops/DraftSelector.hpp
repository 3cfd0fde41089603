// The draft side's last step before the verify path: laying a decode step's rows out from the trees a draft selector
// grew. The counterpart of ops::DraftSelector::addVerifyRows (runtime/ops/DraftSelector.hpp:139-147) and StepRows
// (runtime/ops/LaneRows.hpp:49-67); the selector's scoring kernels (top-16 candidates, edge scores, tree growth) are not
// part of this library.
#pragma once
#include "abi/Sampling.h"
#include "hip/Backend.hpp"

#include <cstdint>

namespace splash::ops {

// A decode step's rows: `rows` rows over `lanes` lanes, packed in lane order, each lane 1 to `laneCap` of them.
struct StepRows final {
  uint32_t lanes = 0;
  uint32_t rows = 0;
  uint32_t laneCap = 0;
};

struct DraftVerifyRowsBuffers final {
  // Each lane's tree, 16 rows a lane, in the order the selector took them, best first:
  hip::Buffer treeTokens;   // uint32 [lanes][16]
  hip::Buffer trees;        // AttentionTreeRow [lanes][16]
  hip::Buffer treeScores;   // fp32 [lanes][16][2]: a row's draft probability and its estimate
  hip::Buffer treeSizes;    // uint32 [lanes]: the rows each tree holds
  // The step's rows as the verify path reads them:
  hip::Buffer inputTokens;    // uint32 [rows]
  hip::Buffer treeRows;       // AttentionTreeRow [rows]
  hip::Buffer laneRows;       // {first, rows} [lanes]
  hip::Buffer verifySources;  // uint32 [rows]: the row of its lane's tree each row is, SAMPLING_NO_TOKEN for a row of no lane
};

class DraftSelector final {
public:
  // The trees' best rows that the step's rows and its lane cap hold, none past an anchor estimated below `floor`, each
  // lane's numbered in preorder, and the step's rows past them of no lane.
  static void addVerifyRows(hip::CommandGraph &graph, const DraftVerifyRowsBuffers &buffers, const StepRows &step, float floor = 0.0f);
};

} // namespace splash::ops
