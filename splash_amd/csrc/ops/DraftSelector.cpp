#include "ops/DraftSelector.hpp"

#include "abi/PagedAttention.h"  // AttentionTreeRow
#include "ops/Linear.hpp"        // requireBytes

#include <cmath>
#include <stdexcept>

namespace splash::ops {

void DraftSelector::addVerifyRows(hip::CommandGraph &graph, const DraftVerifyRowsBuffers &b, const StepRows &step, float floor) {
  if (!step.lanes || step.lanes > SAMPLING_MAXIMUM_LANES || !step.laneCap || step.laneCap > SAMPLING_MAXIMUM_ROWS ||
      step.rows < step.lanes || step.rows > uint64_t{step.lanes} * step.laneCap)
    throw std::invalid_argument("invalid decode step rows");
  if (!(floor >= 0.0f) || !std::isfinite(floor)) throw std::invalid_argument("invalid verify rows floor");
  const uint64_t treeRows = uint64_t{step.lanes} * SAMPLING_MAXIMUM_ROWS;
  requireBytes(b.treeTokens, treeRows * 4, "draft tree token");
  requireBytes(b.trees, treeRows * sizeof(AttentionTreeRow), "draft tree row");
  requireBytes(b.treeScores, treeRows * 8, "draft tree score");
  requireBytes(b.treeSizes, uint64_t{step.lanes} * 4, "draft tree size");
  requireBytes(b.inputTokens, uint64_t{step.rows} * 4, "verify input token");
  requireBytes(b.treeRows, uint64_t{step.rows} * sizeof(AttentionTreeRow), "verify tree row");
  requireBytes(b.laneRows, uint64_t{step.lanes} * sizeof(SamplingLaneRows), "verify lane rows");
  requireBytes(b.verifySources, uint64_t{step.rows} * 4, "verify source");
  graph.add("draft_verify_rows", {b.treeTokens, b.trees, b.treeScores, b.treeSizes, b.inputTokens, b.treeRows, b.laneRows, b.verifySources},
            VerifyRowsParams{step.lanes, step.rows, step.laneCap, floor}, {1, 1, 1}, {64, 1, 1});
}

} // namespace splash::ops
