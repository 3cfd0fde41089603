// What a completed verify step left in its result buffers, checked before a caller commits anything
// (the reference's Runtime::finalizeDecode, runtime/model/Runtime.cpp:2943-2972, and
// invalidSelection, :1559-1582).
#pragma once
#include "hip/Backend.hpp"

#include <cstdint>
#include <string>
#include <vector>

namespace splash::model {

// One lane of a step: where its rows start among the packed rows, how many it has and how many
// tokens it may still keep.
struct StepLane final {
  uint32_t first = 0;
  uint32_t rows = 0;
  uint32_t remaining = 0xFFFFFFFFu;
};

// A lane's results as read back: tokens points at the lane's first packed row.
struct StepLaneResult final {
  uint32_t retained = 0;      // tokens kept: the accepted draft tokens and the target's next one
  uint32_t accepted = 0;      // draft tokens accepted
  uint32_t retainedRows = 0;  // mask of the lane's rows on the kept path, bit r for its row r
  const uint32_t *tokens = nullptr;
};

// Throws hip::BackendError naming the lane and the rule it breaks:
//   rows fit the step (1..16 a lane, inside stepRows);
//   1 <= retained <= min(rows, remaining), popcount(retainedRows) == retained, bit 0 set (the anchor
//   row is always on the path), no bit at or above `rows`;
//   accepted < rows and accepted <= retained;
//   every retained token is below `vocabulary` (a row with no selectable logit selects the sentinel).
void validateStepResults(const std::vector<StepLane> &lanes, const std::vector<StepLaneResult> &results, uint32_t stepRows,
                         uint32_t vocabulary);

// Reads a completed step's results from the driver's host-visible buffers (tokens uint32 by packed row, the others
// uint32 by lane), validates them and copies them out: tokensOut holds the lanes' rows, packed.
void readStepResults(const std::vector<StepLane> &lanes, const hip::Buffer &tokens, const hip::Buffer &retained,
                     const hip::Buffer &accepted, const hip::Buffer &retainedRows, uint32_t vocabulary, uint32_t *tokensOut,
                     uint32_t *retainedOut, uint32_t *acceptedOut, uint32_t *retainedRowsOut);

} // namespace splash::model
