// The draft side's steps either side of its tree: every proposal position's candidates and their edge scores (the first
// two kernels of the reference's ops::DraftSelector::add, runtime/ops/DraftSelector.cpp:37-140), and laying a decode
// step's rows out from the trees a draft selector grew (ops::DraftSelector::addVerifyRows, runtime/ops/
// DraftSelector.hpp:139-147; StepRows, runtime/ops/LaneRows.hpp:49-67). Growing the tree over the candidates
// (draft_select_tree) is not part of this library.
#pragma once
#include "abi/Sampling.h"
#include "hip/Backend.hpp"

#include <cstdint>
#include <span>

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

// The tokens a draft's logits columns stand for: the target's first `leading` and those from `trailing` on
// (the reference's DraftVocabulary, runtime/ops/DraftSelector.hpp:94-114).
struct DraftVocabulary final {
  uint32_t leading = 0;
  uint32_t trailing = 0;
  [[nodiscard]] constexpr uint32_t columns(uint32_t vocabulary) const noexcept { return leading + (vocabulary - trailing); }
  [[nodiscard]] constexpr uint32_t token(uint32_t column) const noexcept { return column < leading ? column : column - leading + trailing; }
};

// The selector's codebooks, bf16 [vocabulary][DRAFT_SELECTOR_RANK] each.
struct DraftCodebooks final {
  hip::Buffer predecessor;
  hip::Buffer successor;
};

struct DraftCandidateBuffers final {
  hip::Buffer logits;          // fp32 [lanes * 8][columns]: a lane's proposal positions are rows 1-7 of its eight
  hip::Buffer selectorHidden;  // bf16 [lanes * 8][DRAFT_SELECTOR_RANK], the same rows
  hip::Buffer partials;        // scratch, candidateScratchBytes()
  hip::Buffer candidates;      // uint32 [lanes * 7][16]: each position's tokens, the largest logit first
  hip::Buffer unary;           // fp32 [lanes * 7][16]: their logits
  hip::Buffer edges;           // fp32 [lanes * 7][16][16]: [predecessor][candidate]; position 0 writes row 0 alone
};

class DraftSelector final {
public:
  [[nodiscard]] static uint32_t candidateShards(uint32_t columns) noexcept { return (columns + DRAFT_SHARD_COLUMNS - 1) / DRAFT_SHARD_COLUMNS; }
  [[nodiscard]] static uint64_t candidateScratchBytes(uint32_t lanes, uint32_t columns) noexcept {
    return uint64_t{lanes} * DRAFT_PROPOSAL_TOKENS * candidateShards(columns) * DRAFT_CANDIDATES * 8;
  }
  // Every proposal position's DRAFT_CANDIDATES most likely tokens of a draft of `vocabulary` tokens' target, and each
  // candidate's edge score after each candidate of the position before it (after anchors[lane] at position 0).
  static void addCandidates(hip::CommandGraph &graph, const DraftCandidateBuffers &buffers, const DraftCodebooks &codebooks,
                            DraftVocabulary draft, uint32_t vocabulary, std::span<const uint32_t> anchors);
  // The trees' best rows that the step's rows and its lane cap hold, none past an anchor estimated below `floor`, each
  // lane's numbered in preorder, and the step's rows past them of no lane.
  static void addVerifyRows(hip::CommandGraph &graph, const DraftVerifyRowsBuffers &buffers, const StepRows &step, float floor = 0.0f);
};

} // namespace splash::ops
