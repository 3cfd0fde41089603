// The draft side's steps either side of its tree: every proposal position's candidates and their edge scores (the first
// two kernels of the reference's ops::DraftSelector::add, runtime/ops/DraftSelector.cpp:37-140), and laying a decode
// step's rows out from the trees a draft selector grew (ops::DraftSelector::addVerifyRows, runtime/ops/
// DraftSelector.hpp:139-147; StepRows, runtime/ops/LaneRows.hpp:49-67), and between them the tree each lane grows over
// its candidates (draft_select_tree, DraftSelector.cpp:96-118).
#pragma once
#include "abi/Sampling.h"
#include "hip/Backend.hpp"

#include <array>
#include <cstdint>
#include <span>

namespace splash::ops {

// A decode step's rows: `rows` rows over `lanes` lanes, packed in lane order, each lane 1 to `laneCap` of them.
struct StepRows final {
  uint32_t lanes = 0;
  uint32_t rows = 0;
  uint32_t laneCap = 0;
  // Not packed: lane l's rows from row l * laneCap on (rows == lanes * laneCap), the rest of its slot inert rows, so that
  // a step recorded for laneCap rows a lane takes trees of any size (abi/Sampling.h, VerifyRowsParams::slots).
  bool slots = false;
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

// A lane of DraftSelector::addTree (the reference's DraftTreeLane, runtime/ops/DraftSelector.hpp:59-92).
struct DraftTreeLane final {
  uint32_t anchor = 0;       // the token the lane's tree grows from
  uint32_t depth = 0;        // the deepest row a walk of the tree may retain
  uint32_t children = 1;     // candidates a draft row takes: 1..SAMPLING_TREE_CHILDREN
  uint32_t chain = 0;        // tokens of the lane's host chain (chainTokens), 0 for none
  float slope = 1.0f;        // the lane's acceptance model: sigmoid(slope * logit(q) + intercept[position])
  std::array<float, DRAFT_PROPOSAL_TOKENS> intercept{};
  float temperature = 0.0f;  // 0: the likeliest candidates; above: draws from the probabilities at that temperature
  uint64_t noise = 0;        // the seed of a sampled lane's draws
};

struct DraftTreeBuffers final {
  hip::Buffer candidates, unary, edges;  // as addCandidates left them
  hip::Buffer chainTokens;   // uint32 [lanes][15]: each lane's host chain
  hip::Buffer chainRates;    // fp32 [lanes][15][4]: a chain token's rate by its agreement with the draft at its depth
  hip::Buffer treeTokens, trees, treeScores, treeSizes;  // as addVerifyRows reads them
  hip::Buffer treeDraws;     // bytes [lanes][16][4]: a row's drawn children (candidate indices), SAMPLING_NO_DRAW past them
  hip::Buffer treeNext;      // fp32 [lanes][16][16]: a row's next position's probabilities (at the lane's temperature)
  hip::Buffer treeCaps;      // fp32 [lanes][16]: the cap of the draft step that made or joined a row
};

// The step's rows (addVerifyRows' outputs) and the trees they came from, and what a sampled verify step reads of them.
struct DraftVerifyChildrenBuffers final {
  hip::Buffer verifySources, laneRows, treeRows;  // of the step, as addVerifyRows wrote them
  hip::Buffer candidates, treeNext, treeDraws;    // of the trees (addCandidates, addTree)
  hip::Buffer candidateIds;            // uint32 [rows][16]: the candidates of a row's next position
  hip::Buffer candidateProbabilities;  // fp32 [rows][16]
  hip::Buffer candidateDraws;          // bytes [rows][4]: the children the draft drew, SAMPLING_NO_DRAW past them
  hip::Buffer depths;                  // uint32 [rows]: a row's depth below its lane's anchor (the RoPE tables' input)
};

class DraftSelector final {
public:
  // The candidate children of every row of the step (ops::SamplingBuffers' candidate fields) and the rows' depths, from
  // the trees: a step then takes its tree blocks from the draft side without a copy through the host.
  static void addVerifyChildren(hip::CommandGraph &graph, const DraftVerifyChildrenBuffers &buffers, const StepRows &step);
  // Each lane's tree over the candidates and edges addCandidates left, best first by estimate (abi/Sampling.h,
  // DraftTreeParams): rows 16 l .. of the tree buffers, lane l's sizes[l] of them.
  static void addTree(hip::CommandGraph &graph, const DraftTreeBuffers &buffers, std::span<const DraftTreeLane> lanes);
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
