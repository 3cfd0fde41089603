#include "ops/DraftSelector.hpp"

#include "abi/PagedAttention.h"  // AttentionTreeRow
#include "ops/Linear.hpp"        // requireBytes

#include <cmath>
#include <stdexcept>

namespace splash::ops {

void DraftSelector::addCandidates(hip::CommandGraph &graph, const DraftCandidateBuffers &b, const DraftCodebooks &codebooks,
                                  DraftVocabulary draft, uint32_t vocabulary, std::span<const uint32_t> anchors) {
  if (anchors.empty() || anchors.size() > SAMPLING_MAXIMUM_LANES) throw std::invalid_argument("invalid draft selector batch");
  if (draft.leading > draft.trailing || draft.trailing > vocabulary || !draft.columns(vocabulary))
    throw std::invalid_argument("a draft's tokens lie in its vocabulary");
  const uint32_t lanes = static_cast<uint32_t>(anchors.size()), columns = draft.columns(vocabulary);
  const uint32_t shards = candidateShards(columns);
  if (shards > DRAFT_MAXIMUM_SHARDS) throw std::invalid_argument("a draft's vocabulary is more than the selector's shards hold");
  DraftSelectParams params{};
  for (uint32_t lane = 0; lane < lanes; ++lane) params.anchor[lane] = anchors[lane];
  params.lanes = lanes;
  params.vocabulary = vocabulary;
  params.columns = columns;
  params.leading = draft.leading;
  params.trailing = draft.trailing;
  params.shards = shards;
  const uint64_t queryRows = uint64_t{lanes} * DRAFT_QUERY_ROWS, rows = uint64_t{lanes} * DRAFT_PROPOSAL_TOKENS;
  const uint64_t codebook = uint64_t{vocabulary} * DRAFT_SELECTOR_RANK * 2;
  requireBytes(b.logits, queryRows * columns * 4, "draft logits");
  requireBytes(b.selectorHidden, queryRows * DRAFT_SELECTOR_RANK * 2, "draft selector hidden");
  requireBytes(b.partials, candidateScratchBytes(lanes, columns), "draft selector scratch");
  requireBytes(b.candidates, rows * DRAFT_CANDIDATES * 4, "draft candidate");
  requireBytes(b.unary, rows * DRAFT_CANDIDATES * 4, "draft candidate score");
  requireBytes(b.edges, rows * DRAFT_CANDIDATES * DRAFT_CANDIDATES * 4, "draft edge score");
  requireBytes(codebooks.predecessor, codebook, "draft predecessor codebook");
  requireBytes(codebooks.successor, codebook, "draft successor codebook");
  graph.add("draft_select_top16_sharded", {b.logits, b.partials}, params, {static_cast<uint32_t>(rows) * shards, 1, 1}, {256, 1, 1});
  graph.add("draft_select_edges",
            {b.logits, b.partials, b.candidates, b.unary, b.edges, b.selectorHidden, codebooks.predecessor, codebooks.successor}, params,
            {static_cast<uint32_t>(rows), 1, 1}, {256, 1, 1});
}

void DraftSelector::addTree(hip::CommandGraph &graph, const DraftTreeBuffers &b, std::span<const DraftTreeLane> lanes) {
  if (lanes.empty() || lanes.size() > SAMPLING_MAXIMUM_LANES) throw std::invalid_argument("invalid draft selector batch");
  DraftTreeParams params{};
  params.lanes = static_cast<uint32_t>(lanes.size());
  for (uint32_t l = 0; l < params.lanes; ++l) {
    const DraftTreeLane &lane = lanes[l];
    if (!lane.children || lane.children > SAMPLING_TREE_CHILDREN) throw std::invalid_argument("a draft row takes one to four children");
    if (lane.depth >= DRAFT_TREE_ROWS || lane.chain > DRAFT_CHAIN_TOKENS) throw std::invalid_argument("a tree is no deeper than a verify block's rows after its anchor");
    if (!(lane.temperature >= 0.0f) || !std::isfinite(lane.temperature) || !std::isfinite(lane.slope))
      throw std::invalid_argument("invalid draft tree lane");
    for (float value : lane.intercept)
      if (!std::isfinite(value)) throw std::invalid_argument("invalid draft tree lane");
    params.anchor[l] = lane.anchor;
    params.depth[l] = lane.depth;
    params.chain[l] = lane.chain;
    params.children[l] = lane.children;
    params.slope[l] = lane.slope;
    for (uint32_t p = 0; p < DRAFT_PROPOSAL_TOKENS; ++p) params.intercept[l][p] = lane.intercept[p];
    params.temperature[l] = lane.temperature;
    params.noise[l][0] = static_cast<uint32_t>(lane.noise);
    params.noise[l][1] = static_cast<uint32_t>(lane.noise >> 32);
  }
  const uint64_t positions = uint64_t{params.lanes} * DRAFT_PROPOSAL_TOKENS, rows = uint64_t{params.lanes} * DRAFT_TREE_ROWS;
  requireBytes(b.candidates, positions * DRAFT_CANDIDATES * 4, "draft candidate");
  requireBytes(b.unary, positions * DRAFT_CANDIDATES * 4, "draft candidate score");
  requireBytes(b.edges, positions * DRAFT_CANDIDATES * DRAFT_CANDIDATES * 4, "draft edge score");
  requireBytes(b.chainTokens, uint64_t{params.lanes} * DRAFT_CHAIN_TOKENS * 4, "draft chain token");
  requireBytes(b.chainRates, uint64_t{params.lanes} * DRAFT_CHAIN_TOKENS * DRAFT_CHAIN_AGREEMENTS * 4, "draft chain rate");
  requireBytes(b.treeTokens, rows * 4, "draft tree token");
  requireBytes(b.trees, rows * sizeof(AttentionTreeRow), "draft tree row");
  requireBytes(b.treeScores, rows * 8, "draft tree score");
  requireBytes(b.treeSizes, uint64_t{params.lanes} * 4, "draft tree size");
  requireBytes(b.treeDraws, rows * SAMPLING_TREE_CHILDREN, "draft tree draws");
  requireBytes(b.treeNext, rows * DRAFT_CANDIDATES * 4, "draft tree next probabilities");
  requireBytes(b.treeCaps, rows * 4, "draft tree cap");
  graph.add("draft_select_tree",
            {b.candidates, b.unary, b.edges, b.chainTokens, b.chainRates, b.treeTokens, b.trees, b.treeScores, b.treeSizes, b.treeDraws,
             b.treeNext, b.treeCaps},
            params, {params.lanes, 1, 1}, {64, 1, 1});
}

void DraftSelector::addVerifyChildren(hip::CommandGraph &graph, const DraftVerifyChildrenBuffers &b, const StepRows &step) {
  if (!step.lanes || step.lanes > SAMPLING_MAXIMUM_LANES || step.rows < step.lanes) throw std::invalid_argument("invalid decode step rows");
  const uint64_t treeRows = uint64_t{step.lanes} * DRAFT_TREE_ROWS;
  requireBytes(b.verifySources, uint64_t{step.rows} * 4, "verify source");
  requireBytes(b.laneRows, uint64_t{step.lanes} * sizeof(SamplingLaneRows), "verify lane rows");
  requireBytes(b.treeRows, uint64_t{step.rows} * sizeof(AttentionTreeRow), "verify tree row");
  requireBytes(b.candidates, uint64_t{step.lanes} * DRAFT_PROPOSAL_TOKENS * DRAFT_CANDIDATES * 4, "draft candidate");
  requireBytes(b.treeNext, treeRows * DRAFT_CANDIDATES * 4, "draft tree next probabilities");
  requireBytes(b.treeDraws, treeRows * SAMPLING_TREE_CHILDREN, "draft tree draws");
  requireBytes(b.candidateIds, uint64_t{step.rows} * SAMPLING_CANDIDATES * 4, "candidate ids");
  requireBytes(b.candidateProbabilities, uint64_t{step.rows} * SAMPLING_CANDIDATES * 4, "candidate probabilities");
  requireBytes(b.candidateDraws, uint64_t{step.rows} * SAMPLING_TREE_CHILDREN, "drawn children");
  requireBytes(b.depths, uint64_t{step.rows} * 4, "row depths");
  graph.add("draft_verify_children",
            {b.verifySources, b.laneRows, b.treeRows, b.candidates, b.treeNext, b.treeDraws, b.candidateIds, b.candidateProbabilities,
             b.candidateDraws, b.depths},
            VerifyChildrenParams{step.lanes, step.rows, {0, 0}}, {step.rows, 1, 1}, {64, 1, 1});
}

void DraftSelector::addVerifyRows(hip::CommandGraph &graph, const DraftVerifyRowsBuffers &b, const StepRows &step, float floor) {
  if (!step.lanes || step.lanes > SAMPLING_MAXIMUM_LANES || !step.laneCap || step.laneCap > SAMPLING_MAXIMUM_ROWS ||
      step.rows < step.lanes || step.rows > uint64_t{step.lanes} * step.laneCap)
    throw std::invalid_argument("invalid decode step rows");
  if (step.slots && step.rows != step.lanes * step.laneCap) throw std::invalid_argument("rows in slots are a lane cap of rows a lane");
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
            VerifyRowsParams{step.lanes, step.rows, step.laneCap, floor, step.slots ? 1u : 0u, {}}, {1, 1, 1}, {128, 1, 1});
}

} // namespace splash::ops
