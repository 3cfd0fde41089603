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
            VerifyRowsParams{step.lanes, step.rows, step.laneCap, floor}, {1, 1, 1}, {128, 1, 1});
}

} // namespace splash::ops
