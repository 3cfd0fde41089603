#include "ops/Sampling.hpp"
#include "abi/PagedAttention.h"
#include "ops/Linear.hpp"  // requireBytes

#include <algorithm>
#include <cmath>
#include <limits>
#include <stdexcept>
#include <string>

namespace splash::ops {

namespace {
uint32_t packedRows(const std::vector<LaneRows> &lanes) {
  if (lanes.empty() || lanes.size() > SAMPLING_MAXIMUM_LANES) throw std::invalid_argument("acceptance takes 1 to 8 lanes");
  uint32_t rows = 0;
  for (const LaneRows &l : lanes) {
    if (!l.rows || l.rows > SAMPLING_MAXIMUM_ROWS) throw std::invalid_argument("a lane's verify block holds 1 to 16 rows");
    rows = std::max(rows, l.first + l.rows);
  }
  return rows;
}
} // namespace

SamplingWorkspaceSize Sampling::workspace(uint32_t rows) noexcept {
  SamplingWorkspaceSize size;
  size.partialValues = uint64_t{rows} * SAMPLING_SHARDS * 4;
  size.partialIndices = uint64_t{rows} * SAMPLING_SHARDS * 4;
  size.masses = uint64_t{rows} * SAMPLING_SHARDS * 8;
  size.ranges = uint64_t{rows} * SAMPLING_RANGES * 4;
  size.decisions = uint64_t{rows} * SAMPLING_DECISION_WORDS * 4;
  return size;
}

void Sampling::addVerify(hip::CommandGraph &graph, const SamplingBuffers &b, uint32_t vocabulary, uint32_t logitsStride,
                         const std::vector<LaneRows> &lanes, const std::vector<SamplingPolicy> &policies,
                         const std::array<uint32_t, SAMPLING_STOP_TOKENS> &stopTokens) {
  const uint32_t rows = packedRows(lanes);
  if (policies.size() != lanes.size()) throw std::invalid_argument("acceptance takes one policy per lane");
  if (!vocabulary || logitsStride < vocabulary) throw std::invalid_argument("logits rows hold the vocabulary");
  TargetSamplingParams params{};
  params.vocabulary = vocabulary;
  params.rows = rows;
  params.lanes = uint32_t(lanes.size());
  params.logits_stride = logitsStride;
  for (size_t l = 0; l < lanes.size(); ++l) {
    params.lane[l] = {lanes[l].first, lanes[l].rows};
    params.temperature[l] = policies[l].samples() ? policies[l].temperature : 1.0f;
    if (policies[l].samples()) params.sampling_mask |= 1u << l;
    const SamplingPolicy &policy = policies[l];
    if (!(policy.minP >= 0.0f) || !(policy.topP > 0.0f) || !(policy.temperature >= 0.0f))
      throw std::invalid_argument("a sampling policy takes a temperature and a min_p of at least 0 and a top_p above 0");
    if (policy.truncates(vocabulary)) params.truncating_mask |= 1u << l;
    params.min_p[l] = policy.minP;
    params.top_k[l] = policy.topK;
    params.top_p[l] = policy.topP;
    if (policy.constrained) params.constrained_mask |= 1u << l;
    if (policy.excludesStopTokens) params.exclude_stop_mask |= 1u << l;
  }
  for (size_t s = 0; s < stopTokens.size(); ++s) params.stop_tokens[s] = stopTokens[s];
  if (params.constrained_mask) {
    if (uint64_t{b.maskWords} * 32 < vocabulary) throw std::invalid_argument("a constraint-mask row holds a bit for every token");
    requireBytes(b.tokenMask, uint64_t{rows} * b.maskWords * 4, "constraint masks");
    params.mask_words = b.maskWords;
  }
  const SamplingWorkspaceSize need = workspace(rows);
  requireBytes(b.logits, (uint64_t{rows - 1} * logitsStride + vocabulary) * 4, "logits");
  requireBytes(b.tokens, uint64_t{rows} * 4, "selected tokens");
  requireBytes(b.partialValues, need.partialValues, "argmax partial values");
  requireBytes(b.partialIndices, need.partialIndices, "argmax partial indices");
  const bool children = bool(b.candidateIds);
  params.candidate_children = children ? 1u : 0u;
  if (params.sampling_mask) {
    if (children) {
      requireBytes(b.candidateIds, uint64_t{rows} * SAMPLING_CANDIDATES * 4, "candidate ids");
      requireBytes(b.candidateProbabilities, uint64_t{rows} * SAMPLING_CANDIDATES * 4, "candidate probabilities");
      requireBytes(b.candidateDraws, uint64_t{rows} * SAMPLING_TREE_CHILDREN, "drawn children");
      requireBytes(b.childUniforms, uint64_t{rows} * SAMPLING_TREE_CHILDREN * 4, "child uniforms");
    } else {
      requireBytes(b.draftProbabilities, (uint64_t{rows - 1} * logitsStride + vocabulary) * 4, "draft probabilities");
    }
    requireBytes(b.uniforms, uint64_t{rows} * 8, "sampling uniforms");
    requireBytes(b.masses, need.masses, "sampling masses");
    requireBytes(b.ranges, need.ranges, "sampling ranges");
    requireBytes(b.decisions, need.decisions, "sampling decisions");
    requireBytes(b.inputTokens, uint64_t{rows} * 4, "input tokens");
    requireBytes(b.treeRows, uint64_t{rows} * sizeof(AttentionTreeRow), "verify tree rows");
  }
  if (params.constrained_mask || params.exclude_stop_mask)
    graph.add("decode_sample_admit", {b.logits, params.constrained_mask ? b.tokenMask : b.logits}, params,
              {rows, (vocabulary + 1023) / 1024, 1}, {256, 1, 1});
  // Every row gets its argmax; the sampled lanes' rows are then overwritten by their draw.
  graph.add("decode_sample_argmax_sharded", {b.logits, b.partialValues, b.partialIndices}, params, {rows * SAMPLING_SHARDS, 1, 1},
            {SAMPLING_THREADS, 1, 1});
  graph.add("decode_sample_argmax_reduce", {b.partialValues, b.partialIndices, b.tokens}, params, {rows, 1, 1}, {64, 1, 1});
  if (!params.sampling_mask) {
    addThinkingCutoff(graph, b, vocabulary, lanes, policies);
    return;
  }
  graph.add("decode_sample_mass_sharded", {b.logits, b.masses}, params, {rows * SAMPLING_SHARDS, 1, 1}, {SAMPLING_THREADS, 1, 1});
  if (params.truncating_mask)
    graph.add("decode_sample_distribution_end", {b.logits, b.masses, b.decisions}, params, {rows, 1, 1}, {SAMPLING_THREADS, 1, 1});
  // with candidate children no full-vocabulary draft distribution is read: the logits stand in for its binding
  graph.add("decode_sample_residual_ranges",
            {b.logits, children ? b.logits : b.draftProbabilities, b.masses, b.uniforms, b.treeRows, b.inputTokens, b.ranges, b.decisions},
            params, {rows * (SAMPLING_RANGES / 4), 1, 1}, {256, 1, 1});
  if (children)
    graph.add("decode_sample_draw_children",
              {b.logits, b.masses, b.uniforms, b.ranges, b.decisions, b.candidateIds, b.candidateProbabilities, b.candidateDraws,
               b.childUniforms, b.tokens},
              params, {rows, 1, 1}, {64, 1, 1});
  else
    graph.add("decode_sample_draw", {b.logits, b.draftProbabilities, b.masses, b.uniforms, b.ranges, b.decisions, b.tokens}, params,
              {rows, 1, 1}, {64, 1, 1});
  addThinkingCutoff(graph, b, vocabulary, lanes, policies);
}

void Sampling::addThinkingCutoff(hip::CommandGraph &graph, const SamplingBuffers &b, uint32_t vocabulary, const std::vector<LaneRows> &lanes,
                                 const std::vector<SamplingPolicy> &policies) {
  const uint32_t rows = packedRows(lanes);
  if (policies.size() != lanes.size()) throw std::invalid_argument("the thinking cutoffs take one policy per lane");
  ThinkingCutoffParams params{};
  params.vocabulary = vocabulary;
  params.lanes = uint32_t(lanes.size());
  bool any = false;
  for (size_t l = 0; l < lanes.size(); ++l) {
    params.lane[l] = {lanes[l].first, lanes[l].rows};
    const std::optional<ThinkingCutoff> &cutoff = policies[l].thinkingCutoff;
    params.row[l] = cutoff ? std::min<uint32_t>(cutoff->row, SAMPLING_MAXIMUM_ROWS) : SAMPLING_MAXIMUM_ROWS;
    if (params.row[l] >= lanes[l].rows) {   // no row of the block lies that deep
      params.row[l] = SAMPLING_MAXIMUM_ROWS;
      continue;
    }
    if (cutoff->end.empty()) throw std::invalid_argument("a thinking cutoff has an end");
    if (cutoff->waitsForMask) {
      if (!policies[l].constrained) throw std::invalid_argument("only a constrained lane's thinking end waits for its mask");
      if (cutoff->end.front() >= vocabulary) throw std::invalid_argument("a thinking end that waits for a mask starts inside the vocabulary");
      if (uint64_t{b.maskWords} * 32 < vocabulary) throw std::invalid_argument("a constraint-mask row holds a bit for every token");
      requireBytes(b.tokenMask, uint64_t{rows} * b.maskWords * 4, "constraint masks");
      params.waiting_mask |= 1u << l;
      params.mask_words = b.maskWords;
    }
    params.count[l] = uint32_t(std::min<size_t>(cutoff->end.size(), SAMPLING_MAXIMUM_ROWS - params.row[l]));
    std::copy_n(cutoff->end.begin(), params.count[l], params.tokens[l]);
    params.close[l] = cutoff->end.back();
    params.also_ends[l] = cutoff->alsoEnds;
    any = true;
  }
  if (!any) return;
  requireBytes(b.tokens, uint64_t{rows} * 4, "selected tokens");
  requireBytes(b.inputTokens, uint64_t{rows} * 4, "input tokens");
  requireBytes(b.treeRows, uint64_t{rows} * sizeof(AttentionTreeRow), "verify tree rows");
  graph.add("decode_sample_end_thinking", {b.inputTokens, params.waiting_mask ? b.tokenMask : b.inputTokens, b.treeRows, b.tokens}, params,
            {params.lanes, 1, 1}, {64, 1, 1});
}

void Sampling::rebuildPenaltyWords(std::span<uint32_t> words, std::span<const uint32_t> history, uint64_t generatedTokens,
                                   std::optional<uint32_t> pendingToken, bool markPrompt) {
  if (history.size() <= generatedTokens) throw std::logic_error("a request's history holds a prompt");
  const size_t promptTokens = history.size() - size_t(generatedTokens);
  auto inside = [&](uint32_t token) {
    if (token >= words.size()) throw std::invalid_argument("token " + std::to_string(token) + " lies past the vocabulary");
  };
  for (const uint32_t token : history) inside(token);
  if (pendingToken) inside(*pendingToken);
  std::fill(words.begin(), words.end(), 0u);
  for (size_t i = 0; i < history.size(); ++i) {
    if (i >= promptTokens) ++words[history[i]];
    else if (markPrompt) words[history[i]] |= SAMPLING_PENALTY_PROMPT;
  }
  if (pendingToken) ++words[*pendingToken];
}

void Sampling::addPenalties(hip::CommandGraph &graph, const SamplingBuffers &b, uint32_t vocabulary, uint32_t logitsStride,
                            const std::vector<LaneRows> &lanes, const std::vector<SamplingPolicy> &policies, const PenaltyTable &table) {
  const uint32_t rows = packedRows(lanes);
  if (policies.size() != lanes.size()) throw std::invalid_argument("the penalties take one policy per lane");
  if (!vocabulary || logitsStride < vocabulary) throw std::invalid_argument("logits rows hold the vocabulary");
  SamplingPenaltyParams params{};
  params.vocabulary = vocabulary;
  params.logits_stride = logitsStride;
  for (size_t l = 0; l < lanes.size(); ++l) {
    const SamplingPenalties &penalties = policies[l].penalties;
    if (!penalties.active()) continue;
    if (!(penalties.repetition > 0.0f) || !std::isfinite(penalties.repetition) || !std::isfinite(penalties.presence) ||
        !std::isfinite(penalties.frequency))
      throw std::invalid_argument("a repetition penalty is above 0 and every penalty finite");
    if (l >= table.rows.size()) throw std::invalid_argument("a penalized lane names its row of the penalty table");
    const uint32_t e = params.entries++;
    params.lane[e] = {lanes[l].first, lanes[l].rows};
    params.table_row[e] = table.rows[l];
    params.repetition[e] = penalties.repetition;
    params.repetition_inverse[e] = std::min(1.0f / penalties.repetition, std::numeric_limits<float>::max());
    params.presence[e] = penalties.presence;
    params.frequency[e] = penalties.frequency;
    requireBytes(table.words, (uint64_t{table.rows[l]} + 1) * vocabulary * 4, "penalty words");
  }
  if (!params.entries) return;
  requireBytes(b.logits, (uint64_t{rows - 1} * logitsStride + vocabulary) * 4, "logits");
  requireBytes(b.inputTokens, uint64_t{rows} * 4, "input tokens");
  requireBytes(b.treeRows, uint64_t{rows} * sizeof(AttentionTreeRow), "verify tree rows");
  graph.add("decode_sample_penalize", {b.logits, table.words, b.inputTokens, b.treeRows}, params,
            {(vocabulary + 1023) / 1024, params.entries, 1}, {256, 1, 1});
}

void Sampling::addPenaltyCount(hip::CommandGraph &graph, const AcceptanceBuffers &b, uint32_t vocabulary, const std::vector<LaneRows> &lanes,
                               const std::vector<bool> &penalized, const PenaltyTable &table) {
  const uint32_t rows = packedRows(lanes);
  if (penalized.size() != lanes.size()) throw std::invalid_argument("the count takes one flag per lane");
  if (!vocabulary) throw std::invalid_argument("a penalty table row holds the vocabulary");
  SamplingCountParams params{};
  params.vocabulary = vocabulary;
  for (size_t l = 0; l < lanes.size(); ++l) {
    if (!penalized[l]) continue;
    if (l >= table.rows.size()) throw std::invalid_argument("a penalized lane names its row of the penalty table");
    const uint32_t e = params.entries++;
    params.lane[e] = uint32_t(l);
    params.first_row[e] = lanes[l].first;
    params.table_row[e] = table.rows[l];
    requireBytes(table.words, (uint64_t{table.rows[l]} + 1) * vocabulary * 4, "penalty words");
  }
  if (!params.entries) return;
  requireBytes(b.tokens, uint64_t{rows} * 4, "retained tokens");
  requireBytes(b.retained, lanes.size() * 4, "retained counts");
  graph.add("decode_sample_count_tokens", {table.words, b.tokens, b.retained}, params, {params.entries, 1, 1}, {64, 1, 1});
}

void Sampling::addAcceptance(hip::CommandGraph &graph, const AcceptanceBuffers &b, const std::vector<LaneRows> &lanes,
                             const std::vector<uint32_t> &remaining, const std::array<uint32_t, SAMPLING_STOP_TOKENS> &stopTokens) {
  const uint32_t rows = packedRows(lanes);
  if (remaining.size() != lanes.size()) throw std::invalid_argument("acceptance takes one remaining count per lane");
  AcceptBatchParams params{};
  params.lanes = uint32_t(lanes.size());
  for (size_t l = 0; l < lanes.size(); ++l) {
    params.lane[l] = {lanes[l].first, lanes[l].rows};
    params.remaining[l] = remaining[l];
  }
  for (size_t s = 0; s < stopTokens.size(); ++s) params.stop_tokens[s] = stopTokens[s];
  requireBytes(b.inputTokens, uint64_t{rows} * 4, "input tokens");
  requireBytes(b.treeRows, uint64_t{rows} * sizeof(AttentionTreeRow), "verify tree rows");
  requireBytes(b.tokens, uint64_t{rows} * 4, "selected tokens");
  requireBytes(b.retained, lanes.size() * 4, "retained counts");
  requireBytes(b.acceptedCount, lanes.size() * 4, "accepted counts");
  requireBytes(b.retainedRows, lanes.size() * 4, "retained rows");
  graph.add("decode_accept_tree", {b.inputTokens, b.treeRows, b.tokens, b.retained, b.acceptedCount, b.retainedRows}, params,
            {lanes.size(), 1, 1}, {64, 1, 1});
}

} // namespace splash::ops
