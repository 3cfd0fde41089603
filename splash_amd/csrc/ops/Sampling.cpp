#include "ops/Sampling.hpp"
#include "abi/PagedAttention.h"
#include "ops/Linear.hpp"  // requireBytes

#include <algorithm>
#include <cmath>
#include <limits>
#include <stdexcept>

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

void Sampling::rebuildPenaltyWords(std::span<uint32_t> words, std::span<const uint32_t> history, uint64_t generatedTokens,
                                   std::optional<uint32_t> pendingToken, bool markPrompt) {
  if (history.size() <= generatedTokens) throw std::logic_error("request history holds no prompt");
  const auto inside = [&](uint32_t token) {
    if (token >= words.size()) throw std::invalid_argument("penalty token is outside the vocabulary");
  };
  for (uint32_t token : history) inside(token);
  if (pendingToken) inside(*pendingToken);
  const size_t prompt = history.size() - generatedTokens;
  std::fill(words.begin(), words.end(), 0u);
  if (markPrompt)
    for (size_t i = 0; i < prompt; ++i) words[history[i]] |= SAMPLING_PENALTY_PROMPT_BIT;
  for (size_t i = prompt; i < history.size(); ++i) ++words[history[i]];
  if (pendingToken) ++words[*pendingToken];
}

void Sampling::countPenaltyTokens(std::span<uint32_t> words, std::span<const uint32_t> selected) {
  for (uint32_t token : selected)
    if (token >= words.size()) throw std::invalid_argument("penalty token is outside the vocabulary");
  for (uint32_t token : selected) ++words[token];
}

void Sampling::addPenalties(hip::CommandGraph &graph, const hip::Buffer &logits, const hip::Buffer &words,
                            const hip::Buffer &inputTokens, const hip::Buffer &treeRows, uint32_t vocabulary, uint32_t logitsStride,
                            const std::vector<PenalizedLane> &lanes) {
  if (!vocabulary || logitsStride < vocabulary) throw std::invalid_argument("logits rows hold the vocabulary");
  std::vector<LaneRows> rowsOf;
  for (const PenalizedLane &l : lanes) rowsOf.push_back(l.rows);
  const uint32_t rows = packedRows(rowsOf);
  SamplingPenaltyParams params{};
  params.vocabulary = vocabulary;
  params.logits_stride = logitsStride;
  for (const PenalizedLane &l : lanes) {
    if (!l.penalties.active()) continue;
    if (!(l.penalties.repetition > 0.0f) || !std::isfinite(l.penalties.repetition) || !std::isfinite(l.penalties.presence) ||
        !std::isfinite(l.penalties.frequency))
      throw std::invalid_argument("a repetition penalty is positive and every penalty finite");
    // the kernel indexes the whole table by this row
    requireBytes(words, (uint64_t{l.tableRow} + 1) * vocabulary * 4, "penalty table");
    const uint32_t entry = params.entries++;
    params.lane[entry] = {l.rows.first, l.rows.rows};
    params.table_row[entry] = l.tableRow;
    params.repetition[entry] = l.penalties.repetition;
    // 1 / 2^-149 overflows; the saturated inverse keeps the product finite
    params.repetition_inverse[entry] = std::min(1.0f / l.penalties.repetition, std::numeric_limits<float>::max());
    params.presence[entry] = l.penalties.presence;
    params.frequency[entry] = l.penalties.frequency;
  }
  if (!params.entries) return;
  requireBytes(logits, (uint64_t{rows - 1} * logitsStride + vocabulary) * 4, "logits");
  requireBytes(treeRows, uint64_t{rows} * sizeof(AttentionTreeRow), "verify tree rows");
  requireBytes(inputTokens, uint64_t{rows} * 4, "input tokens");
  graph.add("decode_sample_penalize", {logits, words, inputTokens, treeRows}, params, {(vocabulary + 255) / 256, params.entries, 1},
            {256, 1, 1});
}

void Sampling::addThinkingCutoff(hip::CommandGraph &graph, const hip::Buffer &inputTokens, const hip::Buffer &tokenMask,
                                 uint32_t maskWords, const hip::Buffer &treeRows, const hip::Buffer &tokens, uint32_t vocabulary,
                                 const std::vector<LaneRows> &lanes, const std::vector<std::optional<ThinkingCutoff>> &cutoffs) {
  const uint32_t rows = packedRows(lanes);
  if (cutoffs.size() != lanes.size()) throw std::invalid_argument("a thinking cutoff, or none, per lane");
  if (!vocabulary) throw std::invalid_argument("invalid sampling geometry");
  ThinkingCutoffParams params{};
  params.vocabulary = vocabulary;
  params.lanes = uint32_t(lanes.size());
  params.mask_words = maskWords;
  bool cuts = false;
  for (size_t l = 0; l < lanes.size(); ++l) {
    params.lane[l] = {lanes[l].first, lanes[l].rows};
    const std::optional<ThinkingCutoff> &cutoff = cutoffs[l];
    params.row[l] = cutoff ? cutoff->row : lanes[l].rows;
    if (params.row[l] >= lanes[l].rows) {
      params.row[l] = SAMPLING_MAXIMUM_ROWS;  // past every depth: the lane's rows keep their selections
      continue;
    }
    if (cutoff->end.empty()) throw std::invalid_argument("a thinking cutoff has no end");
    if (cutoff->waitsForMask) {
      if (cutoff->end.front() >= vocabulary)
        throw std::invalid_argument("a thinking end that waits for a mask starts outside the vocabulary");
      if (uint64_t{maskWords} * 32 < vocabulary) throw std::invalid_argument("a constraint-mask row holds a bit for every token");
      requireBytes(tokenMask, uint64_t{rows} * maskWords * 4, "constraint masks");
      params.waiting_mask |= 1u << l;
    }
    // The rows from the cutoff's on take as many of its end as the lane's rows hold.
    params.count[l] = uint32_t(std::min<size_t>(cutoff->end.size(), lanes[l].rows - cutoff->row));
    std::copy_n(cutoff->end.begin(), params.count[l], params.tokens[l]);
    params.close[l] = cutoff->end.back();
    params.also_ends[l] = cutoff->alsoEnds;
    cuts = true;
  }
  if (!cuts) return;
  requireBytes(inputTokens, uint64_t{rows} * 4, "input tokens");
  requireBytes(treeRows, uint64_t{rows} * sizeof(AttentionTreeRow), "verify tree rows");
  requireBytes(tokens, uint64_t{rows} * 4, "selected tokens");
  graph.add("decode_sample_thinking_cutoff", {inputTokens, params.waiting_mask ? tokenMask : inputTokens, treeRows, tokens}, params,
            {uint32_t(lanes.size()), 1, 1}, {64, 1, 1});
}

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
  if (params.sampling_mask) {
    requireBytes(b.draftProbabilities, (uint64_t{rows - 1} * logitsStride + vocabulary) * 4, "draft probabilities");
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
  if (!params.sampling_mask) return;
  graph.add("decode_sample_mass_sharded", {b.logits, b.masses}, params, {rows * SAMPLING_SHARDS, 1, 1}, {SAMPLING_THREADS, 1, 1});
  if (params.truncating_mask)
    graph.add("decode_sample_distribution_end", {b.logits, b.masses, b.decisions}, params, {rows, 1, 1}, {SAMPLING_THREADS, 1, 1});
  graph.add("decode_sample_residual_ranges",
            {b.logits, b.draftProbabilities, b.masses, b.uniforms, b.treeRows, b.inputTokens, b.ranges, b.decisions}, params,
            {rows * (SAMPLING_RANGES / 4), 1, 1}, {256, 1, 1});
  graph.add("decode_sample_draw", {b.logits, b.draftProbabilities, b.masses, b.uniforms, b.ranges, b.decisions, b.tokens}, params,
            {rows, 1, 1}, {64, 1, 1});
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
