// Acceptance of a verify block: ops::Sampling (runtime/ops/Sampling.hpp:64-254, Sampling.cpp:283-357
// in the reference) over kernels/sampling.hip. addVerify selects each row's token (argmax, or
// rejection sampling over the row's drafted child at temperature > 0, from the distribution the
// lane's min_p, top_k and top_p leave); addAcceptance walks each
// lane's block from its first row and writes the retained tokens, counts and retained-row mask.
#pragma once
#include "abi/Sampling.h"
#include "hip/Backend.hpp"

#include <algorithm>
#include <array>
#include <optional>
#include <span>
#include <vector>

namespace splash::ops {

// The sampling penalties (Sampling.hpp:17-30 in the reference), which rewrite a lane's target logits before its policy
// selects from them: repetition scales the logit of every token the prompt or the output holds, presence and frequency
// lower that of every token the output holds. The defaults leave the logits unchanged.
struct SamplingPenalties final {
  float repetition = 1.0f;
  float presence = 0.0f;
  float frequency = 0.0f;
  [[nodiscard]] bool active() const noexcept { return repetition != 1.0f || presence != 0.0f || frequency != 0.0f; }
};

// The penalty words of every state lane, one row of `vocabulary` words each, in device memory, and the row each lane of
// a dispatch reads (PenaltyTable, Sampling.hpp:85-91 in the reference).
struct PenaltyTable final {
  hip::Buffer words;
  std::span<const uint32_t> rows;
};

// Where a lane's thinking budget runs out in a selection (ThinkingCutoff, Sampling.hpp:30-55 in the reference): its
// selected rows of depth `row` on take the `end` tokens in order, as many as the block holds, unless a draft token on a
// row's path up to depth `row` is the last of `end`, which closes thinking, or `alsoEnds`: either ended thinking first.
// An end that waits for the mask of a constrained lane starts instead, along each row's path, at the first of the
// path's rows from depth `row` on whose mask admits its first token.
struct ThinkingCutoff final {
  uint32_t row = 0;
  std::vector<uint32_t> end;
  uint32_t alsoEnds = SAMPLING_NO_TOKEN;
  bool waitsForMask = false;
  // How many of the lane's proposals, from the first, the end makes (tokens the draft did not propose): the caller
  // proposes them as a host chain of the lane's tree, so that acceptance keeps them.
  [[nodiscard]] uint32_t replacedProposals() const noexcept {
    return row || waitsForMask ? 0u : uint32_t(std::min<size_t>(end.size(), SAMPLING_MAXIMUM_ROWS - 1));
  }
};

// Sampling.hpp:56-83 in the reference.
struct SamplingPolicy final {
  float temperature = 0.0f;
  // A sampling lane keeps the tokens minP leaves it (those that weigh at least minP of the
  // heaviest; 0 drops none), then its topK most likely of those (0, or a topK past the vocabulary:
  // all), then its topP nucleus of those.
  float minP = 0.0f;
  uint32_t topK = 0;
  float topP = 1.0f;
  // The lane's rows admit only the tokens of their rows of SamplingBuffers::tokenMask.
  bool constrained = false;
  // The lane ignores end-of-sequence: it never selects a stop token (addVerify's stopTokens).
  bool excludesStopTokens = false;
  // Greedy lanes take the argmax of the penalized logits, sampling lanes draw from them.
  SamplingPenalties penalties{};
  // While the lane thinks under a budget, where that budget runs out; the rows from there on select the end of
  // thinking whatever their logits.
  std::optional<ThinkingCutoff> thinkingCutoff{};
  // A lane samples unless it keeps only its most likely token (Sampling.hpp:79-82).
  [[nodiscard]] bool samples() const noexcept { return temperature > 0.0f && minP < 1.0f && topK != 1; }
  [[nodiscard]] bool truncates(uint32_t vocabulary) const noexcept {
    return samples() && (minP > 0.0f || (topK && topK < vocabulary) || topP < 1.0f);
  }
};

struct LaneRows final {
  uint32_t first = 0, rows = 0;
};

struct SamplingWorkspaceSize final {
  uint64_t partialValues = 0, partialIndices = 0, masses = 0, ranges = 0, decisions = 0;
};
struct SamplingBuffers final {
  hip::Buffer logits;         // fp32 [rows][stride]
  hip::Buffer tokens;         // uint32 [rows]: each row's selection
  hip::Buffer partialValues, partialIndices;  // greedy shards
  // sampled rows only:
  hip::Buffer draftProbabilities;  // fp32 [rows][stride]: the distribution each row's child was drawn from
  hip::Buffer uniforms;            // fp32 [rows][2]: the row's draw, its child's test
  hip::Buffer masses, ranges;
  hip::Buffer decisions;  // SAMPLING_DECISION_WORDS words a row: its child's test and the end of its distribution
  hip::Buffer inputTokens, treeRows;  // the block's input tokens and SplashTreeRow rows
  // Constrained lanes only: uint32 [rows][maskWords], bit t % 32 of word t / 32 of a row admits token t.
  hip::Buffer tokenMask;
  uint32_t maskWords = 0;
  // A tree block's sampled rows (Sampling.hpp:119-136 in the reference, DrawChildren): each row's sixteen candidates
  // (uint32 ids and fp32 draft probabilities [rows][16]), the candidate indices of the children its draft drew, in the
  // order drawn (bytes [rows][4], 0xFF past them), and a uniform for each child's test (fp32 [rows][4]). With these the
  // sampled lanes' rows run recursive rejection sampling over their children; draftProbabilities is then not read.
  hip::Buffer candidateIds, candidateProbabilities, candidateDraws, childUniforms;
};
struct AcceptanceBuffers final {
  hip::Buffer inputTokens;    // uint32 [rows]
  hip::Buffer treeRows;       // AttentionTreeRow [rows]
  hip::Buffer tokens;         // in: selections; out: each lane's retained tokens from its first row
  hip::Buffer retained;       // uint32 [lanes]: retained token count
  hip::Buffer acceptedCount;  // uint32 [lanes]
  hip::Buffer retainedRows;   // uint32 [lanes]: mask of the block rows retained
};

class Sampling final {
public:
  [[nodiscard]] static SamplingWorkspaceSize workspace(uint32_t rows) noexcept;
  // One policy per lane. Throws for no or too many lanes, rows outside 1..16, or missing buffers.
  // The logits rows of a constrained or stop-excluding lane are rewritten first: -infinity at the
  // tokens the lane does not admit (TargetRow::admits in the reference, which reads a mask instead).
  static void addVerify(hip::CommandGraph &graph, const SamplingBuffers &buffers, uint32_t vocabulary, uint32_t logitsStride,
                        const std::vector<LaneRows> &lanes, const std::vector<SamplingPolicy> &policies,
                        const std::array<uint32_t, SAMPLING_STOP_TOKENS> &stopTokens = {SAMPLING_NO_TOKEN, SAMPLING_NO_TOKEN,
                                                                                       SAMPLING_NO_TOKEN, SAMPLING_NO_TOKEN});
  static void addAcceptance(hip::CommandGraph &graph, const AcceptanceBuffers &buffers, const std::vector<LaneRows> &lanes,
                            const std::vector<uint32_t> &remaining, const std::array<uint32_t, SAMPLING_STOP_TOKENS> &stopTokens);

  // The thinking cutoff of each lane that has one, over the selections addVerify left in buffers.tokens and before
  // addAcceptance walks them (the end of Sampling::addSelection, Sampling.cpp:314-327; addVerify runs it last). Reads
  // buffers.inputTokens and buffers.treeRows, and buffers.tokenMask for a lane whose end waits for its mask. Nothing is
  // dispatched when no lane's cutoff lies inside its block.
  static void addThinkingCutoff(hip::CommandGraph &graph, const SamplingBuffers &buffers, uint32_t vocabulary,
                                const std::vector<LaneRows> &lanes, const std::vector<SamplingPolicy> &policies);

  // A penalized request's penalty words, rebuilt when it takes a state lane (Sampling::rebuildPenaltyWords,
  // Sampling.cpp:91-114 in the reference): from its history, the prompt and then the `generatedTokens` outputs it
  // emitted. Every prompt token gets the prompt bit when markPrompt (only repetition reads it); the counts are of the
  // outputs and of the pending anchor. Host memory; the caller uploads the row. Throws std::logic_error for a history
  // with no prompt and std::invalid_argument for a token past the vocabulary (words.size()).
  static void rebuildPenaltyWords(std::span<uint32_t> words, std::span<const uint32_t> history, uint64_t generatedTokens,
                                  std::optional<uint32_t> pendingToken, bool markPrompt);
  // Each lane with active penalties has the logits rows of its block rewritten in place from its row of the table, a
  // row's context adding the block's draft tokens on its path (Sampling::addPenalties, Sampling.cpp:163-180; addVerify
  // runs it first). Nothing is dispatched when no lane's penalties are active. Runs before addVerify on the LM head's
  // fresh rows; buffers.inputTokens and buffers.treeRows are read for every penalized lane.
  static void addPenalties(hip::CommandGraph &graph, const SamplingBuffers &buffers, uint32_t vocabulary, uint32_t logitsStride,
                           const std::vector<LaneRows> &lanes, const std::vector<SamplingPolicy> &policies, const PenaltyTable &table);
  // The tokens each lane retained of the step are counted into its row of the table, on the device (the reference's
  // engine calls Sampling::countPenaltyTokens on the host, Sampling.cpp:116-121). `penalized[l]` selects the lanes.
  static void addPenaltyCount(hip::CommandGraph &graph, const AcceptanceBuffers &buffers, uint32_t vocabulary,
                              const std::vector<LaneRows> &lanes, const std::vector<bool> &penalized, const PenaltyTable &table);
};

} // namespace splash::ops
