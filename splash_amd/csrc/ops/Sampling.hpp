// Acceptance of a verify block: ops::Sampling (runtime/ops/Sampling.hpp:64-254, Sampling.cpp:283-357
// in the reference) over kernels/sampling.hip. addVerify selects each row's token (argmax, or
// rejection sampling over the row's drafted child at temperature > 0, from the distribution the
// lane's min_p, top_k and top_p leave); addAcceptance walks each
// lane's block from its first row and writes the retained tokens, counts and retained-row mask.
#pragma once
#include "abi/Sampling.h"
#include "hip/Backend.hpp"

#include <array>
#include <optional>
#include <span>
#include <vector>

namespace splash::ops {

// Sampling.hpp:56-83 in the reference, without penalties, constraints and the thinking cutoff.
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
  // A lane samples unless it keeps only its most likely token (Sampling.hpp:79-82).
  [[nodiscard]] bool samples() const noexcept { return temperature > 0.0f && minP < 1.0f && topK != 1; }
  [[nodiscard]] bool truncates(uint32_t vocabulary) const noexcept {
    return samples() && (minP > 0.0f || (topK && topK < vocabulary) || topP < 1.0f);
  }
};

// The sampling penalties, which rewrite a lane's target logits before its policy selects from them (the reference's
// SamplingPenalties, runtime/ops/Sampling.hpp:17-29): repetition scales the logit of every token the prompt or the
// output holds, presence and frequency lower that of every token the output holds. The defaults change nothing.
struct SamplingPenalties final {
  float repetition = 1.0f;
  float presence = 0.0f;
  float frequency = 0.0f;
  [[nodiscard]] bool active() const noexcept { return repetition != 1.0f || presence != 0.0f || frequency != 0.0f; }
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
};
struct AcceptanceBuffers final {
  hip::Buffer inputTokens;    // uint32 [rows]
  hip::Buffer treeRows;       // AttentionTreeRow [rows]
  hip::Buffer tokens;         // in: selections; out: each lane's retained tokens from its first row
  hip::Buffer retained;       // uint32 [lanes]: retained token count
  hip::Buffer acceptedCount;  // uint32 [lanes]
  hip::Buffer retainedRows;   // uint32 [lanes]: mask of the block rows retained
};

// Where a lane's thinking budget runs out in a selection (the reference's ThinkingCutoff, Sampling.hpp:30-55): its
// selected rows of depth `row` on take the `end` tokens in order, as many as the block holds, unless a draft token on
// the row's path up to depth `row` is the last of `end`, which closes thinking, or `alsoEnds`. An end that waits for
// the mask of a constrained lane starts instead, along each row's path, at the first of the path's rows from depth
// `row` on whose constraint-mask row admits its first token.
struct ThinkingCutoff final {
  uint32_t row = 0;
  std::vector<uint32_t> end;
  uint32_t alsoEnds = SAMPLING_NO_TOKEN;
  bool waitsForMask = false;
};

// A lane whose logits rows the penalties rewrite, from row `tableRow` of the penalty table.
struct PenalizedLane final {
  LaneRows rows;
  uint32_t tableRow = 0;
  SamplingPenalties penalties;
};

class Sampling final {
public:
  // A request's penalty words (abi/Sampling.h), rebuilt from its history of prompt and generated tokens: the prompt
  // bit on every prompt token (markPrompt), the count of every generated token and of a pending one
  // (Sampling.cpp:91-114 in the reference). Throws for a token outside the vocabulary (words.size()).
  static void rebuildPenaltyWords(std::span<uint32_t> words, std::span<const uint32_t> history, uint64_t generatedTokens,
                                  std::optional<uint32_t> pendingToken, bool markPrompt);
  // Counts the tokens one step selected into a request's penalty words (Sampling.cpp:116-121).
  static void countPenaltyTokens(std::span<uint32_t> words, std::span<const uint32_t> selected);
  // Rewrites the logits rows of the lanes whose penalties are active, in place, before addVerify reads them
  // (Sampling::addPenalties, Sampling.cpp:129-172): `words` holds uint32 [table rows][vocabulary]; a row of a lane also
  // counts the draft tokens of its path, from the block's input tokens and tree rows. Nothing when no lane is active.
  static void addPenalties(hip::CommandGraph &graph, const hip::Buffer &logits, const hip::Buffer &words,
                           const hip::Buffer &inputTokens, const hip::Buffer &treeRows, uint32_t vocabulary,
                           uint32_t logitsStride, const std::vector<PenalizedLane> &lanes);
  [[nodiscard]] static SamplingWorkspaceSize workspace(uint32_t rows) noexcept;
  // One policy per lane. Throws for no or too many lanes, rows outside 1..16, or missing buffers.
  // The logits rows of a constrained or stop-excluding lane are rewritten first: -infinity at the
  // tokens the lane does not admit (TargetRow::admits in the reference, which reads a mask instead).
  static void addVerify(hip::CommandGraph &graph, const SamplingBuffers &buffers, uint32_t vocabulary, uint32_t logitsStride,
                        const std::vector<LaneRows> &lanes, const std::vector<SamplingPolicy> &policies,
                        const std::array<uint32_t, SAMPLING_STOP_TOKENS> &stopTokens = {SAMPLING_NO_TOKEN, SAMPLING_NO_TOKEN,
                                                                                       SAMPLING_NO_TOKEN, SAMPLING_NO_TOKEN});
  // After addVerify: the selections of the rows each lane's thinking end reaches become its end tokens
  // (decode_sample_thinking_cutoff, Sampling.cpp:41-78 and :314-327 in the reference). One optional cutoff a lane; a
  // lane without one, or whose cutoff row is past its rows, keeps its selections. Nothing when no lane is cut.
  // tokenMask (uint32 [rows][maskWords]) only for a lane whose end waits for its mask.
  static void addThinkingCutoff(hip::CommandGraph &graph, const hip::Buffer &inputTokens, const hip::Buffer &tokenMask,
                                uint32_t maskWords, const hip::Buffer &treeRows, const hip::Buffer &tokens, uint32_t vocabulary,
                                const std::vector<LaneRows> &lanes, const std::vector<std::optional<ThinkingCutoff>> &cutoffs);
  static void addAcceptance(hip::CommandGraph &graph, const AcceptanceBuffers &buffers, const std::vector<LaneRows> &lanes,
                            const std::vector<uint32_t> &remaining, const std::array<uint32_t, SAMPLING_STOP_TOKENS> &stopTokens);
};

} // namespace splash::ops
