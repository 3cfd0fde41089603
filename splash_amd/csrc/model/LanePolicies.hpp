// What a driver's lanes add to their sampling policies between steps: each dispatch lane's thinking cutoff
// (ops::ThinkingCutoff), whether it is constrained by its rows of the token mask and whether it ignores end-of-sequence,
// the step's stop tokens, the lane's penalties (ops::SamplingPenalties) and its row of the penalty table the driver owns,
// `vocabulary` words a lane in device memory, allocated (zeroed) when a lane first takes active penalties. The reference's model keeps the table per state lane and the engine counts a step's tokens into it
// on the host (Sampling.hpp:85-91, Sampling::countPenaltyTokens); here a step that commits counts them on the device.
#pragma once
#include "hip/Backend.hpp"
#include "ops/Sampling.hpp"

#include <array>
#include <numeric>
#include <optional>
#include <stdexcept>
#include <vector>

namespace splash::model {

class LanePolicies final {
public:
  using StopTokens = std::array<uint32_t, SAMPLING_STOP_TOKENS>;
  LanePolicies(hip::Backend &backend, uint32_t lanes, uint32_t vocabulary)
      : backend_(backend), vocabulary_(vocabulary), penalties_(lanes), cutoffs_(lanes), constrained_(lanes), excludesStop_(lanes),
        rows_(lanes) {
    std::iota(rows_.begin(), rows_.end(), 0u);
    stopTokens_.fill(SAMPLING_NO_TOKEN);
  }
  // The lane's rows admit only the tokens of their rows of tokenMask(); the lane never selects a stop token.
  void setAdmission(uint32_t lane, bool constrained, bool excludesStopTokens) {
    if (lane >= constrained_.size()) throw std::invalid_argument("the admission of a lane past the driver's");
    constrained_[lane] = constrained;
    excludesStop_[lane] = excludesStopTokens;
  }
  // The tokens that end a sequence: acceptance keeps nothing past one, and a lane that ignores them never selects one.
  void setStopTokens(const StopTokens &tokens) noexcept { stopTokens_ = tokens; }
  [[nodiscard]] const StopTokens &stopTokens() const noexcept { return stopTokens_; }
  [[nodiscard]] uint32_t maskWords() const noexcept { return (vocabulary_ + 31) / 32; }
  // The constraint masks: uint32 [rows][maskWords()], bit t % 32 of word t / 32 of a packed row admits token t.
  const hip::Buffer &tokenMask(uint32_t rows) {
    if (!tokenMask_) tokenMask_ = backend_.allocateBuffer(uint64_t{rows} * maskWords() * 4, hip::BufferStorage::Private, "token masks");
    return tokenMask_;
  }
  [[nodiscard]] bool anyConstrained(size_t lanes) const {
    for (size_t l = 0; l < lanes && l < constrained_.size(); ++l)
      if (constrained_[l]) return true;
    return false;
  }
  void setPenalties(uint32_t lane, ops::SamplingPenalties penalties) {
    if (lane >= penalties_.size()) throw std::invalid_argument("penalties of a lane past the driver's");
    penalties_[lane] = penalties;
    if (penalties.active()) (void)words();
  }
  void setCutoff(uint32_t lane, std::optional<ops::ThinkingCutoff> cutoff) {
    if (lane >= cutoffs_.size()) throw std::invalid_argument("a thinking cutoff of a lane past the driver's");
    cutoffs_[lane] = std::move(cutoff);
  }
  // The table: lane l's row is words [l * vocabulary, (l + 1) * vocabulary). A request that takes a lane uploads its row
  // (ops::Sampling::rebuildPenaltyWords).
  const hip::Buffer &words() {
    if (!words_) words_ = backend_.allocateBuffer(uint64_t{penalties_.size()} * vocabulary_ * 4, hip::BufferStorage::Private, "penalty words");
    return words_;
  }
  // The step's lanes take their penalties and cutoffs; true when any lane's penalties are active.
  bool apply(std::vector<ops::SamplingPolicy> &policies) const {
    bool any = false;
    for (size_t l = 0; l < policies.size() && l < penalties_.size(); ++l) {
      policies[l].thinkingCutoff = cutoffs_[l];
      policies[l].constrained = constrained_[l];
      policies[l].excludesStopTokens = excludesStop_[l];
      policies[l].penalties = penalties_[l];
      any = any || penalties_[l].active();
    }
    return any;
  }
  [[nodiscard]] ops::PenaltyTable table() { return {words(), rows_}; }
  [[nodiscard]] std::vector<bool> penalized(size_t lanes) const {
    std::vector<bool> out(lanes);
    for (size_t l = 0; l < lanes && l < penalties_.size(); ++l) out[l] = penalties_[l].active();
    return out;
  }

private:
  hip::Backend &backend_;
  uint32_t vocabulary_;
  std::vector<ops::SamplingPenalties> penalties_;
  std::vector<std::optional<ops::ThinkingCutoff>> cutoffs_;
  std::vector<bool> constrained_, excludesStop_;
  StopTokens stopTokens_{};
  std::vector<uint32_t> rows_;
  hip::Buffer words_, tokenMask_;
};

} // namespace splash::model
