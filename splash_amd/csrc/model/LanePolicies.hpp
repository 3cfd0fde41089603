// What a driver's lanes add to their sampling policies between steps: each dispatch lane's thinking cutoff
// (ops::ThinkingCutoff), its penalties (ops::SamplingPenalties) and its row of the penalty table the driver owns, `vocabulary` words a lane in device memory, allocated (zeroed) when a lane first takes
// active penalties. The reference's model keeps the table per state lane and the engine counts a step's tokens into it
// on the host (Sampling.hpp:85-91, Sampling::countPenaltyTokens); here a step that commits counts them on the device.
#pragma once
#include "hip/Backend.hpp"
#include "ops/Sampling.hpp"

#include <numeric>
#include <optional>
#include <stdexcept>
#include <vector>

namespace splash::model {

class LanePolicies final {
public:
  LanePolicies(hip::Backend &backend, uint32_t lanes, uint32_t vocabulary)
      : backend_(backend), vocabulary_(vocabulary), penalties_(lanes), cutoffs_(lanes), rows_(lanes) {
    std::iota(rows_.begin(), rows_.end(), 0u);
  }
  void set(uint32_t lane, ops::SamplingPenalties penalties) {
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
      policies[l].penalties = penalties_[l];
      any = any || penalties_[l].active();
    }
    return any;
  }
  [[nodiscard]] ops::PenaltyTable table() { return {words(), rows_}; }
  [[nodiscard]] std::vector<bool> active(size_t lanes) const {
    std::vector<bool> out(lanes);
    for (size_t l = 0; l < lanes && l < penalties_.size(); ++l) out[l] = penalties_[l].active();
    return out;
  }

private:
  hip::Backend &backend_;
  uint32_t vocabulary_;
  std::vector<ops::SamplingPenalties> penalties_;
  std::vector<std::optional<ops::ThinkingCutoff>> cutoffs_;
  std::vector<uint32_t> rows_;
  hip::Buffer words_;
};

} // namespace splash::model
