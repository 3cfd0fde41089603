#include "model/StepResults.hpp"

#include <algorithm>
#include <bit>
#include <stdexcept>

namespace splash::model {

void validateStepResults(const std::vector<StepLane> &lanes, const std::vector<StepLaneResult> &results, uint32_t stepRows,
                         uint32_t vocabulary) {
  if (lanes.empty() || lanes.size() != results.size()) throw std::invalid_argument("a step's lanes and their results come in pairs");
  for (size_t i = 0; i < lanes.size(); ++i) {
    const StepLane &lane = lanes[i];
    const StepLaneResult &r = results[i];
    const std::string who = "lane " + std::to_string(i) + ": ";
    if (!lane.rows || lane.rows > 16 || uint64_t{lane.first} + lane.rows > stepRows)
      throw hip::BackendError(who + "its rows are not rows of the step");
    if (!r.tokens) throw std::invalid_argument(who + "no tokens to check");
    const uint32_t most = std::min(lane.rows, lane.remaining);
    const bool pastRows = lane.rows < 32 && (r.retainedRows >> lane.rows) != 0;
    if (!r.retained || r.retained > most || std::popcount(r.retainedRows) != static_cast<int>(r.retained) ||
        !(r.retainedRows & 1u) || pastRows)
      throw hip::BackendError(who + "invalid retention (retained " + std::to_string(r.retained) + " of " + std::to_string(lane.rows) +
                              " rows, path mask " + std::to_string(r.retainedRows) + ")");
    if (r.accepted >= lane.rows || r.accepted > r.retained)
      throw hip::BackendError(who + "accepted more than the draft proposed (" + std::to_string(r.accepted) + ")");
    for (uint32_t k = 0; k < r.retained; ++k)
      if (r.tokens[k] >= vocabulary)
        throw hip::BackendError(who + "retained token " + std::to_string(k) + " is not of the vocabulary: its logits row had no selectable token");
  }
}

void readStepResults(const std::vector<StepLane> &lanes, const hip::Buffer &tokens, const hip::Buffer &retained,
                     const hip::Buffer &accepted, const hip::Buffer &retainedRows, uint32_t vocabulary, uint32_t *tokensOut,
                     uint32_t *retainedOut, uint32_t *acceptedOut, uint32_t *retainedRowsOut) {
  const auto words = [](const hip::Buffer &b, const char *what) {
    const uint32_t *p = static_cast<const uint32_t *>(b.contents());
    if (!p) throw hip::BackendError(std::string(what) + " is not host-visible");
    return p;
  };
  const uint32_t *t = words(tokens, "selected tokens"), *r = words(retained, "retained counts"), *a = words(accepted, "accepted counts"),
                 *m = words(retainedRows, "retained rows");
  uint32_t stepRows = 0;
  for (const StepLane &lane : lanes) stepRows = std::max(stepRows, lane.first + lane.rows);
  if (uint64_t{stepRows} * 4 > tokens.sizeBytes() || lanes.size() * 4 > retained.sizeBytes())
    throw std::invalid_argument("more lanes or rows than the driver holds");
  std::vector<StepLaneResult> results;
  for (size_t i = 0; i < lanes.size(); ++i) results.push_back({r[i], a[i], m[i], t + lanes[i].first});
  validateStepResults(lanes, results, stepRows, vocabulary);
  for (size_t i = 0; i < lanes.size(); ++i) {
    std::copy(t + lanes[i].first, t + lanes[i].first + lanes[i].rows, tokensOut + lanes[i].first);
    retainedOut[i] = r[i];
    acceptedOut[i] = a[i];
    retainedRowsOut[i] = m[i];
  }
}

} // namespace splash::model
