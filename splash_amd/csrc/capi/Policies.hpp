// The C structs of a lane's sampling policy as the operators' types.
#pragma once
#include "ops/Sampling.hpp"
#include "splash_ops.h"

#include <optional>
#include <stdexcept>
#include <vector>

namespace splash::capi {

inline std::optional<ops::ThinkingCutoff> cutoffOf(const spo_thinking_cutoff *c) {
  if (!c || !c->active) return std::nullopt;
  if (c->count > 16) throw std::invalid_argument("a thinking end holds at most 16 tokens here");
  ops::ThinkingCutoff out;
  out.row = c->row;
  out.end.assign(c->end, c->end + c->count);
  out.alsoEnds = c->also_ends;
  out.waitsForMask = c->waits_for_mask != 0;
  return out;
}

// The lanes of spo_sampling_add_penalties / _add_penalty_count as the operator takes them.
struct PenalizedLanes {
  std::vector<ops::LaneRows> rows;
  std::vector<ops::SamplingPolicy> policies;
  std::vector<uint32_t> tableRows;
  std::vector<bool> active;
};
inline PenalizedLanes penalizedLanes(const spo_lane_rows *lanes, const spo_sampling_penalties *penalties, uint32_t count) {
  PenalizedLanes out;
  for (uint32_t i = 0; i < count; ++i) {
    out.rows.push_back({lanes[i].first, lanes[i].rows});
    ops::SamplingPolicy policy;
    policy.penalties = {penalties[i].repetition, penalties[i].presence, penalties[i].frequency};
    out.policies.push_back(policy);
    out.tableRows.push_back(penalties[i].table_row);
    out.active.push_back(policy.penalties.active());
  }
  return out;
}

} // namespace splash::capi
