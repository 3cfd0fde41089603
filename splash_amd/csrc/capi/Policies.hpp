// The C structs of a lane's sampling policy as the operators' types.
#pragma once
#include "ops/Sampling.hpp"
#include "splash_ops.h"

#include <optional>
#include <stdexcept>

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

} // namespace splash::capi
