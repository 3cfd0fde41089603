#include "model/LookupProposals.hpp"

#include <algorithm>

namespace splash::model {

LookupIndex::LookupIndex() { states_.push_back({}); }

uint32_t LookupIndex::next(uint32_t state, uint32_t token) const {
  const auto it = stepOf_.find((uint64_t{state} << 32) | token);
  return it == stepOf_.end() ? kNone : steps_[it->second].to;
}

void LookupIndex::setNext(uint32_t state, uint32_t token, uint32_t to) {
  const auto [it, fresh] = stepOf_.try_emplace((uint64_t{state} << 32) | token, uint32_t(steps_.size()));
  if (!fresh) {
    steps_[it->second].to = to;
    return;
  }
  steps_.push_back({token, to, states_[state].steps});
  states_[state].steps = it->second;
}

std::span<const uint32_t> LookupIndex::proposals(uint32_t count) const noexcept {
  if (!match_.length) return {};
  const size_t first = size_t{match_.end} + 1;
  return std::span<const uint32_t>(tokens_).subspan(first, std::min<size_t>(count, tokens_.size() - first));
}

void LookupIndex::append(std::span<const uint32_t> tokens) {
  for (const uint32_t token : tokens) extend(token);
}

void LookupIndex::extend(uint32_t token) {
  const uint32_t position = uint32_t(tokens_.size());
  const uint32_t cappedLength = std::min(position, kLongestMatch);   // of the tokens before this one
  tokens_.push_back(token);

  // The automaton's step: a class for the whole string, reached from the class of every suffix that had no such step;
  // where a suffix's step leads to a class with longer strings too, that class parts into those that now end here (the
  // copy) and those that do not.
  const uint32_t added = uint32_t(states_.size());
  states_.push_back({states_[whole_].longest + 1, kNone, position, kNone});
  uint32_t from = whole_;
  for (; from != kNone && next(from, token) == kNone; from = states_[from].link) setNext(from, token, added);
  if (from == kNone) {
    states_[added].link = 0;
  } else {
    const uint32_t target = next(from, token);
    if (states_[target].longest == states_[from].longest + 1) {
      states_[added].link = target;
    } else {
      const uint32_t copy = uint32_t(states_.size());
      states_.push_back({states_[from].longest + 1, states_[target].link, states_[target].recent, kNone});
      for (uint32_t step = states_[target].steps; step != kNone; step = steps_[step].sibling) setNext(copy, steps_[step].token, steps_[step].to);
      for (uint32_t walk = from; walk != kNone && next(walk, token) == target; walk = states_[walk].link) setNext(walk, token, copy);
      states_[target].link = copy;
      states_[added].link = copy;
      // the last tokens' class, if it parted, is the part that holds their length
      if (capped_ == target && cappedLength <= states_[copy].longest) capped_ = copy;
    }
  }
  whole_ = added;

  // The class of the last min(size, kLongestMatch) tokens: one step on from that of the tokens before; where that made
  // the string one token too long, its suffix of kLongestMatch tokens lies in the same class or is its link's longest.
  capped_ = next(capped_, token);
  if (cappedLength == kLongestMatch && states_[states_[capped_].link].longest >= kLongestMatch) capped_ = states_[capped_].link;

  // The match: the longest suffix that ends elsewhere is the link's longest string; counted up to kLongestMatch it lies
  // in the last tokens' class. Read before this position enters the classes' latest ends.
  match_ = {};
  const uint32_t elsewhere = states_[states_[added].link].longest;
  if (elsewhere >= kMinimumMatch) {
    const uint32_t holder = elsewhere <= kLongestMatch ? states_[added].link : capped_;
    match_ = {std::min(elsewhere, kLongestMatch), states_[holder].recent};
  }
  for (uint32_t state = capped_; state != kNone && state != 0; state = states_[state].link) states_[state].recent = position;
}

LookupAgreement lookupAgreement(uint32_t token, uint32_t depth, std::span<const uint32_t> candidates, uint32_t perPosition) {
  if (!perPosition || (size_t{depth} + 1) * perPosition > candidates.size()) return LookupAgreement::Unknown;
  const std::span<const uint32_t> position = candidates.subspan(size_t{depth} * perPosition, perPosition);
  if (position.front() == token) return LookupAgreement::Top;
  return std::find(position.begin(), position.end(), token) != position.end() ? LookupAgreement::Candidate : LookupAgreement::Absent;
}

} // namespace splash::model
