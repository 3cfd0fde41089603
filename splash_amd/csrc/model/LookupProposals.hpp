// Proposals a request's own tokens make (prompt lookup; the reference's model::LookupIndex, LookupProposals.hpp:17-105):
// where the latest tokens occurred before, the tokens that followed them there are a guess at what follows now, which a
// decode cycle verifies beside the draft's as the host chain of the lane's tree (ops::DraftTreeLane::chain).
//
// The match after the latest token: the longest suffix of the tokens, counted up to kLongestMatch, that also ends at an
// earlier token (occurrences may overlap), none shorter than kMinimumMatch, and of its earlier occurrences the most
// recent. A suffix automaton over the tokens gives it as each token is appended: the state of a string knows every
// position the string ends at, the suffixes of the tokens lie along the suffix links of the whole string's state, and a
// state's most recent end is kept exact for the states that hold a string of at most kLongestMatch tokens, which are the
// at most kLongestMatch states above the one of the last kLongestMatch tokens. An append is amortized constant work
// plus that walk.
#pragma once
#include <cstdint>
#include <span>
#include <unordered_map>
#include <vector>

namespace splash::model {

class LookupIndex final {
public:
  static constexpr uint32_t kMinimumMatch = 3;
  static constexpr uint32_t kLongestMatch = 64;

  struct Match final {
    uint32_t length = 0;   // kMinimumMatch..kLongestMatch; 0: the latest tokens occurred nowhere before
    uint32_t end = 0;      // the index of the earlier occurrence's last token
    bool operator==(const Match &) const = default;
  };

  LookupIndex();
  void append(std::span<const uint32_t> tokens);
  [[nodiscard]] std::span<const uint32_t> tokens() const noexcept { return tokens_; }
  [[nodiscard]] Match match() const noexcept { return match_; }
  // Up to `count` tokens that followed the match's occurrence, at most as far as the latest token; empty without a match.
  [[nodiscard]] std::span<const uint32_t> proposals(uint32_t count) const noexcept;

private:
  static constexpr uint32_t kNone = UINT32_MAX;
  struct State final {
    uint32_t longest = 0;    // the longest string of the class; its shortest is one longer than its link's longest
    uint32_t link = kNone;   // the class of the longest suffix that ends at more positions
    uint32_t recent = 0;     // the latest position its strings end at (exact while it holds a string of <= kLongestMatch)
    uint32_t steps = kNone;  // its first step (Step::sibling chains the others)
  };
  struct Step final {
    uint32_t token = 0, to = 0, sibling = kNone;
  };
  [[nodiscard]] uint32_t next(uint32_t state, uint32_t token) const;
  void setNext(uint32_t state, uint32_t token, uint32_t to);
  void extend(uint32_t token);

  std::vector<uint32_t> tokens_;
  std::vector<State> states_;
  std::vector<Step> steps_;
  std::unordered_map<uint64_t, uint32_t> stepOf_;   // (state, token) -> its step
  uint32_t whole_ = 0;    // the class of all the tokens
  uint32_t capped_ = 0;   // the class of their last min(size, kLongestMatch) tokens
  Match match_;
};

// How a lookup token compares with the draft's candidates at its depth (LookupAgreement, LookupProposals.hpp:107-118):
// the lane's candidates at each proposal position, `perPosition` a position, most likely first.
enum class LookupAgreement : uint8_t { Top, Candidate, Absent, Unknown };
[[nodiscard]] LookupAgreement lookupAgreement(uint32_t token, uint32_t depth, std::span<const uint32_t> candidates, uint32_t perPosition);

} // namespace splash::model
