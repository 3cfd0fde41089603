// TEST INFRASTRUCTURE ONLY: the CPU statement of the draft selector's tree growth (draft_select_tree,
// runtime/metal/kernels/decode/sampling.metal:1357-1766; its parameters, runtime/metal/abi/Sampling.h:209-255). One lane a call.
// The product path never links this file.
//
// The rule: a lattice of every proposal position's candidates' probabilities after each predecessor candidate (the softmax
// at temperature 1 of unary + edge scores) and each predecessor's four likeliest; then a best-first growth over steps
// ("entries") from a row to a token one deeper, the largest estimate first, the earlier-made entry first among equal ones.
// A draft row pushes its drawn children (a greedy lane's likeliest, a sampled lane's Gumbel-top-k draws from q_T), each
// estimated min(sigmoid(slope * logit(q) + intercept[position]), cap) times its parent's score and at most the sibling
// drawn before it, the caps being what the row's host-chain child and the siblings drawn before left of 1; a row on the
// host chain's path pushes the chain's next token at its rate. One row a token path.
#include "oracle.h"

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <limits>
#include <vector>

namespace {
constexpr uint32_t kPositions = 7, kCandidates = 16, kChildren = 4, kRows = 16, kNone = 0xFF;

uint64_t mix(uint64_t v) {  // the splitmix64 finalizer (sampling.metal:1509-1513)
  v = (v ^ (v >> 30)) * 0xbf58476d1ce4e5b9ull;
  v = (v ^ (v >> 27)) * 0x94d049bb133111ebull;
  return v ^ (v >> 31);
}
uint64_t child_key(uint64_t parent, uint32_t token) { return mix(parent + 0x9e3779b97f4a7c15ull * (uint64_t(token) + 1)); }
float gumbel(uint64_t key, uint32_t token) {  // sampling.metal:1525-1529: a uniform of the hash's top 23 bits, inside (0, 1)
  const uint64_t v = mix(key ^ 0xd1b54a32d192ed03ull * (uint64_t(token) + 1));
  const float uniform = (float(v >> 41) + 0.5f) * 0x1p-23f;
  return -std::log(-std::log(uniform));
}
float estimate_of(const OrcDraftTreeLane &lane, float q, uint32_t position) {  // sampling.metal:1472-1480
  q = std::min(std::max(q, 1.0e-6f), 1.0f - 1.0e-6f);
  const float z = lane.slope * std::log(q / (1.0f - q)) + lane.intercept[position];
  return 1.0f / (1.0f + std::exp(-z));
}

struct Entry {
  float score;
  bool chain;
  uint32_t parent, position, index;
  bool live;
};
} // namespace

extern "C" void orc_draft_tree(const uint32_t *candidates, const float *unary, const float *edges, const uint32_t *chain_tokens,
                               const float *chain_rates, const OrcDraftTreeLane *lane_in, uint32_t *tokens, OrcTreeRow *tree,
                               float *scores, uint32_t *size, uint8_t *draws, float *next, float *caps) {
  const OrcDraftTreeLane &lane = *lane_in;
  // ---- the lattice (sampling.metal:1655-1692)
  static thread_local float probability[kPositions][kCandidates][kCandidates];
  static thread_local uint8_t likeliest[kPositions][kCandidates][kChildren];
  for (uint32_t p = 0; p < kPositions; ++p)
    for (uint32_t pred = 0; pred < kCandidates; ++pred) {
      if (p == 0 && pred != 0) continue;
      float score[kCandidates];
      for (uint32_t i = 0; i < kCandidates; ++i) score[i] = unary[p * kCandidates + i] + edges[(p * kCandidates + pred) * kCandidates + i];
      float best = score[0];
      for (uint32_t i = 1; i < kCandidates; ++i) best = std::max(best, score[i]);
      float weight[kCandidates], mass = 0.f;
      for (uint32_t i = 0; i < kCandidates; ++i) {
        weight[i] = std::exp(score[i] - best);
        mass += weight[i];
      }
      for (uint32_t i = 0; i < kCandidates; ++i) probability[p][pred][i] = weight[i] / mass;
      uint32_t taken = 0;
      for (uint32_t c = 0; c < kChildren; ++c) {
        uint32_t pick = kCandidates;
        for (uint32_t i = 0; i < kCandidates; ++i)
          if (!(taken >> i & 1u) && (pick == kCandidates || score[i] > score[pick])) pick = i;
        taken |= 1u << pick;
        likeliest[p][pred][c] = uint8_t(pick);
      }
    }
  auto agreement = [&](uint32_t token, uint32_t depth) -> uint32_t {  // sampling.metal:1486-1496
    if (depth >= kPositions) return 3;
    if (token == candidates[depth * kCandidates]) return 0;
    for (uint32_t i = 1; i < kCandidates; ++i)
      if (token == candidates[depth * kCandidates + i]) return 1;
    return 2;
  };
  auto chain_rate = [&](uint32_t depth) { return chain_rates[depth * 4 + agreement(chain_tokens[depth], depth)]; };

  // ---- the rows
  struct Row {
    uint32_t token, ancestors, parent, depth;
    bool onChain;
    float q, estimate, cap;
    uint64_t key;
    uint8_t draw[kChildren];
    float left[kChildren], next[kCandidates];
  };
  std::vector<Row> rows;
  std::vector<Entry> entries;
  auto fresh = [](Row &r) {
    for (uint32_t c = 0; c < kChildren; ++c) r.draw[c] = kNone, r.left[c] = 0.f;
    for (uint32_t i = 0; i < kCandidates; ++i) r.next[i] = 0.f;
  };
  // A draft row's children at `position`, after its candidate `predecessor` (sampling.metal:1560-1613).
  auto expand = [&](uint32_t row, uint32_t position, uint32_t predecessor, float score, bool hasChain, uint32_t chainToken, float chainRate) {
    const float *q = probability[position][predecessor];
    const float T = lane.temperature;
    float top = 0.f;
    for (uint32_t i = 0; i < kCandidates; ++i) top = std::max(top, q[i]);
    float mass = 0.f;
    for (uint32_t i = 0; i < kCandidates; ++i) {
      const float w = T == 0.f || !(q[i] > 0.f) ? q[i] : std::exp((std::log(q[i]) - std::log(top)) / T);
      rows[row].next[i] = w;
      mass += w;
    }
    for (uint32_t i = 0; i < kCandidates; ++i) rows[row].next[i] /= mass;
    float keys[kCandidates];
    for (uint32_t i = 0; i < kCandidates; ++i)
      keys[i] = T > 0.f && rows[row].next[i] > 0.f ? std::log(rows[row].next[i]) + gumbel(rows[row].key, candidates[position * kCandidates + i])
                                                   : -std::numeric_limits<float>::infinity();
    uint32_t taken = 0;
    float bound = score, left = 1.0f - chainRate, reserved = chainRate;
    for (uint32_t child = 0; child < lane.children; ++child) {
      uint32_t drawn = kCandidates;
      if (T == 0.f) {
        const uint32_t l = likeliest[position][predecessor][child];
        if (q[l] > 0.f) drawn = l;
      } else {
        for (uint32_t i = 0; i < kCandidates; ++i)
          if (!(taken >> i & 1u) && keys[i] > -std::numeric_limits<float>::infinity() && (drawn == kCandidates || keys[i] > keys[drawn])) drawn = i;
      }
      if (drawn == kCandidates) return;
      taken |= 1u << drawn;
      const bool joins = hasChain && candidates[position * kCandidates + drawn] == chainToken;
      const float cap = joins ? left + reserved : left;
      rows[row].draw[child] = uint8_t(drawn);
      rows[row].left[child] = cap;
      const float own = std::min(estimate_of(lane, rows[row].next[drawn], position), cap);
      left = joins ? cap - std::max(own, reserved) : left - own;
      reserved = joins ? 0.f : reserved;
      bound = std::min(bound, score * own);
      entries.push_back({bound, false, row, position, drawn, true});
    }
  };
  auto cap_of = [&](uint32_t parent, uint32_t index) {
    for (uint32_t c = 0; c < kChildren; ++c)
      if (rows[parent].draw[c] == index) return rows[parent].left[c];
    return 1.0f;
  };

  Row anchor{};
  anchor.token = lane.anchor;
  anchor.ancestors = 1;
  anchor.parent = 0xFFFF;
  anchor.depth = 0;
  anchor.onChain = true;
  anchor.q = anchor.estimate = anchor.cap = 1.0f;
  anchor.key = uint64_t(lane.noise[1]) << 32 | lane.noise[0];
  fresh(anchor);
  rows.push_back(anchor);
  const uint32_t deepest = lane.depth, chained = lane.chain;
  if (deepest > 0) {
    const float rate = chained ? chain_rate(0) : 0.f;
    expand(0, 0, 0, 1.0f, chained != 0, chained ? chain_tokens[0] : 0u, rate);
    if (chained) entries.push_back({rate, true, 0, 0, 0, true});
  }
  const uint32_t most = std::min(kRows, deepest + 1);
  while (rows.size() < most) {
    // the largest score, the earliest entry among equal ones
    int best = -1;
    for (size_t e = 0; e < entries.size(); ++e)
      if (entries[e].live && (best < 0 || entries[e].score > entries[size_t(best)].score)) best = int(e);
    if (best < 0) break;
    const Entry entry = entries[size_t(best)];
    entries[size_t(best)].live = false;
    const uint32_t parent = entry.parent, position = entry.position, index = entry.index;
    const uint32_t token = entry.chain ? chain_tokens[position] : candidates[position * kCandidates + index];
    uint32_t row = 0;
    for (uint32_t other = 1; other < rows.size() && !row; ++other)
      if (rows[other].parent == parent && rows[other].token == token) row = other;
    if (!row) {
      row = uint32_t(rows.size());
      Row r{};
      r.token = token;
      r.ancestors = rows[parent].ancestors | 1u << row;
      r.parent = parent;
      r.depth = position + 1;
      r.onChain = rows[parent].onChain && position < chained && token == chain_tokens[position];
      r.q = entry.chain ? -1.0f : rows[parent].next[index];
      r.estimate = entry.score;
      r.cap = entry.chain ? 1.0f : cap_of(parent, index);
      r.key = child_key(rows[parent].key, token);
      fresh(r);
      rows.push_back(r);
    } else if (!entry.chain && rows[row].q < 0.f) {
      rows[row].q = rows[parent].next[index];
      rows[row].cap = cap_of(parent, index);
    }
    if (position + 1 >= deepest) continue;
    const bool chainChild = rows[row].onChain && position + 1 < chained;
    if (!entry.chain && position + 1 < kPositions)
      expand(row, position + 1, index, entry.score, chainChild, chainChild ? chain_tokens[position + 1] : 0u,
             chainChild ? chain_rate(position + 1) : 0.f);
    else if (entry.chain && position + 1 < chained)
      entries.push_back({entry.score * chain_rate(position + 1), true, row, position + 1, 0, true});
  }
  *size = uint32_t(rows.size());
  for (uint32_t r = 0; r < rows.size(); ++r) {
    tokens[r] = rows[r].token;
    tree[r] = {rows[r].ancestors, uint16_t(rows[r].parent), uint16_t(rows[r].depth)};
    scores[2 * r] = rows[r].q;
    scores[2 * r + 1] = rows[r].estimate;
    caps[r] = rows[r].cap;
    for (uint32_t c = 0; c < kChildren; ++c) draws[r * kChildren + c] = rows[r].draw[c];
    for (uint32_t i = 0; i < kCandidates; ++i) next[r * kCandidates + i] = rows[r].next[i];
  }
}
