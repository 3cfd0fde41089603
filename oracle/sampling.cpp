// CPU oracle, acceptance of a verify block (test infrastructure only; see oracle.h).
#include "oracle.h"
#include "common.hpp"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>
#include <vector>

using namespace orc;

namespace {
bool unselectable(float v) { return !(v > -std::numeric_limits<float>::infinity()); }  // NaN or -inf
constexpr uint32_t kShards = 32, kThreads = 256, kRanges = 256;

struct Mass { float maximum, sum; };
// sampling.metal:122-154 merge_masses
Mass merge(Mass a, Mass b, float inv) {
  const float m = std::max(a.maximum, b.maximum);
  if (m == -std::numeric_limits<float>::infinity()) return {m, 0.f};
  const float sa = a.maximum == -std::numeric_limits<float>::infinity() ? 0.f : a.sum * std::exp((a.maximum - m) * inv);
  const float sb = b.maximum == -std::numeric_limits<float>::infinity() ? 0.f : b.sum * std::exp((b.maximum - m) * inv);
  return {m, sa + sb};
}
// The row's (max, total): each thread of each shard folds its tokens in id order (shard * 256 + tid
// + n * shards * 256), a wavefront's lanes merge by butterfly, its four wavefronts in order, the
// shards in order (sampling.metal:102-154 on 64-lane wavefronts).
Mass rowMass(const float *x, uint32_t V, float inv) {
  Mass row{0, 0};
  for (uint32_t shard = 0; shard < kShards; ++shard) {
    Mass thread[kThreads];
    for (uint32_t t = 0; t < kThreads; ++t) {
      Mass mine{-std::numeric_limits<float>::infinity(), 0.f};
      for (uint32_t token = shard * 256 + t; token < V; token += kShards * 256)
        if (!unselectable(x[token])) mine = merge(mine, Mass{x[token], 1.0f}, inv);
      thread[t] = mine;
    }
    Mass waves[4];
    for (int w = 0; w < 4; ++w) {
      Mass lane[64];
      for (int l = 0; l < 64; ++l) lane[l] = thread[64 * w + l];
      for (int o = 32; o > 0; o >>= 1) {
        Mass next[64];
        for (int l = 0; l < 64; ++l) next[l] = merge(lane[l], lane[l ^ o], inv);
        for (int l = 0; l < 64; ++l) lane[l] = next[l];
      }
      waves[w] = lane[0];
    }
    Mass all = waves[0];
    for (int w = 1; w < 4; ++w) all = merge(all, waves[w], inv);
    row = shard ? merge(row, all, inv) : all;
  }
  return row;
}
float tokenWeight(float logit, Mass m, float inv) { return unselectable(logit) ? 0.f : std::exp((logit - m.maximum) * inv); }
// sampling.metal:197-207: the order of the logits as an unsigned key
uint32_t logitKey(float value) {
  uint32_t bits;
  std::memcpy(&bits, &value, 4);
  bits = (bits << 1) ? bits : 0u;
  return (bits & 0x80000000u) ? ~bits : bits | 0x80000000u;
}
struct OrderEnd { uint32_t key, last; };
bool atOrBefore(uint32_t key, uint32_t token, OrderEnd end) { return key > end.key || (key == end.key && token <= end.last); }
// A row's distribution: its maximum, the mass it keeps (m.sum) and the last token it keeps.
struct Kept { Mass m; OrderEnd end; };
float keptWeight(float logit, uint32_t token, const Kept &k, float inv) {
  if (unselectable(logit) || !atOrBefore(logitKey(logit), token, k.end)) return 0.f;
  return std::exp((logit - k.m.maximum) * inv);
}
float residualOf(float logit, uint32_t token, float q, const Kept &k, float inv, bool rejected) {
  const float w = keptWeight(logit, token, k, inv);
  return rejected ? std::max(w / k.m.sum - q, 0.f) : w;
}
void note(double *closeness, double value, double threshold);
// distribution_end (sampling.metal:603-670) by a sort: the tokens in the order of the logits (larger
// first, among equals the smaller id first); min_p keeps those at or above the logit that weighs min_p
// of the heaviest, top_k the first top_k of those, top_p of those the tokens up to the one at which
// their mass first exceeds top_p of the kept mass. Masses are summed in fp64 in that order; closeness
// takes the relative distance of the nucleus from the masses either side of its last token.
Kept distributionEnd(const float *x, uint32_t V, const OrcSamplingPolicy &policy, uint32_t *count, double *closeness) {
  const float inv = 1.0f / policy.temperature;
  Kept kept{rowMass(x, V, inv), {0u, 0u}};
  std::vector<std::pair<uint32_t, uint32_t>> order;  // (key, id)
  for (uint32_t t = 0; t < V; ++t)
    if (!unselectable(x[t])) order.push_back({logitKey(x[t]), t});
  std::sort(order.begin(), order.end(), [](const auto &a, const auto &b) { return a.first != b.first ? a.first > b.first : a.second < b.second; });
  size_t keep = order.size();
  const bool cuts = policy.min_p > 0.f || (policy.top_k && policy.top_k < V) || policy.top_p < 1.f;
  if (count) *count = uint32_t(keep);
  if (!cuts) return kept;
  if (policy.min_p > 0.f) {
    const uint32_t lowest = logitKey(std::min(kept.m.maximum + policy.temperature * std::log(policy.min_p), kept.m.maximum));
    size_t n = 0;
    while (n < order.size() && order[n].first >= lowest) ++n;
    if (n < order.size()) { keep = n; kept.end = {lowest, 0xFFFFFFFFu}; }
  }
  if (policy.top_k && policy.top_k < keep) {
    keep = policy.top_k;
    kept.end = {order[keep - 1].first, order[keep - 1].second};
  }
  auto weight = [&](size_t i) { return double(tokenWeight(x[order[i].second], kept.m, inv)); };
  double mass = 0;
  for (size_t i = 0; i < keep; ++i) mass += weight(i);
  if (policy.top_p < 1.f) {
    const double nucleus = double(policy.top_p * float(mass));
    double walked = 0;
    for (size_t i = 0; i < keep; ++i) {
      const double before = walked;
      walked += weight(i);
      if (walked > nucleus) {
        note(closeness, walked, nucleus);
        if (i) note(closeness, before, nucleus);
        keep = i + 1;
        kept.end = {order[i].first, order[i].second};
        mass = walked;
        break;
      }
    }
  }
  kept.m.sum = float(mass);
  if (count) *count = uint32_t(keep);
  // An end after the last token of its key's run is written with every id (the same kept set).
  if (kept.end.key && (keep == order.size() || order[keep].first != kept.end.key)) kept.end.last = 0xFFFFFFFFu;
  return kept;
}
void note(double *closeness, double value, double threshold) {
  if (!closeness) return;
  const double scale = std::max(std::fabs(value), std::fabs(threshold));
  const double distance = scale > 0 ? std::fabs(value - threshold) / scale : 1.0;
  *closeness = std::min(*closeness, distance);
}
} // namespace

extern "C" {

// sampling.metal:1050-1052 top_beats, :1099-1232 draft_select_top16_sharded, :1236-1264 top16_merge_shards: a sorted list
// of sixteen, begun as empty entries (-infinity, token 0xffffffff), takes every column that beats its last entry; shards
// and their merge select what one list over the whole row does. A column's token is itself below `leading`, else
// column - leading + trailing. Rows 1-7 of a lane's eight query rows are its proposal positions.
void orc_draft_candidates(const float *logits, uint32_t lanes, uint32_t columns, uint32_t leading, uint32_t trailing,
                          uint32_t *candidates, float *unary) {
  constexpr uint32_t K = 16, kPositions = 7, kQueryRows = 8;
  for (uint32_t row = 0; row < lanes * kPositions; ++row) {
    const float *x = logits + (size_t(row / kPositions) * kQueryRows + row % kPositions + 1) * columns;
    float values[K];
    uint32_t ids[K];
    for (uint32_t i = 0; i < K; ++i) values[i] = -INFINITY, ids[i] = 0xffffffffu;
    const auto beats = [](float value, uint32_t token, float other, uint32_t other_token) {
      return value > other || (value == other && token < other_token);
    };
    for (uint32_t column = 0; column < columns; ++column) {
      if (!beats(x[column], column, values[K - 1], ids[K - 1])) continue;
      uint32_t at = K - 1;
      for (; at > 0 && beats(x[column], column, values[at - 1], ids[at - 1]); --at) values[at] = values[at - 1], ids[at] = ids[at - 1];
      values[at] = x[column], ids[at] = column;
    }
    for (uint32_t i = 0; i < K; ++i) {
      candidates[row * K + i] = ids[i] < leading || ids[i] == 0xffffffffu ? ids[i] : ids[i] - leading + trailing;
      unary[row * K + i] = values[i];
    }
  }
}

// sampling.metal:1271-1356 draft_select_edges: edges[row][predecessor][candidate] = sum over the rank of 256 of
// (predecessor_codebook[predecessor token] * hidden[row]) * successor_codebook[candidate token], the factors bf16, each
// product rounded to fp32; tokens clamp to the vocabulary. The reference leaves the order of the sum to its simdgroup
// reduction; this one adds in fp64. Position 0 scores its anchor's row alone.
void orc_draft_edges(const uint32_t *candidates, const uint32_t *anchors, uint32_t lanes, uint32_t vocabulary, const uint16_t *hidden,
                     const uint16_t *predecessor_codebook, const uint16_t *successor_codebook, float *edges) {
  constexpr uint32_t K = 16, kPositions = 7, kQueryRows = 8, kRank = 256;
  const auto f = [](uint16_t bits) {
    const uint32_t u = uint32_t{bits} << 16;
    float v;
    std::memcpy(&v, &u, 4);
    return v;
  };
  for (uint32_t row = 0; row < lanes * kPositions; ++row) {
    const uint32_t lane = row / kPositions, position = row % kPositions;
    const uint16_t *h = hidden + (size_t(lane) * kQueryRows + position + 1) * kRank;
    for (uint32_t predecessor = 0; predecessor < (position ? K : 1u); ++predecessor) {
      const uint32_t before = std::min(position ? candidates[(row - 1) * K + predecessor] : anchors[lane], vocabulary - 1);
      for (uint32_t candidate = 0; candidate < K; ++candidate) {
        const uint32_t token = std::min(candidates[row * K + candidate], vocabulary - 1);
        double sum = 0.0;
        for (uint32_t d = 0; d < kRank; ++d) {
          const float context = f(predecessor_codebook[size_t(before) * kRank + d]) * f(h[d]);
          sum += double(context * f(successor_codebook[size_t(token) * kRank + d]));
        }
        edges[(size_t(row) * K + predecessor) * K + candidate] = float(sum);
      }
    }
  }
}

void orc_draft_verify_rows(const uint32_t *tree_tokens, const struct OrcTreeRow *trees, const float *scores, const uint32_t *sizes,
                           uint32_t lanes, uint32_t rows, uint32_t lane_cap, float floor, uint32_t *tokens, struct OrcTreeRow *tree,
                           uint32_t *lane_rows, uint32_t *sources) {
  constexpr uint32_t kRows = 16;
  std::vector<float> estimates;
  std::vector<uint32_t> owners;
  for (uint32_t lane = 0; lane < lanes; ++lane)
    for (uint32_t row = 1; row < sizes[lane]; ++row) {
      const float estimate = scores[(lane * kRows + row) * 2 + 1];
      size_t at = estimates.size();
      estimates.push_back(estimate);
      owners.push_back(lane);
      for (; at > 0 && estimates[at - 1] < estimate; --at) {   // an earlier row first among equal ones
        estimates[at] = estimates[at - 1];
        owners[at] = owners[at - 1];
      }
      estimates[at] = estimate;
      owners[at] = lane;
    }
  std::vector<uint32_t> taken_of(lanes, 1);
  uint32_t taken = lanes;
  for (size_t i = 0; i < estimates.size() && taken < rows; ++i) {
    if (estimates[i] < floor) break;
    if (taken_of[owners[i]] == lane_cap) continue;
    ++taken_of[owners[i]];
    ++taken;
  }
  uint32_t first = 0;
  for (uint32_t lane = 0; lane < lanes; ++lane) {
    const uint32_t mine = taken_of[lane];
    uint32_t order[kRows], placed[kRows], stack[kRows], size = 0, next = 0;
    stack[size++] = 0;
    while (size) {
      const uint32_t row = stack[--size];
      placed[row] = next;
      order[next++] = row;
      for (uint32_t child = mine; child-- > row + 1;)
        if (trees[lane * kRows + child].parent == row) stack[size++] = child;
    }
    uint32_t ancestors[kRows], depths[kRows];
    for (uint32_t at = 0; at < next; ++at) {
      const uint32_t row = order[at];
      const uint32_t up = at ? placed[trees[lane * kRows + row].parent] : 0xFFFFu;
      ancestors[at] = (at ? ancestors[up] : 0u) | (1u << at);
      depths[at] = at ? depths[up] + 1 : 0;
      tokens[first + at] = tree_tokens[lane * kRows + row];
      tree[first + at] = {ancestors[at], uint16_t(up), uint16_t(depths[at])};
      sources[first + at] = row;
    }
    lane_rows[2 * lane] = first;
    lane_rows[2 * lane + 1] = next;
    first += next;
  }
  for (uint32_t row = first; row < rows; ++row) {
    tokens[row] = tree_tokens[0];
    tree[row] = {0u, 0xFFFFu, 0};
    sources[row] = 0xFFFFFFFFu;
  }
}

// The same rows in slots: lane l's from row l * lane_cap on (every lane may take its cap, so the step's rows never bind),
// the rest of its slot inert rows -- no token, on no path but their own, a child of the anchor, no source.
void orc_draft_verify_row_slots(const uint32_t *tree_tokens, const struct OrcTreeRow *trees, const float *scores, const uint32_t *sizes,
                                uint32_t lanes, uint32_t lane_cap, float floor, uint32_t *tokens, struct OrcTreeRow *tree,
                                uint32_t *lane_rows, uint32_t *sources) {
  const uint32_t rows = lanes * lane_cap;
  std::vector<uint32_t> packed_tokens(rows), packed_sources(rows), packed_lanes(2 * lanes);
  std::vector<OrcTreeRow> packed_tree(rows);
  orc_draft_verify_rows(tree_tokens, trees, scores, sizes, lanes, rows, lane_cap, floor, packed_tokens.data(), packed_tree.data(),
                        packed_lanes.data(), packed_sources.data());
  for (uint32_t lane = 0; lane < lanes; ++lane) {
    const uint32_t from = packed_lanes[2 * lane], mine = packed_lanes[2 * lane + 1], first = lane * lane_cap;
    for (uint32_t row = 0; row < lane_cap; ++row) {
      const bool own = row < mine;
      tokens[first + row] = own ? packed_tokens[from + row] : ORC_NO_TOKEN;
      tree[first + row] = own ? packed_tree[from + row] : OrcTreeRow{1u << row, uint16_t(0), uint16_t(1)};
      sources[first + row] = own ? packed_sources[from + row] : ORC_NO_TOKEN;
    }
    lane_rows[2 * lane] = first;
    lane_rows[2 * lane + 1] = mine;
  }
}

uint32_t orc_argmax(const float *logits, uint32_t vocab) {
  float best = -std::numeric_limits<float>::infinity();
  uint32_t index = ORC_NO_TOKEN;
  for (uint32_t t = 0; t < vocab; ++t) {
    if (unselectable(logits[t])) continue;
    if (logits[t] > best || (logits[t] == best && t < index)) { best = logits[t]; index = t; }
  }
  return index;
}

// sampling.metal:2044-2083
uint32_t orc_accept_tree(const struct OrcTreeRow *tree, const uint32_t *tokens, const uint32_t *selected, uint32_t rows,
                         uint32_t remaining, const uint32_t *stop_tokens, uint32_t stops, uint32_t *out_tokens,
                         uint32_t *accepted, uint32_t *retained_rows) {
  uint32_t path[32];
  path[0] = 0;
  uint32_t count = 0;
  for (uint32_t row = 0;;) {
    uint32_t next = 0;
    for (uint32_t child = row + 1; child < rows && !next; ++child)
      next = tree[child].parent == row && tokens[child] == selected[row] ? child : 0;
    if (!next) break;
    path[++count] = next;
    row = next;
  }
  uint32_t kept = std::min(count + 1, std::max(remaining, 1u));
  for (uint32_t i = 0; i < kept; ++i) {
    const uint32_t token = selected[path[i]];
    out_tokens[i] = token;
    for (uint32_t s = 0; s < stops; ++s)
      if (stop_tokens[s] != ORC_NO_TOKEN && stop_tokens[s] == token) kept = i + 1;
  }
  *accepted = std::min(count, kept);
  *retained_rows = tree[path[kept - 1]].ancestors;
  return kept;
}

uint32_t orc_distribution_end(const float *x, uint32_t V, const OrcSamplingPolicy *policy, uint32_t *key, uint32_t *last, float *mass,
                              double *closeness) {
  if (closeness) *closeness = 1.0;
  uint32_t count = 0;
  const Kept kept = distributionEnd(x, V, *policy, &count, closeness);
  *key = kept.end.key;
  *last = kept.end.last;
  *mass = kept.m.sum;
  return count;
}

uint32_t orc_rejection_row(const float *x, uint32_t V, float temperature, const float *q, uint32_t draft_token, float u_child,
                           float u_row, int *accepted_draft, double *closeness) {
  const OrcSamplingPolicy policy{temperature, 0.f, 0u, 1.f};
  return orc_rejection_row_policy(x, V, &policy, q, draft_token, u_child, u_row, accepted_draft, closeness);
}

uint32_t orc_rejection_row_policy(const float *x, uint32_t V, const OrcSamplingPolicy *policy, const float *q, uint32_t draft_token,
                                  float u_child, float u_row, int *accepted_draft, double *closeness) {
  const float inv = 1.0f / policy->temperature;
  if (closeness) *closeness = 1.0;
  const Kept mass = distributionEnd(x, V, *policy, nullptr, closeness);
  if (accepted_draft) *accepted_draft = 0;
  bool rejected = false;
  if (q && draft_token != ORC_NO_TOKEN && draft_token < V) {
    const float pc = keptWeight(x[draft_token], draft_token, mass, inv) / mass.m.sum;
    note(closeness, double(u_child) * q[draft_token], pc);
    rejected = !(u_child * q[draft_token] < pc);   // accept iff u q < p (sampling.metal:790-800)
    if (!rejected) { if (accepted_draft) *accepted_draft = 1; return draft_token; }
  }
  // ranges: 64 lanes each sum their tokens in id order, lanes added in order
  const uint32_t size = (V + kRanges - 1) / kRanges, per = (size + 63) / 64;
  std::vector<float> ranges(kRanges, 0.f), lanes(64);
  auto laneSums = [&](uint32_t range) {
    const uint32_t begin = range * size, end = std::min(V, begin + size);
    for (uint32_t l = 0; l < 64; ++l) {
      float s = 0.f;
      for (uint32_t i = 0; i < per; ++i) {
        const uint32_t t = begin + l * per + i;
        if (t < end) s += residualOf(x[t], t, rejected ? q[t] : 0.f, mass, inv, rejected);
      }
      lanes[l] = s;
    }
  };
  float total = 0.f;
  for (uint32_t j = 0; j < kRanges; ++j) {
    laneSums(j);
    float s = 0.f;
    for (int l = 0; l < 64; ++l) s += lanes[l];
    ranges[j] = s;
  }
  for (uint32_t j = 0; j < kRanges; ++j) total += ranges[j];
  if (!(total > 0.f)) return ORC_NO_TOKEN;
  const float point = u_row * total;
  uint32_t hit = kRanges, lastWeighted = 0;
  float before = 0.f, lastBefore = 0.f, cumulative = 0.f;
  for (uint32_t j = 0; j < kRanges && hit == kRanges; ++j) {
    if (ranges[j] > 0.f) { lastWeighted = j; lastBefore = cumulative; }
    if (point < cumulative + ranges[j]) { hit = j; before = cumulative; note(closeness, point, cumulative + ranges[j]); if (cumulative > 0) note(closeness, point, cumulative); }
    cumulative += ranges[j];
  }
  if (hit == kRanges) { hit = lastWeighted; before = lastBefore; }
  float target = point - before;
  laneSums(hit);
  uint32_t chunk = 64, lastChunk = 0;
  float chunkBefore = 0.f, lastChunkBefore = 0.f;
  cumulative = 0.f;
  for (uint32_t l = 0; l < 64; ++l) {
    if (lanes[l] > 0.f) { lastChunk = l; lastChunkBefore = cumulative; }
    if (chunk == 64 && target < cumulative + lanes[l]) { chunk = l; chunkBefore = cumulative; note(closeness, double(target) + before, double(cumulative) + lanes[l] + before); }
    cumulative += lanes[l];
  }
  if (chunk == 64) { chunk = lastChunk; chunkBefore = lastChunkBefore; }
  target -= chunkBefore;
  const uint32_t begin = hit * size, end = std::min(V, begin + size);
  uint32_t selected = ORC_NO_TOKEN, lastToken = ORC_NO_TOKEN;
  float walked = 0.f;
  for (uint32_t i = 0; i < per; ++i) {
    const uint32_t t = begin + chunk * per + i;
    if (t >= end) break;
    const float w = residualOf(x[t], t, rejected ? q[t] : 0.f, mass, inv, rejected);
    if (w > 0.f) lastToken = t;
    walked += w;
    if (selected == ORC_NO_TOKEN && w > 0.f && target < walked) {
      selected = t;
      note(closeness, double(target) + before + chunkBefore, double(walked) + before + chunkBefore);
      note(closeness, double(target) + before + chunkBefore, double(walked - w) + before + chunkBefore);
    }
  }
  return selected != ORC_NO_TOKEN ? selected : lastToken;
}

// sampling.metal:697-880 (vocabulary_draw with children): a verify row of a tree block tests the children its draft drew
// among the sixteen candidates ids[] (draft probabilities q[], candidate indices draws[0 .. n_draws) in the order drawn,
// one uniform a child): child c is selected iff u_c q_c < p_c; on a rejection the target's distribution becomes its
// residual max(p - q, 0) over the candidates with the mass outside them kept, renormalized, and the draft's loses the
// child, renormalized. A row that selects none draws at point = u_row (inside + outside): a candidate with residual
// weight in index order, or past them a token outside the candidates by the target's own weights in id order. Sums
// in fp32 in the orders of the kernel: ranges of (V + 255) / 256 tokens, 64 lane chunks a range, tokens of a chunk.
uint32_t orc_children_row(const float *x, uint32_t V, const OrcSamplingPolicy *policy, const uint32_t *ids, const float *q_in,
                          const uint8_t *draws, uint32_t n_draws, const float *u_children, float u_row, double *closeness) {
  constexpr uint32_t K = 16;
  const float inv = 1.0f / policy->temperature;
  if (closeness) *closeness = 1.0;
  const Kept mass = distributionEnd(x, V, *policy, nullptr, closeness);
  const uint32_t size = (V + kRanges - 1) / kRanges, per = (size + 63) / 64;
  std::vector<float> ranges(kRanges, 0.f), lanes(64);
  bool excluding = false;
  uint32_t excluded[K];
  auto weightOf = [&](uint32_t t) {
    if (excluding)
      for (uint32_t i = 0; i < K; ++i)
        if (excluded[i] == t) return 0.f;
    return keptWeight(x[t], t, mass, inv);
  };
  auto laneSums = [&](uint32_t range) {
    const uint32_t begin = range * size, end = std::min(V, begin + size);
    for (uint32_t l = 0; l < 64; ++l) {
      float s = 0.f;
      for (uint32_t i = 0; i < per; ++i) {
        const uint32_t t = begin + l * per + i;
        if (t < end) s += weightOf(t);
      }
      lanes[l] = s;
    }
  };
  for (uint32_t j = 0; j < kRanges; ++j) {
    laneSums(j);
    float s = 0.f;
    for (int l = 0; l < 64; ++l) s += lanes[l];
    ranges[j] = s;
  }
  float total = 0.f;
  for (uint32_t j = 0; j < kRanges; ++j) total += ranges[j];
  if (!(total > 0.f)) return ORC_NO_TOKEN;
  float target = u_row * total;
  if (n_draws && draws[0] != 0xFF) {
    float p[K], q[K];
    for (uint32_t i = 0; i < K; ++i) {
      const float w = ids[i] < V ? keptWeight(x[ids[i]], ids[i], mass, inv) : 0.f;
      if (ids[i] < V) ranges[ids[i] / size] = std::max(ranges[ids[i] / size] - w, 0.f);
      excluded[i] = ids[i];
      p[i] = w / total;
      q[i] = q_in[i];
    }
    float outsideWeight = 0.f;
    for (uint32_t j = 0; j < kRanges; ++j) outsideWeight += ranges[j];
    float outside = outsideWeight / total;
    for (uint32_t child = 0; child < n_draws && child < 4; ++child) {
      const uint32_t c = draws[child];
      if (c == 0xFF) break;
      note(closeness, double(u_children[child]) * q[c], p[c]);
      if (u_children[child] * q[c] < p[c]) return ids[c];
      float residual = outside;
      for (uint32_t i = 0; i < K; ++i) residual += std::max(p[i] - q[i], 0.f);
      if (!(residual > 0.f)) break;
      for (uint32_t i = 0; i < K; ++i) p[i] = std::max(p[i] - q[i], 0.f) / residual;
      outside /= residual;
      q[c] = 0.f;
      float rest = 0.f;
      for (uint32_t i = 0; i < K; ++i) rest += q[i];
      for (uint32_t i = 0; rest > 0.f && i < K; ++i) q[i] /= rest;
    }
    float inside = 0.f;
    for (uint32_t i = 0; i < K; ++i) inside += p[i];
    const float point = u_row * (inside + outside);
    float cumulative = 0.f;
    uint32_t last = K;
    for (uint32_t i = 0; i < K && !(point < cumulative); ++i)
      if (p[i] > 0.f) {
        last = i;
        note(closeness, point, cumulative + p[i]);
        if (cumulative > 0) note(closeness, point, cumulative);
        cumulative += p[i];
      }
    if (last < K && (point < cumulative || !(outside > 0.f))) return ids[last];
    excluding = true;
    target = (point - inside) / outside * outsideWeight;
  }
  // the range that holds the target; the last weighted one on a rounding shortfall
  uint32_t hit = kRanges, lastWeighted = 0;
  float before = 0.f, lastBefore = 0.f, cumulative = 0.f;
  for (uint32_t j = 0; j < kRanges && hit == kRanges; ++j) {
    if (ranges[j] > 0.f) { lastWeighted = j; lastBefore = cumulative; }
    if (ranges[j] > 0.f && target < cumulative + ranges[j]) {
      hit = j; before = cumulative;
      note(closeness, double(target), double(cumulative) + ranges[j]);
      if (cumulative > 0) note(closeness, double(target), cumulative);
    }
    cumulative += ranges[j];
  }
  if (hit == kRanges) { hit = lastWeighted; before = lastBefore; }
  float within = target - before;
  laneSums(hit);   // with the candidates left out when the draw is past them
  uint32_t chunk = 64, lastChunk = 0;
  float chunkBefore = 0.f, lastChunkBefore = 0.f;
  cumulative = 0.f;
  for (uint32_t l = 0; l < 64; ++l) {
    if (lanes[l] > 0.f) { lastChunk = l; lastChunkBefore = cumulative; }
    if (chunk == 64 && lanes[l] > 0.f && within < cumulative + lanes[l]) {
      chunk = l; chunkBefore = cumulative;
      note(closeness, double(within) + before, double(cumulative) + lanes[l] + before);
    }
    cumulative += lanes[l];
  }
  if (chunk == 64) { chunk = lastChunk; chunkBefore = lastChunkBefore; }
  within -= chunkBefore;
  const uint32_t begin = hit * size, end = std::min(V, begin + size);
  uint32_t selected = ORC_NO_TOKEN, lastToken = ORC_NO_TOKEN;
  float walked = 0.f;
  for (uint32_t i = 0; i < per; ++i) {
    const uint32_t t = begin + chunk * per + i;
    if (t >= end) break;
    const float w = weightOf(t);
    if (w > 0.f) lastToken = t;
    walked += w;
    if (selected == ORC_NO_TOKEN && w > 0.f && within < walked) {
      selected = t;
      note(closeness, double(within) + before + chunkBefore, double(walked) + before + chunkBefore);
      note(closeness, double(within) + before + chunkBefore, double(walked - w) + before + chunkBefore);
    }
  }
  return selected != ORC_NO_TOKEN ? selected : lastToken;
}

// The law of that selection when the draft draws its n_draws children from q without replacement (each next child from
// the rest of q, renormalized), in fp64 by enumerating every sequence of rejected children
// (target_sampling_metal_test.mm:2560-2600): out[t] = P(the row selects t). It equals the target's own distribution
// whatever q and the candidates are: that is what the rule is for.
void orc_children_law(const double *p_target, uint32_t V, const uint32_t *ids, const double *q_in, uint32_t n_draws, double *out) {
  constexpr uint32_t K = 16;
  struct State { double p[K], q[K], outside; };
  std::vector<bool> candidate(V, false);
  double outsideMass = 0;
  for (uint32_t i = 0; i < K; ++i) if (ids[i] < V) candidate[ids[i]] = true;
  for (uint32_t t = 0; t < V; ++t) { out[t] = 0; if (!candidate[t]) outsideMass += p_target[t]; }
  State start{};
  for (uint32_t i = 0; i < K; ++i) { start.p[i] = ids[i] < V ? p_target[ids[i]] : 0.0; start.q[i] = q_in[i]; }
  start.outside = outsideMass;
  struct Walker {
    const double *p_target; uint32_t V; const uint32_t *ids; const std::vector<bool> &candidate; double outsideMass; double *out;
    void step(const State &r, uint32_t left, double weight) {
      double draft = 0;
      for (double v : r.q) draft += v;
      if (!left || !(draft > 0)) {
        for (uint32_t i = 0; i < K; ++i) if (ids[i] < V) out[ids[i]] += weight * r.p[i];
        for (uint32_t t = 0; t < V && outsideMass > 0; ++t) if (!candidate[t]) out[t] += weight * r.outside * p_target[t] / outsideMass;
        return;
      }
      for (uint32_t i = 0; i < K; ++i) {
        if (!(r.q[i] > 0)) continue;
        const double drawn = r.q[i] / draft, accept = std::min(1.0, r.p[i] / r.q[i] * draft);   // q renormalized to its rest
        if (ids[i] < V) out[ids[i]] += weight * drawn * accept;
        if (accept < 1.0) {
          State next = r;
          double residual = next.outside;
          for (uint32_t j = 0; j < K; ++j) residual += std::max(next.p[j] - next.q[j] / draft, 0.0);
          if (!(residual > 0)) continue;
          for (uint32_t j = 0; j < K; ++j) next.p[j] = std::max(next.p[j] - next.q[j] / draft, 0.0) / residual;
          next.outside /= residual;
          next.q[i] = 0;
          step(next, left - 1, weight * drawn * (1.0 - accept));
        }
      }
    }
  } walker{p_target, V, ids, candidate, outsideMass, out};
  walker.step(start, n_draws, 1.0);
}

// P(select t) = q_t min(1, p_t / q_t) + (1 - sum_s q_s min(1, p_s / q_s)) * max(p_t - q_t, 0) / Z:
// the first term is "child t drawn and accepted", the second "child rejected, residual draws t".
void orc_rejection_law(const float *x, uint32_t V, float temperature, const float *q, double *out) {
  const OrcSamplingPolicy policy{temperature, 0.f, 0u, 1.f};
  orc_rejection_law_policy(x, V, &policy, q, out);
}

void orc_rejection_law_policy(const float *x, uint32_t V, const OrcSamplingPolicy *policy, const float *q, double *out) {
  const float temperature = policy->temperature;
  std::vector<double> p(V);
  double mx = -std::numeric_limits<double>::infinity(), total = 0;
  for (uint32_t t = 0; t < V; ++t) if (!unselectable(x[t])) mx = std::max(mx, double(x[t]));
  const Kept kept = distributionEnd(x, V, *policy, nullptr, nullptr);
  for (uint32_t t = 0; t < V; ++t) {
    const bool stays = !unselectable(x[t]) && atOrBefore(logitKey(x[t]), t, kept.end);
    p[t] = stays ? std::exp((double(x[t]) - mx) / temperature) : 0.0;
    total += p[t];
  }
  for (uint32_t t = 0; t < V; ++t) p[t] /= total;
  double acceptMass = 0, Z = 0;
  for (uint32_t t = 0; t < V; ++t) { acceptMass += std::min(double(q[t]), p[t]); Z += std::max(p[t] - double(q[t]), 0.0); }
  for (uint32_t t = 0; t < V; ++t)
    out[t] = std::min(double(q[t]), p[t]) + (Z > 0 ? (1.0 - acceptMass) * std::max(p[t] - double(q[t]), 0.0) / Z : 0.0);
}

// The sampling penalties of a lane's verify rows, in place. One logit (PenaltyReference.hpp:27-40, referencePenalty): a
// token the output holds `count` times or the prompt holds has its logit divided by the repetition penalty when
// positive and multiplied otherwise, then lowered by frequency * count + presence when count is not 0, and the result
// saturates at the largest float; NaN and -infinity stay. Which rows count which tokens (sampling.metal:1008-1050): row
// r's count is the table's (the word without its prompt bit) plus the block's rows 1.. on r's path (its ancestors mask,
// itself included) whose input token is the token; row 0's input, the anchor, is in the table already.
void orc_penalize(float *logits, uint32_t rows, uint32_t vocabulary, uint32_t stride, const uint32_t *words, const uint32_t *input_tokens,
                  const uint32_t *ancestors, float repetition, float presence, float frequency) {
  constexpr float kLargest = std::numeric_limits<float>::max();
  const float inverse = std::min(1.0f / repetition, kLargest);
  for (uint32_t r = 0; r < rows; ++r)
    for (uint32_t t = 0; t < vocabulary; ++t) {
      uint32_t count = words[t] & 0x7FFFFFFFu;
      for (uint32_t j = 1; j < rows; ++j)
        if (((ancestors[r] >> j) & 1u) && input_tokens[j] == t) ++count;
      const bool prompt = words[t] >> 31;
      float &x = logits[size_t(r) * stride + t];
      if ((!count && !prompt) || unselectable(x)) continue;
      float v = x * (x > 0.0f ? inverse : repetition);
      if (count) v -= frequency * float(count) + presence;
      x = std::clamp(v, -kLargest, kLargest);
    }
}

// The thinking cutoff of one lane over its selections, in place (sampling.metal:1993-2039, ThinkingCutoffParams in
// abi/Sampling.h:147-175): for every row, the cut is the depth of the first row of its path, from the anchor down, at
// depth cutoff_row or deeper (and, when `admits` is given, an end that waits for its mask, whose admits[] is set); a
// row `i` levels below its cut, i < count, selects end[i], unless a draft token of a path row other than the anchor at
// depth <= cut is `close` or `also_ends`, or the row's selection is no token of the vocabulary.
void orc_thinking_cutoff(uint32_t *tokens, const uint32_t *input_tokens, const struct OrcTreeRow *tree, uint32_t rows, uint32_t vocabulary,
                         uint32_t cutoff_row, const uint32_t *end, uint32_t count, uint32_t close, uint32_t also_ends,
                         const uint8_t *admits) {
  for (uint32_t r = 0; r < rows; ++r) {
    const uint32_t path = tree[r].ancestors, depth = tree[r].depth;
    uint32_t cut = 0;
    bool found = false;
    for (uint32_t j = 0; j < rows && !found; ++j) {
      if (!((path >> j) & 1u)) continue;
      if (cut >= cutoff_row && (!admits || admits[j])) found = true;
      else ++cut;
    }
    if (!found || cut > depth || depth - cut >= count) continue;
    bool ended = false;
    for (uint32_t j = 1; j < rows; ++j)
      if (((path >> j) & 1u) && tree[j].depth <= cut && (input_tokens[j] == close || input_tokens[j] == also_ends)) ended = true;
    if (!ended && tokens[r] < vocabulary) tokens[r] = end[depth - cut];
  }
}

} // extern "C"
