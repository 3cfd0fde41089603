// CPU oracle, acceptance of a verify block (test infrastructure only; see oracle.h).
#include "oracle.h"
#include "common.hpp"

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
float residualOf(float logit, float q, Mass m, float inv, bool rejected) {
  const float w = tokenWeight(logit, m, inv);
  return rejected ? std::max(w / m.sum - q, 0.f) : w;
}
void note(double *closeness, double value, double threshold) {
  if (!closeness) return;
  const double scale = std::max(std::fabs(value), std::fabs(threshold));
  const double distance = scale > 0 ? std::fabs(value - threshold) / scale : 1.0;
  *closeness = std::min(*closeness, distance);
}
} // namespace

extern "C" {

// sampling.metal:1896-1997: larger value, ties to the lowest id, NaN and -inf skipped.
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

uint32_t orc_rejection_row(const float *x, uint32_t V, float temperature, const float *q, uint32_t draft_token, float u_child,
                           float u_row, int *accepted_draft, double *closeness) {
  const float inv = 1.0f / temperature;
  const Mass mass = rowMass(x, V, inv);
  if (closeness) *closeness = 1.0;
  if (accepted_draft) *accepted_draft = 0;
  bool rejected = false;
  if (q && draft_token != ORC_NO_TOKEN && draft_token < V) {
    const float pc = tokenWeight(x[draft_token], mass, inv) / mass.sum;
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
        if (t < end) s += residualOf(x[t], rejected ? q[t] : 0.f, mass, inv, rejected);
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
    const float w = residualOf(x[t], rejected ? q[t] : 0.f, mass, inv, rejected);
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

// P(select t) = q_t min(1, p_t / q_t) + (1 - sum_s q_s min(1, p_s / q_s)) * max(p_t - q_t, 0) / Z:
// the first term is "child t drawn and accepted", the second "child rejected, residual draws t".
void orc_rejection_law(const float *x, uint32_t V, float temperature, const float *q, double *out) {
  std::vector<double> p(V);
  double mx = -std::numeric_limits<double>::infinity(), total = 0;
  for (uint32_t t = 0; t < V; ++t) if (!unselectable(x[t])) mx = std::max(mx, double(x[t]));
  for (uint32_t t = 0; t < V; ++t) { p[t] = unselectable(x[t]) ? 0.0 : std::exp((double(x[t]) - mx) / temperature); total += p[t]; }
  for (uint32_t t = 0; t < V; ++t) p[t] /= total;
  double acceptMass = 0, Z = 0;
  for (uint32_t t = 0; t < V; ++t) { acceptMass += std::min(double(q[t]), p[t]); Z += std::max(p[t] - double(q[t]), 0.0); }
  for (uint32_t t = 0; t < V; ++t)
    out[t] = std::min(double(q[t]), p[t]) + (Z > 0 ? (1.0 - acceptMass) * std::max(p[t] - double(q[t]), 0.0) / Z : 0.0);
}

} // extern "C"
