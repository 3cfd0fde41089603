// CPU oracle of the draft model's attention block (test infrastructure only; see oracle.h): the dynamic convolutions,
// the q/k/v preparation, the attention of a lane's eight query rows over its rings and themselves, the ring writers and
// the 4-bit context window. Restates the reference's kernels/decode/draft.metal:7-105 (convolution, preparation),
// common/draft_context_kv.h:10-45 (a context row's head into its slot), common/draft_context_window.h:37-64 and
// prefill/draft_context.metal:50-72 (the window's codes), and, for the attention, the fp64 reference of the reference's
// own test (dev/tests/engine/draft_attention_metal_test.mm:95-158) under the mask of draft.metal:186-205, :263-279.
#include "common.hpp"
#include "oracle.h"

using namespace orc;

namespace {
constexpr uint32_t kRows = 8, kQueryHeads = 32, kKvHeads = 8, kD = 128, kWindow = 2048, kPairs = 64;
constexpr uint32_t kAttention = kQueryHeads * kD, kKv = kKvHeads * kD, kPacked = kAttention + 2 * kKv;

// One head of 128 values: RMS-normalized, weighed, rounded to bf16, turned by a RoPE row. The squares are added as one
// 64-lane wavefront adds them: lane l its dimensions l and l + 64, then a butterfly 32, 16, ... 1 apart (the order
// inside the reference's simd_sum is its hardware's, so any fixed tree restates it).
void headNormRope(const uint16_t *source, const uint16_t *weight, const float *cosines, const float *sines, uint16_t *destination) {
  float lane[64];
  for (uint32_t l = 0; l < 64; ++l) {
    const float x0 = bf2f(source[l]), x1 = bf2f(source[l + 64]);
    lane[l] = x0 * x0 + x1 * x1;
  }
  for (int step = 32; step; step >>= 1)
    for (int l = 0; l < step; ++l) lane[l] += lane[l + step];
  const float inverse = 1.0f / std::sqrt(lane[0] / float(kD) + 1e-6f);
  uint16_t normalized[kD];
  for (uint32_t d = 0; d < kD; ++d) normalized[d] = f2bf(bf2f(source[d]) * inverse * bf2f(weight[d]));
  for (uint32_t i = 0; i < kPairs; ++i) {
    const float first = bf2f(normalized[i]), second = bf2f(normalized[i + kPairs]);
    destination[i] = f2bf(first * cosines[i] - second * sines[i]);
    destination[i + kPairs] = f2bf(second * cosines[i] + first * sines[i]);
  }
}
} // namespace

extern "C" {

void orc_draft_conv(const uint16_t *input, const uint16_t *dynamic, const uint16_t *base, const uint16_t *residual, uint16_t *output,
                    uint32_t hidden, uint32_t lanes, int finish) {
  const uint32_t groups = hidden / 16, dynamicWidth = 4 * groups, tap = finish ? 2 : 0;
  for (uint32_t lane = 0; lane < lanes; ++lane)
    for (uint32_t row = 0; row < kRows; ++row)
      for (uint32_t channel = 0; channel < hidden; ++channel) {
        const size_t at = (size_t(lane) * kRows + row) * hidden + channel;
        const uint16_t *dyn = dynamic + (size_t(lane) * kRows + row) * dynamicWidth;
        float value = bf2f(input[at]) * (bf2f(base[tap * hidden + channel]) + bf2f(dyn[tap * groups + channel / 16]));
        if (row > 0) value += bf2f(input[at - hidden]) * (bf2f(base[(tap + 1) * hidden + channel]) + bf2f(dyn[(tap + 1) * groups + channel / 16]));
        if (finish) value += bf2f(residual[at]);
        output[at] = f2bf(value);
      }
}

// qkv bf16 [lanes * 8][6144]; cosines / sines fp32 [lane][16][64]; queries [lane][query head][8][128];
// keys [lane][KV head][8][128]; values [lane][KV head][128][8].
void orc_draft_prepare(const uint16_t *qkv, const uint16_t *query_norm, const uint16_t *key_norm, const float *cosines, const float *sines,
                       uint32_t lanes, uint16_t *queries, uint16_t *keys, uint16_t *values) {
  for (uint32_t lane = 0; lane < lanes; ++lane)
    for (uint32_t row = 0; row < kRows; ++row) {
      const uint16_t *packed = qkv + (size_t(lane) * kRows + row) * kPacked;
      const float *c = cosines + (size_t(lane) * 16 + row) * kPairs, *s = sines + (size_t(lane) * 16 + row) * kPairs;
      for (uint32_t head = 0; head < kQueryHeads; ++head)
        headNormRope(packed + head * kD, query_norm, c, s, queries + ((size_t(lane) * kQueryHeads + head) * kRows + row) * kD);
      for (uint32_t head = 0; head < kKvHeads; ++head) {
        headNormRope(packed + kAttention + head * kD, key_norm, c, s, keys + ((size_t(lane) * kKvHeads + head) * kRows + row) * kD);
        for (uint32_t d = 0; d < kD; ++d)
          values[((size_t(lane) * kKvHeads + head) * kD + d) * kRows + row] = packed[kAttention + kKv + head * kD + d];
      }
    }
}

// `count` context rows (bf16 [.][1024 keys | 1024 values]) into one lane's rings: row source_rows[i] at position
// positions[i], turned by RoPE row rope_rows[i] of cosines / sines (fp32 [.][64]).
void orc_draft_context_write(const uint16_t *context_kv, const uint16_t *key_norm, const float *cosines, const float *sines,
                             const uint32_t *source_rows, const uint32_t *positions, const uint32_t *rope_rows, uint32_t count,
                             uint16_t *ring_keys, uint16_t *ring_values) {
  for (uint32_t i = 0; i < count; ++i) {
    const uint32_t slot = positions[i] % kWindow;
    const uint16_t *row = context_kv + size_t(source_rows[i]) * 2 * kKv;
    for (uint32_t head = 0; head < kKvHeads; ++head) {
      headNormRope(row + head * kD, key_norm, cosines + size_t(rope_rows[i]) * kPairs, sines + size_t(rope_rows[i]) * kPairs,
                   ring_keys + (size_t(head) * kWindow + slot) * kD);
      for (uint32_t d = 0; d < kD; ++d) ring_values[(size_t(head) * kD + d) * kWindow + slot] = row[kKv + head * kD + d];
    }
  }
}

// One lane and KV head in fp64: queries [32][128] (row 8 j + r: query head j's row r), the head's rings (keys
// [2048][128], values [128][2048]), the current rows' keys [8][128] and values [128][8]. Row r sits at position
// cache_length + r and sees the ring's positions of its window of 2048 (itself included, so the 2047 - ... before it)
// and all eight current rows.
void orc_draft_attention(const uint16_t *queries, const uint16_t *ring_keys, const uint16_t *ring_values, const uint16_t *query_keys,
                         const uint16_t *query_values, uint32_t cache_length, double *output) {
  const uint32_t commonStart = cache_length >= kWindow - 1 ? cache_length - (kWindow - 1) : 0, oldCount = cache_length - commonStart;
  const double scale = 0.08838834765;
  std::vector<double> scores(oldCount + kRows);
  for (uint32_t row = 0; row < 4 * kRows; ++row) {
    const uint32_t position = cache_length + row % kRows;
    const uint32_t rowStart = position >= kWindow - 1 ? position - (kWindow - 1) : 0, hiddenPrefix = rowStart - commonStart;
    const uint16_t *query = queries + size_t(row) * kD;
    double best = -INFINITY;
    for (uint32_t key = 0; key < oldCount + kRows; ++key) {
      const uint16_t *k = key >= oldCount ? query_keys + size_t(key - oldCount) * kD : ring_keys + size_t((commonStart + key) % kWindow) * kD;
      double score = -INFINITY;
      if (key >= oldCount || key >= hiddenPrefix) {
        double dot = 0;
        for (uint32_t d = 0; d < kD; ++d) dot += double(bf2f(query[d])) * double(bf2f(k[d]));
        score = dot * scale;
      }
      scores[key] = score;
      best = std::max(best, score);
    }
    double sum = 0, acc[kD] = {};
    for (uint32_t key = 0; key < oldCount + kRows; ++key) {
      if (scores[key] == -INFINITY) continue;
      const double weight = std::exp(scores[key] - best);
      sum += weight;
      for (uint32_t d = 0; d < kD; ++d)
        acc[d] += weight * double(key >= oldCount ? bf2f(query_values[size_t(d) * kRows + key - oldCount])
                                                  : bf2f(ring_values[size_t(d) * kWindow + (commonStart + key) % kWindow]));
    }
    for (uint32_t d = 0; d < kD; ++d) output[size_t(row) * kD + d] = acc[d] / sum;
  }
}

uint64_t orc_draft_window_bytes(uint32_t width) { return uint64_t(kWindow) * (width / 2) + uint64_t(kWindow) * (width / 64) * 4; }

// `rows` context rows (row source_rows[i] of `context`, bf16 [.][width]) into the slots of positions start + i.
void orc_draft_window_store(const uint16_t *context, const uint32_t *source_rows, uint32_t rows, uint32_t start, uint32_t width, uint8_t *window) {
  const uint32_t groups = width / 64;
  uint8_t *pairs = window + uint64_t(kWindow) * (width / 2);
  for (uint32_t i = 0; i < rows; ++i) {
    const uint32_t slot = (start + i) % kWindow;
    for (uint32_t group = 0; group < groups; ++group) {
      const uint16_t *values = context + size_t(source_rows[i]) * width + group * 64;
      float low = bf2f(values[0]), high = low;
      for (uint32_t l = 1; l < 64; ++l) { low = std::min(low, bf2f(values[l])); high = std::max(high, bf2f(values[l])); }
      const uint16_t scaleBits = f2h((high - low) / 15.0f), minimumBits = f2h(low);
      const float scale = h2f(scaleBits), minimum = h2f(minimumBits);
      for (uint32_t l = 0; l < 64; l += 2) {
        uint32_t code[2] = {0, 0};
        if (scale > 0)
          for (int e = 0; e < 2; ++e) code[e] = uint32_t(std::min(std::max(std::nearbyint((bf2f(values[l + e]) - minimum) / scale), 0.0f), 15.0f));
        window[size_t(slot) * (width / 2) + group * 32 + l / 2] = uint8_t(code[0] | code[1] << 4);
      }
      const uint32_t pair = uint32_t(scaleBits) | uint32_t(minimumBits) << 16;
      std::memcpy(pairs + (size_t(slot) * groups + group) * 4, &pair, 4);
    }
  }
}

void orc_draft_window_load(const uint8_t *window, uint32_t rows, uint32_t start, uint32_t width, uint16_t *context) {
  const uint32_t groups = width / 64;
  const uint8_t *pairs = window + uint64_t(kWindow) * (width / 2);
  for (uint32_t i = 0; i < rows; ++i) {
    const uint32_t slot = (start + i) % kWindow;
    for (uint32_t group = 0; group < groups; ++group) {
      uint32_t pair;
      std::memcpy(&pair, pairs + (size_t(slot) * groups + group) * 4, 4);
      const float scale = h2f(uint16_t(pair)), minimum = h2f(uint16_t(pair >> 16));
      for (uint32_t l = 0; l < 64; ++l) {
        const uint8_t byte = window[size_t(slot) * (width / 2) + group * 32 + l / 2];
        context[size_t(i) * width + group * 64 + l] = f2bf(std::fmaf(float(l & 1 ? byte >> 4 : byte & 15), scale, minimum));
      }
    }
  }
}

} // extern "C"
