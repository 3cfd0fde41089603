// CPU oracle, glue operators of the verify step (test infrastructure only; see oracle.h).
#include "oracle.h"
#include "common.hpp"

#include <cmath>
#include <vector>

using namespace orc;

extern "C" {

// kernels/shared/normalization.metal:59-99, common/rms_inverse.h:15-33: 256 threads sum the
// squares of columns tid, tid + 256, ... in column order; each 32-lane group is summed, then the
// eight group sums in order; inv = rsqrt(sum / W + 1e-6); out = bf16((x * inv) * w).
void orc_rms_norm(const uint16_t *x, const uint16_t *w, uint32_t rows, uint32_t width, uint16_t *out) {
  for (uint32_t r = 0; r < rows; ++r) {
    const uint16_t *xr = x + size_t(r) * width;
    float partial[256] = {};
    for (uint32_t c = 0; c < width; ++c) { const float v = bf2f(xr[c]); partial[c % 256] += v * v; }
    float groups[8];
    for (int g = 0; g < 8; ++g) {
      // a butterfly sum over the 32 lanes of a group
      float lane[32];
      for (int l = 0; l < 32; ++l) lane[l] = partial[32 * g + l];
      for (int step = 16; step; step >>= 1)
        for (int l = 0; l < step; ++l) lane[l] += lane[l + step];
      groups[g] = lane[0];
    }
    float sum = 0;
    for (int g = 0; g < 8; ++g) sum += groups[g];
    const float inv = 1.0f / std::sqrt(sum / float(width) + 1e-6f);
    for (uint32_t c = 0; c < width; ++c) out[size_t(r) * width + c] = f2bf((bf2f(xr[c]) * inv) * bf2f(w[c]));
  }
}

// The fp32 projection of weights kept as rows (kernels/shared/gguf_float.metal:1-8; addGgufFloat, LinearGguf.cpp:545-612):
// out[r][n] = sum_k x[r][k] W[n][k] with every operand exact in fp32 (bf16 rows widened, F32 weights as stored, BF16
// ones widened) and fp32 accumulation. The reference accumulates in the order of its 8x8 matrix fragments; this
// restatement fixes the order the gfx950 kernel runs: four chains of fused multiply-adds, chain j over k = j mod 4
// ascending, added as (c0 + c1) + (c2 + c3). What the reference promises of the result holds for it and is what pins
// it: it differs from the fp64 product only by fp32 accumulation, and BF16 weights give the bits of their F32 values.
void orc_float_projection(const uint16_t *x, const void *w, uint32_t bf16_weights, uint32_t rows, uint32_t n, uint32_t k, float *out) {
  for (uint32_t r = 0; r < rows; ++r)
    for (uint32_t c = 0; c < n; ++c) {
      float chain[4] = {0.f, 0.f, 0.f, 0.f};
      for (uint32_t i = 0; i < k; ++i) {
        const float weight = bf16_weights ? bf2f(static_cast<const uint16_t *>(w)[size_t(c) * k + i]) : static_cast<const float *>(w)[size_t(c) * k + i];
        chain[i % 4] = std::fma(bf2f(x[size_t(r) * k + i]), weight, chain[i % 4]);
      }
      out[size_t(r) * n + c] = (chain[0] + chain[1]) + (chain[2] + chain[3]);
    }
}

int orc_embed(uint32_t fmt, const uint8_t *table, uint32_t vocab, uint32_t hidden, const uint32_t *tokens,
              uint32_t rows, uint16_t *out) {
  const uint64_t rb = orc_row_bytes(fmt, hidden);
  if (!rb) return -1;
  std::vector<float> row(hidden);
  for (uint32_t r = 0; r < rows; ++r) {
    if (tokens[r] >= vocab) { for (uint32_t c = 0; c < hidden; ++c) out[size_t(r) * hidden + c] = 0; continue; }
    orc_dequant_rows(fmt, table + tokens[r] * rb, 1, hidden, row.data());
    for (uint32_t c = 0; c < hidden; ++c) out[size_t(r) * hidden + c] = f2bf(row[c]);
  }
  return 0;
}

void orc_rope_tables(uint32_t anchor, const uint32_t *depth, uint32_t rows, const float *invfreq, uint32_t pairs,
                     float *cosv, float *sinv) {
  for (uint32_t r = 0; r < rows; ++r)
    for (uint32_t p = 0; p < pairs; ++p) {
      const float angle = float(anchor + depth[r]) * invfreq[p];
      cosv[size_t(r) * pairs + p] = std::cos(angle);
      sinv[size_t(r) * pairs + p] = std::sin(angle);
    }
}

} // extern "C"
