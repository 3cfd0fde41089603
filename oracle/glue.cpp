// CPU oracle, glue operators of the verify step (test infrastructure only; see oracle.h).
#include "oracle.h"
#include "common.hpp"

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
