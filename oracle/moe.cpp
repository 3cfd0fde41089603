// CPU oracle, mixture-of-experts routing (test infrastructure only; see oracle.h).
#include "oracle.h"
#include "common.hpp"

#include <cmath>
#include <vector>

using namespace orc;

extern "C" {

// kernels/shared/moe.metal:23-113: rank by (score descending, expert id ascending); weight of rank r =
// exp2((s_r - s_0) log2 e) / sum over the k selected, the sum in rank order, fp32.
void orc_moe_route(const float *scores, uint32_t rows, uint32_t experts, uint32_t stride, uint32_t top_k, uint32_t *selected,
                   float *weights) {
  for (uint32_t r = 0; r < rows; ++r) {
    std::vector<float> left(scores + size_t(r) * stride, scores + size_t(r) * stride + experts);
    std::vector<float> ordered(top_k);
    for (uint32_t rank = 0; rank < top_k; ++rank) {
      uint32_t best = 0;
      for (uint32_t e = 1; e < experts; ++e)
        if (left[e] > left[best]) best = e;  // strict: the lowest id among equals
      ordered[rank] = left[best];
      selected[size_t(r) * top_k + rank] = best;
      left[best] = -INFINITY;
    }
    float denominator = 0.f;
    for (uint32_t other = 0; other < top_k; ++other) denominator += std::exp2((ordered[other] - ordered[0]) * 1.44269504089f);
    for (uint32_t rank = 0; rank < top_k; ++rank)
      weights[size_t(r) * top_k + rank] = std::exp2((ordered[rank] - ordered[0]) * 1.44269504089f) / denominator;
  }
}

void orc_moe_route_sigmoid(const float *scores, uint32_t rows, uint32_t experts, uint32_t stride, uint32_t top_k, uint32_t *selected,
                           float *weights) {
  orc_moe_route(scores, rows, experts, stride, top_k, selected, weights);   // the selection is the router's; only the weights differ
  const auto sigmoid = [](float x) { return 1.0f / (1.0f + std::exp2(-1.44269504089f * x)); };
  for (uint32_t r = 0; r < rows; ++r) {
    float denominator = 0.f;
    for (uint32_t k = 0; k < top_k; ++k) denominator += sigmoid(scores[size_t(r) * stride + selected[size_t(r) * top_k + k]]);
    for (uint32_t k = 0; k < top_k; ++k)
      weights[size_t(r) * top_k + k] = sigmoid(scores[size_t(r) * stride + selected[size_t(r) * top_k + k]]) / (denominator + 1e-20f);
  }
}

void orc_moe_shared_weights(const uint16_t *x, const float *gate, uint32_t rows, uint32_t hidden, float *weights) {
  for (uint32_t r = 0; r < rows; ++r) {
    float partial[64];
    for (uint32_t l = 0; l < 64; ++l) {
      float sum = 0.f;
      for (uint32_t d = l; d < hidden; d += 64) {
        const float product = bf2f(x[size_t(r) * hidden + d]) * gate[d];
        sum += product;
      }
      partial[l] = sum;
    }
    for (uint32_t distance = 32; distance; distance >>= 1) {
      float next[64];
      for (uint32_t l = 0; l < 64; ++l) next[l] = partial[l] + partial[l ^ distance];
      std::memcpy(partial, next, sizeof next);
    }
    weights[r] = 1.0f / (1.0f + std::exp2(-1.44269504089f * partial[0]));
  }
}

// kernels/shared/moe.metal:367-392: out = bf16(residual + sum over ranks of w y), fp32 in rank order.
// y bf16 [rows][top_k][hidden]: the expert output of each route.
void orc_moe_combine(const uint16_t *y, const float *weights, const uint16_t *residual, uint32_t rows, uint32_t top_k, uint32_t hidden,
                     uint16_t *out) {
  for (uint32_t r = 0; r < rows; ++r)
    for (uint32_t d = 0; d < hidden; ++d) {
      float value = bf2f(residual[size_t(r) * hidden + d]);
      for (uint32_t k = 0; k < top_k; ++k) value += weights[size_t(r) * top_k + k] * bf2f(y[(size_t(r) * top_k + k) * hidden + d]);
      out[size_t(r) * hidden + d] = f2bf(value);
    }
}

} // extern "C"
