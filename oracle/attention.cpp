// CPU oracle, INT8 KV store and block-causal paged attention (test infrastructure only; see oracle.h).
#include "oracle.h"
#include "common.hpp"

#include <limits>
#include <vector>

using namespace orc;

extern "C" {

// Q8PageFormatReference.hpp:107-122 (storedScale, quantize); attention_store.h:52-85.
void orc_kv_quantize(const float *v, uint32_t D, int half_scale, int8_t *codes, float *scale_out) {
  float maximum = 0.f;
  for (uint32_t d = 0; d < D; ++d) maximum = std::max(maximum, std::fabs(v[d]));
  for (uint32_t d = 0; d < D; ++d) {
    if (maximum == 0.f) { codes[d] = 0; continue; }
    long q = long(std::nearbyint(v[d] * 127.0f / maximum));
    codes[d] = int8_t(std::clamp<long>(q, -127, 127));
  }
  float scale = maximum == 0.f ? 0.f : maximum / 127.0f;
  if (half_scale) scale = h2f(f2h(scale));  // the stored fp16 value dequantizes on both sides
  *scale_out = scale;
}

// attention_qkv_prepare.h:28-91: per head inv = rsqrt(sum x^2 / D + 1e-6); n = bf16(x inv w);
// pairs (i, i + P): bf16(a cos - b sin), bf16(b cos + a sin); V passes through unchanged.
void orc_attention_prepare(const struct OrcAttention *a, const uint16_t *qkv, const uint16_t *qw, const uint16_t *kw,
                           const float *cosv, const float *sinv, uint32_t pairs, uint16_t *q_out, float *k_out,
                           float *v_out) {
  const uint32_t D = a->head_dim, QW = a->q_heads * D, KW = a->kv_heads * D, stride = QW + 2 * KW;
  std::vector<uint16_t> n(D);
  for (uint32_t r = 0; r < a->rows; ++r) {
    const uint16_t *row = qkv + size_t(r) * stride;
    for (uint32_t head = 0; head < a->q_heads + a->kv_heads; ++head) {
      const bool query = head < a->q_heads;
      const uint16_t *src = query ? row + head * D : row + QW + (head - a->q_heads) * D;
      const uint16_t *w = query ? qw : kw;
      if (w) {
        // the head's D threads square their element; each 64-lane wavefront sums its lanes by a
        // butterfly (pairs 32 apart, then 16, ... 1), then the wavefronts are summed in order. The
        // order inside the reference's simd_sum is the hardware's, so any fixed tree restates it.
        float groups[4] = {};
        const uint32_t waves = (D + 63) / 64;
        for (uint32_t g = 0; g < waves; ++g) {
          float lane[64] = {};
          for (uint32_t l = 0; l < 64 && 64 * g + l < D; ++l) { const float x = bf2f(src[64 * g + l]); lane[l] = x * x; }
          for (int step = 32; step; step >>= 1)
            for (int l = 0; l < step; ++l) lane[l] += lane[l + step];
          groups[g] = lane[0];
        }
        float total = 0;
        for (uint32_t g = 0; g < waves; ++g) total += groups[g];
        const float inv = 1.0f / std::sqrt(total / float(D) + 1e-6f);
        for (uint32_t d = 0; d < D; ++d) n[d] = f2bf(bf2f(src[d]) * inv * bf2f(w[d]));
      } else {
        for (uint32_t d = 0; d < D; ++d) n[d] = src[d];
      }
      std::vector<uint16_t> out(n);
      for (uint32_t p = 0; p < pairs; ++p) {
        const float first = bf2f(n[p]), second = bf2f(n[p + pairs]);
        const float c = cosv[size_t(r) * pairs + p], s = sinv[size_t(r) * pairs + p];
        out[p] = f2bf(first * c - second * s);
        out[p + pairs] = f2bf(second * c + first * s);
      }
      if (query) {
        for (uint32_t d = 0; d < D; ++d) q_out[(size_t(r) * a->q_heads + head) * D + d] = out[d];
      } else {
        const uint32_t kh = head - a->q_heads;
        for (uint32_t d = 0; d < D; ++d) {
          k_out[(size_t(r) * a->kv_heads + kh) * D + d] = bf2f(out[d]);
          v_out[(size_t(r) * a->kv_heads + kh) * D + d] = bf2f(row[QW + KW + kh * D + d]);
        }
      }
    }
  }
}

// common/int8_activations.h:22-28 (int8_activation_block, int8_activation_code).
void orc_int8_activation_block(const float *x, uint32_t n, int8_t *codes, float *scale) {
  float largest = 0.f;
  bool finite = true;
  for (uint32_t i = 0; i < n; ++i) {
    finite = finite && std::isfinite(x[i]);
    largest = std::max(largest, std::fabs(x[i]));
  }
  const bool coded = largest > 0x1p-100f;
  const float inverse = coded ? 127.0f / largest : 0.0f;
  for (uint32_t i = 0; i < n; ++i)
    codes[i] = finite ? int8_t(std::clamp(std::nearbyint(x[i] * inverse), -127.0f, 127.0f)) : int8_t(0);
  *scale = !finite ? std::numeric_limits<float>::quiet_NaN() : coded ? largest / 127.0f : 0.0f;
}

// paged_attention_tile.h:179-285 (page softmax), :427-463 (page loop), :499-535 (split merge).
void orc_attention(const struct OrcAttention *a, const uint16_t *q, const int8_t *kcodes, const float *kscales,
                   const int8_t *vcodes, const float *vscales, const uint32_t *page_table,
                   const uint32_t *ancestors, uint16_t *out, double *out64, int threads) {
  const uint32_t D = a->head_dim, PT = a->page_tokens, group = a->q_heads / a->kv_heads;
  const uint32_t total = a->committed + a->rows, pages = (total + PT - 1) / PT;
  const uint32_t splits = std::max(1u, a->splits), pps = std::max(1u, a->pages_per_split);
  const float inv_sqrt = 1.0f / std::sqrt(float(D));
  const size_t pageElems = size_t(a->kv_heads) * PT * D, pageScales = size_t(a->kv_heads) * PT;
  auto visible = [&](uint32_t r, uint32_t t) {
    if (t >= total) return false;
    if (t < a->committed) return true;
    const uint32_t j = t - a->committed;
    return j < 32 && ((ancestors[r] >> j) & 1u) != 0;
  };
  parallelFor(a->rows * a->q_heads, threads, [&](uint32_t lo, uint32_t hi) {
    std::vector<float> o(D), oSum(D), score(PT);
    for (uint32_t item = lo; item < hi; ++item) {
      const uint32_t r = item / a->q_heads, qh = item % a->q_heads, kh = qh / group;
      const uint16_t *qr = q + (size_t(r) * a->q_heads + qh) * D;
      // INT8 queries: the row's codes and scale; the score product is then exact in int32
      std::vector<int8_t> qcodes(D);
      float qscale = 1.f;
      if (a->int8_queries) {
        std::vector<float> values(D);
        for (uint32_t d = 0; d < D; ++d) values[d] = bf2f(qr[d]);
        orc_int8_activation_block(values.data(), D, qcodes.data(), &qscale);
      }
      // ---- fp32 page loop with ordered split merge ----
      std::vector<float> sm(splits, -std::numeric_limits<float>::infinity()), sl(splits, 0.f);
      std::vector<std::vector<float>> so(splits, std::vector<float>(D, 0.f));
      for (uint32_t s = 0; s < splits; ++s) {
        float m = -std::numeric_limits<float>::infinity(), l = 0.f;
        std::fill(o.begin(), o.end(), 0.f);
        const uint32_t first = s * pps, last = s + 1 == splits ? pages : std::min(pages, (s + 1) * pps);
        for (uint32_t p = first; p < last; ++p) {
          const size_t phys = page_table[p];
          const int8_t *kp = kcodes + phys * pageElems + size_t(kh) * PT * D;
          const int8_t *vp = vcodes + phys * pageElems + size_t(kh) * PT * D;
          const float *ks = kscales + phys * pageScales + size_t(kh) * PT, *vs = vscales + phys * pageScales + size_t(kh) * PT;
          float pageMax = -std::numeric_limits<float>::infinity();
          for (uint32_t t = 0; t < PT; ++t) {
            if (!visible(r, p * PT + t)) { score[t] = -std::numeric_limits<float>::infinity(); continue; }
            float dot = 0.f;
            if (a->int8_queries) {
              int32_t exact = 0;
              for (uint32_t d = 0; d < D; ++d) exact += int32_t(qcodes[d]) * int32_t(kp[size_t(t) * D + d]);
              dot = float(exact) * qscale;
            } else {
              for (uint32_t d = 0; d < D; ++d) dot += bf2f(qr[d]) * float(kp[size_t(t) * D + d]);
            }
            score[t] = dot * ks[t] * inv_sqrt;
            pageMax = std::max(pageMax, score[t]);
          }
          if (pageMax == -std::numeric_limits<float>::infinity()) continue;
          const float mNew = std::max(m, pageMax), alpha = std::exp(m - mNew);
          l *= alpha;
          for (uint32_t d = 0; d < D; ++d) o[d] *= alpha;
          for (uint32_t t = 0; t < PT; ++t) {
            if (score[t] == -std::numeric_limits<float>::infinity()) continue;
            const float pr = std::exp(score[t] - mNew);
            l += pr;
            const float weight = bf2f(f2bf(pr * vs[t]));  // P is stored as bf16(p * value_scale)
            for (uint32_t d = 0; d < D; ++d) o[d] += weight * float(vp[size_t(t) * D + d]);
          }
          m = mNew;
        }
        sm[s] = m; sl[s] = l; so[s] = o;
      }
      float M = -std::numeric_limits<float>::infinity();
      for (uint32_t s = 0; s < splits; ++s) M = std::max(M, sm[s]);
      float den = 0.f;
      std::fill(oSum.begin(), oSum.end(), 0.f);
      for (uint32_t s = 0; s < splits; ++s) {
        if (sm[s] == -std::numeric_limits<float>::infinity()) continue;
        const float w = std::exp(sm[s] - M);
        den += w * sl[s];
        for (uint32_t d = 0; d < D; ++d) oSum[d] += w * so[s][d];
      }
      for (uint32_t d = 0; d < D; ++d)
        out[(size_t(r) * a->q_heads + qh) * D + d] = f2bf(den > 0.f ? oSum[d] / den : 0.f);
      // ---- fp64 dense softmax over the stored pages (q8_flash_attention_metal_test.mm:485-536) ----
      if (out64) {
        std::vector<double> sc(total, 0.0);
        double mx = -std::numeric_limits<double>::infinity();
        for (uint32_t t = 0; t < total; ++t) {
          if (!visible(r, t)) { sc[t] = -std::numeric_limits<double>::infinity(); continue; }
          const size_t phys = page_table[t / PT];
          const int8_t *kp = kcodes + phys * pageElems + (size_t(kh) * PT + t % PT) * D;
          double dot = 0;
          for (uint32_t d = 0; d < D; ++d) dot += double(bf2f(qr[d])) * double(kp[d]);
          sc[t] = dot * double(kscales[phys * pageScales + size_t(kh) * PT + t % PT]) / std::sqrt(double(D));
          mx = std::max(mx, sc[t]);
        }
        std::vector<double> acc(D, 0.0);
        double sum = 0;
        for (uint32_t t = 0; t < total; ++t) {
          if (sc[t] == -std::numeric_limits<double>::infinity()) continue;
          const double pr = std::exp(sc[t] - mx);
          sum += pr;
          const size_t phys = page_table[t / PT];
          const int8_t *vp = vcodes + phys * pageElems + (size_t(kh) * PT + t % PT) * D;
          const double vsc = vscales[phys * pageScales + size_t(kh) * PT + t % PT];
          for (uint32_t d = 0; d < D; ++d) acc[d] += pr * vsc * double(vp[d]);
        }
        for (uint32_t d = 0; d < D; ++d) out64[(size_t(r) * a->q_heads + qh) * D + d] = sum > 0 ? acc[d] / sum : 0.0;
      }
    }
  });
}

} // extern "C"
