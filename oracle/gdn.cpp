// CPU oracle, Gated DeltaNet verify step (test infrastructure only; see oracle.h).
//
// A restatement of the reference's decode step for one lane and one layer
// (runtime/metal/kernels/decode/gdn.metal:139-526, common/gdn_primitives.h:20-99) in its order of
// operations: short convolution + SiLU, q/k RMS norms, gates, the fold of the pending (previously
// accepted) rows into the state, the block rows' outputs, the gated output norm, the step's tape.
// Sums over a head's 128 channels or a state row's 128 columns are four (resp. one) tree sums
// over 32 lanes (neighbouring pairs first), as the kernels compute them.
//
// A block that is not a chain (gdn.metal:417-478): every row's convolution taps follow its path,
// and its output comes from the committed state through its transformed query and its path's
// coefficients, S_-1 z_-1 + sum_j c_j v_j.
#include "oracle.h"
#include "common.hpp"

#include <cmath>
#include <vector>

using namespace orc;

namespace {

constexpr uint32_t kTaps = 4, kDim = 128, kRowsMax = 16;
constexpr float kEps = 1e-6f;

// a binary tree over neighbours: pairs, quads, eights, sixteens, then the two sixteens
float butterfly32(float *lane) {
  for (int step = 1; step < 32; step <<= 1)
    for (int l = 0; l < 32; l += 2 * step) lane[l] += lane[l + step];
  return lane[0];
}
// sum of 128 squares: four 32-channel groups, added in channel order
float sumSquares128(const float *v) {
  float total = 0.f;
  for (int g = 0; g < 4; ++g) {
    float lane[32];
    for (int l = 0; l < 32; ++l) lane[l] = v[32 * g + l] * v[32 * g + l];
    total += butterfly32(lane);
  }
  return total;
}
float silu(float x) { return x / (1.0f + std::exp2(-1.44269504089f * x)); }
float sigmoid(float x) { return 1.0f / (1.0f + std::exp2(-1.44269504089f * x)); }

uint32_t pathRow(uint32_t path, uint32_t depth) {
  for (uint32_t i = 0; i < depth; ++i) path &= path - 1;
  return uint32_t(__builtin_ctz(path));
}

struct Tape {
  uint16_t *inputs, *kv;
  float *decay;
  uint16_t *beta;
};
Tape tapeOf(uint8_t *base, const OrcGdnShape &s) {
  const uint32_t kvWidth = (s.key_heads + s.value_heads) * kDim;
  uint8_t *p = base;
  Tape t;
  t.inputs = reinterpret_cast<uint16_t *>(p);
  p += size_t(kRowsMax) * s.conv_dim * 2;
  t.kv = reinterpret_cast<uint16_t *>(p);
  p += size_t(kRowsMax) * kvWidth * 2;
  t.decay = reinterpret_cast<float *>(p);
  p += size_t(kRowsMax) * s.value_heads * 4;
  t.beta = reinterpret_cast<uint16_t *>(p);
  return t;
}

// The three rows of convolution inputs before a command's first row, after `consumed` rows of
// the pending path (gdn_primitives.h:20-35).
void history(const uint16_t *carried, const Tape *pending, uint32_t convDim, uint32_t consumed, uint32_t path,
             const uint16_t *rows[3]) {
  for (uint32_t r = 0; r < 3; ++r) {
    const uint32_t source = consumed + r;
    rows[r] = source < 3 ? carried + size_t(source) * convDim : pending->inputs + size_t(pathRow(path, source - 3)) * convDim;
  }
}

// delta-rule update of one state row over `count` tokens (gdn.metal:270-298); with q, also the outputs.
void foldRow(float *state /*[128]*/, uint32_t valueDim, uint32_t count, const uint16_t *keys /*[count][128]*/,
             const uint16_t *values, const float *decay, const uint16_t *beta, const uint16_t *queries, uint16_t *out /*[count][128]*/) {
  for (uint32_t t = 0; t < count; ++t) {
    const float d = decay[t], b = bf2f(beta[t]);
    float lane[32];
    for (int l = 0; l < 32; ++l) {
      float memory = 0.f;
      for (int i = 0; i < 4; ++i) {
        state[4 * l + i] *= d;
        memory += state[4 * l + i] * bf2f(keys[t * kDim + 4 * l + i]);
      }
      lane[l] = memory;
    }
    const float memory = butterfly32(lane);
    const float delta = (bf2f(values[t * kDim + valueDim]) - memory) * b;
    for (int l = 0; l < 32; ++l) {
      float result = 0.f;
      for (int i = 0; i < 4; ++i) {
        state[4 * l + i] += bf2f(keys[t * kDim + 4 * l + i]) * delta;
        if (queries) result += state[4 * l + i] * bf2f(queries[t * kDim + 4 * l + i]);
      }
      lane[l] = result;
    }
    if (queries) out[t * kDim + valueDim] = f2bf(butterfly32(lane));
  }
}

} // namespace

extern "C" {

uint64_t orc_gdn_tape_bytes(const OrcGdnShape *s) {
  const uint32_t kvWidth = (s->key_heads + s->value_heads) * kDim;
  return (uint64_t(kRowsMax) * (uint64_t(s->conv_dim) * 2 + uint64_t(kvWidth) * 2 + uint64_t(s->value_heads) * 6) + 15) / 16 * 16;
}

void orc_gdn_step(float *S, uint32_t D, const float *k, const float *v, float decay, float beta, const float *q, float *o) {
  // fp32 textbook form of one token on S [D v][D k]: S *= d; mem = S k; delta = beta (v - mem); S += delta k^T; o = S q.
  for (uint32_t r = 0; r < D; ++r) {
    double memory = 0;
    for (uint32_t c = 0; c < D; ++c) { S[r * D + c] *= decay; memory += double(S[r * D + c]) * k[c]; }
    const float delta = float((double(v[r]) - memory) * beta);
    double result = 0;
    for (uint32_t c = 0; c < D; ++c) { S[r * D + c] += k[c] * delta; result += double(S[r * D + c]) * (q ? q[c] : 0.f); }
    if (o) o[r] = float(result);
  }
}

int orc_gdn_decode(const OrcGdnShape *s, const uint16_t *packed, uint32_t rows, const uint32_t *ancestors, const uint16_t *conv_weights,
                   const float *a_scale, const uint16_t *dt_bias, const void *norm_weight, const uint16_t *conv_in, const float *state_in,
                   uint8_t *pending_tape, uint32_t pending_path, uint16_t *conv_out, float *state_out, uint8_t *step_tape,
                   uint16_t *hidden) {
  if (!rows || rows > kRowsMax || s->conv_dim != (2 * s->key_heads + s->value_heads) * kDim) return -1;
  // each row's path within the block, itself the last; without tree rows, a chain
  uint32_t paths[kRowsMax];
  bool chain = true;
  for (uint32_t t = 0; t < rows; ++t) {
    paths[t] = ancestors ? (ancestors[t] & ((1u << t) - 1u)) | (1u << t) : (2u << t) - 1u;
    chain = chain && paths[t] == (2u << t) - 1u;
  }
  const uint32_t KH = s->key_heads, VH = s->value_heads, C = s->conv_dim, P = s->packed_width, perKey = VH / KH;
  const uint32_t keyWidth = KH * kDim, kvWidth = keyWidth + VH * kDim;
  const uint32_t zOffset = C, bOffset = C + VH * kDim, aOffset = bOffset + VH;
  const uint32_t pending = uint32_t(__builtin_popcount(pending_path));
  Tape pend{}, step = tapeOf(step_tape, *s);
  if (pending) pend = tapeOf(pending_tape, *s);
  const uint16_t *hist[3];
  history(conv_in, &pend, C, pending, pending_path, hist);
  // conv carry the pending path leaves
  std::vector<uint16_t> carry(3 * size_t(C));
  for (uint32_t r = 0; r < 3; ++r) std::copy(hist[r], hist[r] + C, carry.begin() + size_t(r) * C);

  // conv + SiLU of every conv channel of every row: the taps are the last four tokens of the
  // row's path, those before the block from the history (gdn_primitives.h:37-50, gdn.metal:198-206)
  std::vector<uint16_t> conv(size_t(rows) * C);
  for (uint32_t t = 0; t < rows; ++t) {
    const uint32_t depth = uint32_t(__builtin_popcount(paths[t])) - 1;
    const uint16_t *taps[kTaps];
    for (uint32_t tap = kTaps, up = paths[t]; tap-- > 0;) {
      const uint32_t row = up ? 31u - uint32_t(__builtin_clz(up)) : 0u;
      up &= ~(1u << row);
      taps[tap] = depth + tap < 3 ? carry.data() + size_t(depth + tap) * C : packed + size_t(row) * P;
    }
    for (uint32_t c = 0; c < C; ++c) {
      float value = 0.f;
      for (uint32_t tap = 0; tap < kTaps; ++tap) value += bf2f(taps[tap][c]) * bf2f(conv_weights[size_t(c) * kTaps + tap]);
      value = bf2f(f2bf(value));
      conv[size_t(t) * C + c] = f2bf(silu(value));
    }
  }
  // per key head: normalized q and k rows; per value head: gates
  std::vector<uint16_t> queries(size_t(KH) * rows * kDim), keys(size_t(KH) * rows * kDim);
  for (uint32_t kh = 0; kh < KH; ++kh)
    for (uint32_t t = 0; t < rows; ++t) {
      float q[kDim], k[kDim];
      for (uint32_t d = 0; d < kDim; ++d) {
        q[d] = bf2f(conv[size_t(t) * C + kh * kDim + d]);
        k[d] = bf2f(conv[size_t(t) * C + keyWidth + kh * kDim + d]);
      }
      const float qs = 1.0f / std::sqrt(sumSquares128(q) / float(kDim) + kEps), ks = 1.0f / std::sqrt(sumSquares128(k) / float(kDim) + kEps);
      for (uint32_t d = 0; d < kDim; ++d) {
        queries[(size_t(kh) * rows + t) * kDim + d] = f2bf(bf2f(f2bf(q[d] * qs)) * 0.0078125f);
        keys[(size_t(kh) * rows + t) * kDim + d] = f2bf(bf2f(f2bf(k[d] * ks)) * 0.08838834765f);
      }
    }
  // tape: inputs, k, v, gates
  for (uint32_t t = 0; t < rows; ++t) {
    std::copy(packed + size_t(t) * P, packed + size_t(t) * P + C, step.inputs + size_t(t) * C);
    for (uint32_t kh = 0; kh < KH; ++kh)
      std::copy(keys.begin() + (size_t(kh) * rows + t) * kDim, keys.begin() + (size_t(kh) * rows + t + 1) * kDim,
                step.kv + size_t(t) * kvWidth + kh * kDim);
    for (uint32_t c = 0; c < VH * kDim; ++c) step.kv[size_t(t) * kvWidth + keyWidth + c] = conv[size_t(t) * C + 2 * keyWidth + c];
    for (uint32_t h = 0; h < VH; ++h) {
      const float b = bf2f(packed[size_t(t) * P + bOffset + h]);
      step.beta[t * VH + h] = f2bf(sigmoid(b));
      const float x = bf2f(f2bf(bf2f(packed[size_t(t) * P + aOffset + h]) + bf2f(dt_bias[h])));
      const float softplus = bf2f(f2bf(std::max(x, 0.0f) + std::log2(1.0f + std::exp2(-1.44269504089f * std::fabs(x))) * 0.69314718056f));
      step.decay[t * VH + h] = std::exp(a_scale[h] * softplus);
    }
  }
  std::copy(carry.begin(), carry.end(), conv_out);

  // per value head: fold the pending rows -> state_out; then the block rows for their outputs
  for (uint32_t h = 0; h < VH; ++h) {
    const uint32_t kh = h / perKey;
    uint16_t pk[kRowsMax * kDim], pv[kRowsMax * kDim], pb[kRowsMax];
    float pd[kRowsMax];
    for (uint32_t t = 0; t < pending; ++t) {
      const uint32_t row = pathRow(pending_path, t);
      std::copy(pend.kv + size_t(row) * kvWidth + kh * kDim, pend.kv + size_t(row) * kvWidth + (kh + 1) * kDim, pk + t * kDim);
      std::copy(pend.kv + size_t(row) * kvWidth + keyWidth + h * kDim, pend.kv + size_t(row) * kvWidth + keyWidth + (h + 1) * kDim, pv + t * kDim);
      pd[t] = pend.decay[row * VH + h];
      pb[t] = pend.beta[row * VH + h];
    }
    uint16_t bv[kRowsMax * kDim], bb[kRowsMax], out[kRowsMax * kDim];
    float bd[kRowsMax];
    for (uint32_t t = 0; t < rows; ++t) {
      std::copy(step.kv + size_t(t) * kvWidth + keyWidth + h * kDim, step.kv + size_t(t) * kvWidth + keyWidth + (h + 1) * kDim, bv + t * kDim);
      bd[t] = step.decay[t * VH + h];
      bb[t] = step.beta[t * VH + h];
    }
    // tree rows: the transformed query z_-1 and the path's coefficients (gdn.metal:435-478)
    float transformed[kRowsMax][kDim], coefficient[kRowsMax][kRowsMax] = {};
    if (!chain)
      for (uint32_t t = 0; t < rows; ++t) {
        float *z = transformed[t];
        for (uint32_t d = 0; d < kDim; ++d) z[d] = bf2f(queries[(size_t(kh) * rows + t) * kDim + d]);
        for (uint32_t up = paths[t]; up;) {
          const uint32_t row = 31u - uint32_t(__builtin_clz(up));
          up &= ~(1u << row);
          const uint16_t *key = keys.data() + (size_t(kh) * rows + row) * kDim;
          float lane[32];
          for (int l = 0; l < 32; ++l) {
            float product = 0.f;
            for (int i = 0; i < 4; ++i) product += bf2f(key[4 * l + i]) * z[4 * l + i];
            lane[l] = product;
          }
          const float c = bf2f(bb[row]) * butterfly32(lane), d = bd[row];
          for (uint32_t i = 0; i < kDim; ++i) z[i] = d * (z[i] - c * bf2f(key[i]));
          coefficient[t][row] = c;
        }
      }
    for (uint32_t r = 0; r < kDim; ++r) {
      float state[kDim];
      const size_t base = (size_t(h) * kDim + r) * kDim;
      std::copy(state_in + base, state_in + base + kDim, state);
      foldRow(state, r, pending, pk, pv, pd, pb, nullptr, nullptr);
      std::copy(state, state + kDim, state_out + base);
      if (chain) {
        foldRow(state, r, rows, keys.data() + size_t(kh) * rows * kDim, bv, bd, bb, queries.data() + size_t(kh) * rows * kDim, out);
        continue;
      }
      // a lane per block row carries the path's term beside its four columns' products (gdn.metal:363-377)
      for (uint32_t t = 0; t < rows; ++t) {
        float lane[32];
        for (uint32_t l = 0; l < 32; ++l) {
          float result = l < kRowsMax && ((paths[t] >> l) & 1u) ? coefficient[t][l] * bf2f(bv[l * kDim + r]) : 0.0f;
          for (int i = 0; i < 4; ++i) result += state[4 * l + i] * transformed[t][4 * l + i];
          lane[l] = result;
        }
        out[t * kDim + r] = f2bf(butterfly32(lane));
      }
    }
    // gated output norm (gdn.metal:489-526)
    const uint32_t outHead = (s->flags & 1u) ? (h % perKey) * KH + h / perKey : h;
    for (uint32_t t = 0; t < rows; ++t) {
      float value[kDim];
      for (uint32_t d = 0; d < kDim; ++d) value[d] = bf2f(out[t * kDim + d]);
      const float inverse = 1.0f / std::sqrt(sumSquares128(value) / float(kDim) + kEps);
      for (uint32_t d = 0; d < kDim; ++d) {
        const float w = (s->flags & 4u) ? static_cast<const float *>(norm_weight)[d] : bf2f(static_cast<const uint16_t *>(norm_weight)[d]);
        const float normalized = bf2f(f2bf((value[d] * inverse) * w));
        const float z = bf2f(packed[size_t(t) * P + zOffset + h * kDim + d]);
        hidden[(size_t(t) * VH + outHead) * kDim + d] = f2bf((normalized * ((s->flags & 2u) ? 1.0f : z)) / (1.0f + std::exp2(-1.44269504089f * z)));
      }
    }
  }
  return 0;
}

int orc_gdn_fold(const OrcGdnShape *s, const uint16_t *conv_in, const float *state_in, uint8_t *step_tape, uint32_t path, uint32_t rows,
                 uint16_t *conv_out, float *state_out) {
  if (uint32_t(__builtin_popcount(path)) < rows) return 1;
  const uint32_t KH = s->key_heads, VH = s->value_heads, C = s->conv_dim, perKey = VH / KH, keyWidth = KH * kDim, kvWidth = keyWidth + VH * kDim;
  Tape step = tapeOf(step_tape, *s);
  const uint16_t *hist[3];
  history(conv_in, &step, C, rows, path, hist);
  std::vector<uint16_t> carry(3 * size_t(C));
  for (uint32_t r = 0; r < 3; ++r) std::copy(hist[r], hist[r] + C, carry.begin() + size_t(r) * C);
  std::copy(carry.begin(), carry.end(), conv_out);
  for (uint32_t h = 0; h < VH; ++h) {
    const uint32_t kh = h / perKey;
    uint16_t pk[kRowsMax * kDim], pv[kRowsMax * kDim], pb[kRowsMax];
    float pd[kRowsMax];
    for (uint32_t t = 0; t < rows; ++t) {
      const uint32_t row = pathRow(path, t);
      std::copy(step.kv + size_t(row) * kvWidth + kh * kDim, step.kv + size_t(row) * kvWidth + (kh + 1) * kDim, pk + t * kDim);
      std::copy(step.kv + size_t(row) * kvWidth + keyWidth + h * kDim, step.kv + size_t(row) * kvWidth + keyWidth + (h + 1) * kDim, pv + t * kDim);
      pd[t] = step.decay[row * VH + h];
      pb[t] = step.beta[row * VH + h];
    }
    for (uint32_t r = 0; r < kDim; ++r) {
      float state[kDim];
      const size_t base = (size_t(h) * kDim + r) * kDim;
      std::copy(state_in + base, state_in + base + kDim, state);
      foldRow(state, r, rows, pk, pv, pd, pb, nullptr, nullptr);
      std::copy(state, state + kDim, state_out + base);
    }
  }
  return 0;
}

// A prompt chunk of `tokens` rows of one lane and layer (kernels/prefill/gdn.metal:196-262 the prepare pass,
// :24-160 the scan, :312-341 the gate; GDN.cpp:176-222): every row enters the state. Row t's taps are rows
// t - 3 .. t of the carried inputs followed by the chunk's own; its k, v and gates are those a decode step
// leaves on its tape for the same rows, a state row's recurrence is foldRow's, and its output reads the state
// after its own token, o_t = S_t q_t (prefill/gdn.metal:124-141). The reference's prefill sums a row's dot
// products eight lanes of sixteen columns at a time where its decode kernels sum 32 lanes of four; this
// restatement keeps the decode order for both, so that a chunk and the same rows as accepted blocks leave one
// state, and is held to the reference's fp64 bounds for the pass (gdn_metal_test.mm:283-409).
int orc_gdn_prefill(const OrcGdnShape *s, const uint16_t *packed, uint32_t tokens, const uint16_t *conv_weights, const float *a_scale,
                    const uint16_t *dt_bias, const void *norm_weight, const uint16_t *conv_in, const float *state_in, uint16_t *queries,
                    uint16_t *keys, uint16_t *values, float *decay, uint16_t *beta, uint16_t *conv_out, float *state_out,
                    uint16_t *recurrent, uint16_t *hidden) {
  if (!tokens || s->conv_dim != (2 * s->key_heads + s->value_heads) * kDim) return -1;
  const uint32_t KH = s->key_heads, VH = s->value_heads, C = s->conv_dim, P = s->packed_width, perKey = VH / KH;
  const uint32_t keyWidth = KH * kDim, valueWidth = VH * kDim, zOffset = C, bOffset = C + valueWidth, aOffset = bOffset + VH;
  auto input = [&](uint32_t position) { return position < 3 ? conv_in + size_t(position) * C : packed + size_t(position - 3) * P; };
  std::vector<uint16_t> conv(C);
  for (uint32_t t = 0; t < tokens; ++t) {
    for (uint32_t c = 0; c < C; ++c) {
      float value = 0.f;
      for (uint32_t tap = 0; tap < kTaps; ++tap) value += bf2f(input(t + tap)[c]) * bf2f(conv_weights[size_t(c) * kTaps + tap]);
      value = bf2f(f2bf(value));
      conv[c] = f2bf(silu(value));
    }
    for (uint32_t kh = 0; kh < KH; ++kh) {
      float q[kDim], k[kDim];
      for (uint32_t d = 0; d < kDim; ++d) {
        q[d] = bf2f(conv[kh * kDim + d]);
        k[d] = bf2f(conv[keyWidth + kh * kDim + d]);
      }
      const float qs = 1.0f / std::sqrt(sumSquares128(q) / float(kDim) + kEps), ks = 1.0f / std::sqrt(sumSquares128(k) / float(kDim) + kEps);
      for (uint32_t d = 0; d < kDim; ++d) {
        queries[size_t(t) * keyWidth + kh * kDim + d] = f2bf(bf2f(f2bf(q[d] * qs)) * 0.0078125f);
        keys[size_t(t) * keyWidth + kh * kDim + d] = f2bf(bf2f(f2bf(k[d] * ks)) * 0.08838834765f);
      }
    }
    for (uint32_t c = 0; c < valueWidth; ++c) values[size_t(t) * valueWidth + c] = conv[2 * keyWidth + c];
    for (uint32_t h = 0; h < VH; ++h) {
      const float b = bf2f(packed[size_t(t) * P + bOffset + h]);
      beta[size_t(t) * VH + h] = f2bf(sigmoid(b));
      const float x = bf2f(f2bf(bf2f(packed[size_t(t) * P + aOffset + h]) + bf2f(dt_bias[h])));
      const float softplus = bf2f(f2bf(std::max(x, 0.0f) + std::log2(1.0f + std::exp2(-1.44269504089f * std::fabs(x))) * 0.69314718056f));
      decay[size_t(t) * VH + h] = std::exp(a_scale[h] * softplus);
    }
  }
  for (uint32_t r = 0; r < 3; ++r) std::copy(input(tokens + r), input(tokens + r) + C, conv_out + size_t(r) * C);
  // per value head: its rows' k, q, v and gates side by side, then each state row through the chunk
  std::vector<uint16_t> hk(size_t(tokens) * kDim), hq(size_t(tokens) * kDim), hv(size_t(tokens) * kDim), hb(tokens), out(size_t(tokens) * kDim);
  std::vector<float> hd(tokens);
  for (uint32_t h = 0; h < VH; ++h) {
    const uint32_t kh = h / perKey;
    for (uint32_t t = 0; t < tokens; ++t) {
      std::copy(keys + size_t(t) * keyWidth + kh * kDim, keys + size_t(t) * keyWidth + (kh + 1) * kDim, hk.begin() + size_t(t) * kDim);
      std::copy(queries + size_t(t) * keyWidth + kh * kDim, queries + size_t(t) * keyWidth + (kh + 1) * kDim, hq.begin() + size_t(t) * kDim);
      std::copy(values + size_t(t) * valueWidth + h * kDim, values + size_t(t) * valueWidth + (h + 1) * kDim, hv.begin() + size_t(t) * kDim);
      hd[t] = decay[size_t(t) * VH + h];
      hb[t] = beta[size_t(t) * VH + h];
    }
    for (uint32_t r = 0; r < kDim; ++r) {
      float state[kDim];
      const size_t base = (size_t(h) * kDim + r) * kDim;
      std::copy(state_in + base, state_in + base + kDim, state);
      foldRow(state, r, tokens, hk.data(), hv.data(), hd.data(), hb.data(), hq.data(), out.data());
      std::copy(state, state + kDim, state_out + base);
    }
    const uint32_t outHead = (s->flags & 1u) ? (h % perKey) * KH + h / perKey : h;
    for (uint32_t t = 0; t < tokens; ++t) {
      float value[kDim];
      for (uint32_t d = 0; d < kDim; ++d) {
        recurrent[size_t(t) * valueWidth + h * kDim + d] = out[size_t(t) * kDim + d];
        value[d] = bf2f(out[size_t(t) * kDim + d]);
      }
      const float inverse = 1.0f / std::sqrt(sumSquares128(value) / float(kDim) + kEps);
      for (uint32_t d = 0; d < kDim; ++d) {
        const float w = (s->flags & 4u) ? static_cast<const float *>(norm_weight)[d] : bf2f(static_cast<const uint16_t *>(norm_weight)[d]);
        const float normalized = bf2f(f2bf((value[d] * inverse) * w));
        const float z = bf2f(packed[size_t(t) * P + zOffset + h * kDim + d]);
        hidden[(size_t(t) * VH + outHead) * kDim + d] = f2bf((normalized * ((s->flags & 2u) ? 1.0f : z)) / (1.0f + std::exp2(-1.44269504089f * z)));
      }
    }
  }
  return 0;
}

// The reference's own check of a decode step (gdn_decode_metal_test.mm:373-522): convolution + SiLU,
// normalized heads, gates and the recurrence in fp64 from the same packed rows, no intermediate
// rounding but the stored bf16 inputs. Outputs: k and v rows [rows][kv_width], beta and decay
// [rows][vh], the state after `rows` rows and the un-normed recurrent outputs [rows][vh][128].
int orc_gdn_reference(const OrcGdnShape *s, const uint16_t *packed, uint32_t rows, const uint16_t *conv_weights, const float *a_scale,
                      const uint16_t *dt_bias, const uint16_t *conv_in, const float *state_in, double *kv, double *beta, double *decay,
                      double *state_out, double *outputs) {
  const uint32_t KH = s->key_heads, VH = s->value_heads, C = s->conv_dim, P = s->packed_width, perKey = VH / KH;
  const uint32_t keyWidth = KH * kDim, kvWidth = keyWidth + VH * kDim, bOffset = C + VH * kDim, aOffset = bOffset + VH;
  std::vector<double> conv(size_t(rows) * C);
  for (uint32_t t = 0; t < rows; ++t)
    for (uint32_t c = 0; c < C; ++c) {
      double value = 0;
      for (uint32_t tap = 0; tap < kTaps; ++tap) {
        const int position = int(t) + int(tap) - 3;
        const uint16_t *row = position < 0 ? conv_in + size_t(position + 3) * C : packed + size_t(position) * P;
        value += double(bf2f(row[c])) * double(bf2f(conv_weights[size_t(c) * kTaps + tap]));
      }
      conv[size_t(t) * C + c] = value / (1.0 + std::exp(-value));
    }
  std::vector<double> q(size_t(rows) * keyWidth);
  for (uint32_t t = 0; t < rows; ++t) {
    for (uint32_t kh = 0; kh < KH; ++kh) {
      double qs = 0, ks = 0;
      for (uint32_t d = 0; d < kDim; ++d) {
        qs += conv[size_t(t) * C + kh * kDim + d] * conv[size_t(t) * C + kh * kDim + d];
        ks += conv[size_t(t) * C + keyWidth + kh * kDim + d] * conv[size_t(t) * C + keyWidth + kh * kDim + d];
      }
      qs = 1.0 / std::sqrt(qs / kDim + 1e-6);
      ks = 1.0 / std::sqrt(ks / kDim + 1e-6);
      for (uint32_t d = 0; d < kDim; ++d) {
        q[size_t(t) * keyWidth + kh * kDim + d] = conv[size_t(t) * C + kh * kDim + d] * qs / 128.0;
        kv[size_t(t) * kvWidth + kh * kDim + d] = conv[size_t(t) * C + keyWidth + kh * kDim + d] * ks / std::sqrt(128.0);
      }
    }
    for (uint32_t c = 0; c < VH * kDim; ++c) kv[size_t(t) * kvWidth + keyWidth + c] = conv[size_t(t) * C + 2 * keyWidth + c];
    for (uint32_t h = 0; h < VH; ++h) {
      beta[t * VH + h] = 1.0 / (1.0 + std::exp(-double(bf2f(packed[size_t(t) * P + bOffset + h]))));
      const double x = double(bf2f(packed[size_t(t) * P + aOffset + h])) + double(bf2f(dt_bias[h]));
      decay[t * VH + h] = std::exp(double(a_scale[h]) * (std::max(x, 0.0) + std::log1p(std::exp(-std::fabs(x)))));
    }
  }
  for (uint32_t h = 0; h < VH; ++h) {
    const uint32_t kh = h / perKey;
    for (uint32_t r = 0; r < kDim; ++r) {
      double state[kDim];
      const size_t base = (size_t(h) * kDim + r) * kDim;
      for (uint32_t c = 0; c < kDim; ++c) state[c] = state_in[base + c];
      for (uint32_t t = 0; t < rows; ++t) {
        const double d = decay[t * VH + h], b = beta[t * VH + h];
        double memory = 0;
        for (uint32_t c = 0; c < kDim; ++c) { state[c] *= d; memory += state[c] * kv[size_t(t) * kvWidth + kh * kDim + c]; }
        const double delta = (kv[size_t(t) * kvWidth + keyWidth + h * kDim + r] - memory) * b;
        double result = 0;
        for (uint32_t c = 0; c < kDim; ++c) {
          state[c] += kv[size_t(t) * kvWidth + kh * kDim + c] * delta;
          result += state[c] * q[size_t(t) * keyWidth + kh * kDim + c];
        }
        outputs[(size_t(t) * VH + h) * kDim + r] = result;
      }
      for (uint32_t c = 0; c < kDim; ++c) state_out[base + c] = state[c];
    }
  }
  return 0;
}

} // extern "C"
