// CPU oracle, GGUF K-quants and the quantized projection (test infrastructure only; see oracle.h).
#include "oracle.h"
#include "common.hpp"

#include <random>

using namespace orc;

namespace {

constexpr uint32_t kQ4KBytes = 144, kQ5KBytes = 176, kQ6KBytes = 210, kQ3KBytes = 110, kQ80Bytes = 34, kQ40Bytes = 18, kQ50Bytes = 22, kIQ4XSBytes = 136, kIQ4NLBytes = 18, kBlock = 256;
// The 4-bit non-linear codebook of IQ4_NL and IQ4_XS (ggml's kvalues_iq4nl; GgufFormatReference.hpp:382-403 reads it).
constexpr int8_t kIQ4Values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
constexpr uint32_t kQ6KScales = 128 + 64, kQ6KD = kQ6KScales + 16;  // GgufFormatReference.hpp:61
constexpr uint32_t kQ3KScales = 32 + 64, kQ3KD = kQ3KScales + 12;    // GgufFormatReference.hpp:62

// Bytes and elements of a native block: the K-quants' super-block of 256, Q8_0's group of 32.
uint32_t blockBytes(uint32_t fmt) {
  return fmt == ORC_FMT_Q4K ? kQ4KBytes : fmt == ORC_FMT_Q5K ? kQ5KBytes : fmt == ORC_FMT_Q6K ? kQ6KBytes : fmt == ORC_FMT_Q80 ? kQ80Bytes
         : fmt == ORC_FMT_Q3K ? kQ3KBytes : fmt == ORC_FMT_Q40 ? kQ40Bytes : fmt == ORC_FMT_Q50 ? kQ50Bytes : fmt == ORC_FMT_IQ4XS ? kIQ4XSBytes : fmt == ORC_FMT_IQ4NL ? kIQ4NLBytes : 0;
}
uint32_t blockElements(uint32_t fmt) { return fmt == ORC_FMT_Q80 || fmt == ORC_FMT_IQ4NL || fmt == ORC_FMT_Q40 || fmt == ORC_FMT_Q50 ? 32 : kBlock; }

// GgufFormatReference.hpp:326-329
void scaleMinK4(const uint8_t *sc, int j, uint8_t &s, uint8_t &m) {
  if (j < 4) { s = sc[j] & 63; m = sc[j + 4] & 63; }
  else { s = uint8_t((sc[j + 4] & 0xF) | ((sc[j - 4] >> 6) << 4)); m = uint8_t((sc[j + 4] >> 4) | ((sc[j] >> 6) << 4)); }
}

// Codes and fp32 coefficients of one 32-group: value = s * code + m for Q4_K
// (quant_formats.h:105-137); Q6_K has a scale per 16 and code - 32 (quant_formats.h:153-168).
struct Group {
  uint8_t code[32];
  float s[2];  // Q4_K, Q5_K: s[0] = s[1] = d * sc; Q6_K, Q3_K: one per 16 elements; Q8_0, IQ4_NL: d; IQ4_XS: d * (ls - 32)
  float m;     // Q4_K, Q5_K: -dmin * mn; the others: 0
  int bias;    // Q4_K, Q5_K: 0; Q6_K: 32; Q3_K: 4; Q4_0: 8; Q5_0: 16; Q8_0, IQ4_NL, IQ4_XS: 128 (code = value or codebook value + 128)
};
void readGroup(uint32_t fmt, const uint8_t *row, uint32_t g, Group &out) {
  if (fmt == ORC_FMT_Q80) {   // GgufFormatReference.hpp:453-458: value = d * int8
    const uint8_t *blk = row + size_t(g) * kQ80Bytes;
    uint16_t d16; std::memcpy(&d16, blk, 2);
    for (int k = 0; k < 32; ++k) out.code[k] = uint8_t(int(int8_t(blk[2 + k])) + 128);
    out.s[0] = out.s[1] = h2f(d16);
    out.m = 0.f;
    out.bias = 128;
    return;
  }
  if (fmt == ORC_FMT_Q40 || fmt == ORC_FMT_Q50) {   // GgufFormatReference.hpp:529-551: value = d * (code - 8), d * (code - 16);
    const bool five = fmt == ORC_FMT_Q50;           // byte k's low nibble is input k, its high nibble input 16 + k; Q5_0's fifth
    const uint8_t *blk = row + size_t(g) * (five ? kQ50Bytes : kQ40Bytes), *qh = blk + 2, *qs = blk + (five ? 6 : 2);   // bits: bit k of qh
    uint16_t d16; std::memcpy(&d16, blk, 2);
    for (int k = 0; k < 32; ++k) {
      const int low = k < 16 ? qs[k] & 15 : qs[k - 16] >> 4;
      out.code[k] = uint8_t(five ? low | (((qh[k / 8] >> (k % 8)) & 1) << 4) : low);
    }
    out.s[0] = out.s[1] = h2f(d16);
    out.m = 0.f;
    out.bias = five ? 16 : 8;
    return;
  }
  if (fmt == ORC_FMT_IQ4NL) {   // GgufFormatReference.hpp:394-403: value = d * codebook[nibble]; byte k's low nibble is
    const uint8_t *blk = row + size_t(g) * kIQ4NLBytes;   // input k, its high nibble input 16 + k
    uint16_t d16; std::memcpy(&d16, blk, 2);
    for (int k = 0; k < 32; ++k) out.code[k] = uint8_t(kIQ4Values[k < 16 ? blk[2 + k] & 15 : blk[2 + k - 16] >> 4] + 128);
    out.s[0] = out.s[1] = h2f(d16);
    out.m = 0.f;
    out.bias = 128;
    return;
  }
  const uint8_t *blk = row + size_t(g / 8) * blockBytes(fmt);
  const uint32_t j = g % 8;
  if (fmt == ORC_FMT_IQ4XS) {   // GgufFormatReference.hpp:382-393: a 6-bit scale a group, value = d * (ls - 32) * codebook[nibble]
    uint16_t d16, high; std::memcpy(&d16, blk, 2); std::memcpy(&high, blk + 2, 2);
    const int ls = ((blk[4 + j / 2] >> (4 * (j % 2))) & 15) | (((high >> (2 * j)) & 3) << 4);
    const uint8_t *qs = blk + 8 + 16 * j;
    for (int k = 0; k < 32; ++k) out.code[k] = uint8_t(kIQ4Values[k < 16 ? qs[k] & 15 : qs[k - 16] >> 4] + 128);
    out.s[0] = out.s[1] = h2f(d16) * float(ls - 32);  // exact: 11 + 6 bits
    out.m = 0.f;
    out.bias = 128;
    return;
  }
  if (fmt == ORC_FMT_Q3K) {   // GgufFormatReference.hpp:433-451: value = d * (scale - 32) * (two bits, less 4 where the mask bit is clear)
    const uint8_t *mask = blk, *q = blk + 32 + 32 * (j / 4), *packed = blk + kQ3KScales;
    uint16_t d16; std::memcpy(&d16, blk + kQ3KD, 2);
    for (int k = 0; k < 32; ++k) out.code[k] = uint8_t(((q[k] >> (2 * (j % 4))) & 3) | (((mask[k] >> j) & 1) << 2));
    // Sixteen 6-bit scales in twelve bytes: scale i has its low four bits in the low (i < 8) or high nibble of byte
    // i % 8 and its high two bits at bit 2 (i / 4) of byte 8 + i % 4.
    for (uint32_t h = 0; h < 2; ++h) {
      const uint32_t i = 2 * j + h;
      const int low = i < 8 ? packed[i] & 15 : packed[i - 8] >> 4, high = (packed[8 + i % 4] >> (2 * (i / 4))) & 3;
      out.s[h] = h2f(d16) * float((low | (high << 4)) - 32);  // exact: 11 + 6 bits
    }
    out.m = 0.f;
    out.bias = 4;
    return;
  }
  if (fmt == ORC_FMT_Q5K) {   // GgufFormatReference.hpp:405-416: the fifth bits in qh, bit j of byte k
    uint16_t d16, m16; std::memcpy(&d16, blk, 2); std::memcpy(&m16, blk + 2, 2);
    uint8_t sc, mn; scaleMinK4(blk + 4, int(j), sc, mn);
    const uint8_t *qh = blk + 16, *q = blk + 48 + (j / 2) * 32;
    const int sh = int(j % 2) * 4;
    for (int k = 0; k < 32; ++k) out.code[k] = uint8_t(((q[k] >> sh) & 15) | (((qh[k] >> j) & 1) << 4));
    out.s[0] = out.s[1] = h2f(d16) * float(sc);  // exact: 11 + 6 bits
    out.m = -(h2f(m16) * float(mn));             // exact
    out.bias = 0;
  } else if (fmt == ORC_FMT_Q4K) {
    uint16_t d16, m16; std::memcpy(&d16, blk, 2); std::memcpy(&m16, blk + 2, 2);
    uint8_t sc, mn; scaleMinK4(blk + 4, int(j), sc, mn);
    const uint8_t *q = blk + 16 + (j / 2) * 32;
    const int sh = int(j % 2) * 4;
    for (int k = 0; k < 32; ++k) out.code[k] = (q[k] >> sh) & 15;
    out.s[0] = out.s[1] = h2f(d16) * float(sc);  // exact: 11 + 6 bits
    out.m = -(h2f(m16) * float(mn));             // exact
    out.bias = 0;
  } else {
    const uint32_t n = j / 4, r = j % 4;
    const uint8_t *ql = blk + 64 * n, *qh = blk + 128 + 32 * n;
    const int8_t *sc = reinterpret_cast<const int8_t *>(blk + kQ6KScales) + 8 * n;
    uint16_t d16; std::memcpy(&d16, blk + kQ6KD, 2);
    for (int k = 0; k < 32; ++k) {
      const uint8_t l4 = (ql[k + 32 * (r & 1)] >> (4 * (r >> 1))) & 15, h2 = (qh[k] >> (2 * r)) & 3;
      out.code[k] = uint8_t(l4 | (h2 << 4));
    }
    out.s[0] = h2f(d16) * float(sc[2 * r]);
    out.s[1] = h2f(d16) * float(sc[2 * r + 1]);
    out.m = 0.f;
    out.bias = 32;
  }
}

// llama.cpp semantics (GgufFormatReference.hpp:370-381, :405-432, :453-458): Q4_K and Q5_K d*sc*code - dmin*mn
// with one rounding (both products exact); Q6_K d*sc*(q-32), Q3_K d*(sc-32)*q (:433-451), Q8_0 d*q and the IQ4 codebook formats' s*value, exact.
void groupValues(uint32_t fmt, const uint8_t *row, uint32_t g, float *vals) {
  Group grp; readGroup(fmt, row, g, grp);
  for (int k = 0; k < 32; ++k) {
    const float s = grp.s[k / 16];
    if (fmt == ORC_FMT_Q4K || fmt == ORC_FMT_Q5K) vals[k] = s * float(grp.code[k]) + grp.m;   // s*code exact (<= 22 bits)
    else vals[k] = s * float(int(grp.code[k]) - grp.bias);
  }
}

// ---- llama.cpp-style quantizers (parity unpinned) ----
int nearestInt(float v) { return int(std::lrintf(v)); }

float makeQkx2(int n, int nmax, const float *x, const float *w, uint8_t *L, float *theMin, uint8_t *Laux, float rmin,
               float rdelta, int nstep) {
  float mn = x[0], mx = x[0], sumW = w[0], sumX = w[0] * x[0];
  for (int i = 1; i < n; ++i) { mn = std::min(mn, x[i]); mx = std::max(mx, x[i]); sumW += w[i]; sumX += w[i] * x[i]; }
  if (mn > 0) mn = 0;
  if (mx == mn) { for (int i = 0; i < n; ++i) L[i] = 0; *theMin = -mn; return 0.f; }
  float iscale = float(nmax) / (mx - mn), scale = 1 / iscale, best = 0;
  for (int i = 0; i < n; ++i) {
    const int l = std::clamp(nearestInt(iscale * (x[i] - mn)), 0, nmax);
    L[i] = uint8_t(l);
    const float diff = scale * l + mn - x[i];
    best += w[i] * diff * diff;
  }
  for (int is = 0; is <= nstep; ++is) {
    iscale = (rmin + rdelta * is + nmax) / (mx - mn);
    float sumL = 0, sumL2 = 0, sumXL = 0;
    for (int i = 0; i < n; ++i) {
      const int l = std::clamp(nearestInt(iscale * (x[i] - mn)), 0, nmax);
      Laux[i] = uint8_t(l);
      sumL += w[i] * l; sumL2 += w[i] * l * l; sumXL += w[i] * l * x[i];
    }
    const float D = sumW * sumL2 - sumL * sumL;
    if (D <= 0) continue;
    float thisScale = (sumW * sumXL - sumX * sumL) / D, thisMin = (sumL2 * sumX - sumL * sumXL) / D;
    if (thisMin > 0) { thisMin = 0; thisScale = sumXL / sumL2; }
    float mad = 0;
    for (int i = 0; i < n; ++i) { const float diff = thisScale * Laux[i] + thisMin - x[i]; mad += w[i] * diff * diff; }
    if (mad < best) { std::memcpy(L, Laux, size_t(n)); best = mad; scale = thisScale; mn = thisMin; }
  }
  *theMin = -mn;
  return scale;
}

void quantizeQ4K(const float *x, uint8_t *blk) {
  uint8_t L[256], Laux[32];
  float scales[8], mins[8], weights[32], maxScale = 0, maxMin = 0;
  for (int j = 0; j < 8; ++j) {
    float sum2 = 0;
    for (int l = 0; l < 32; ++l) sum2 += x[32 * j + l] * x[32 * j + l];
    const float av = std::sqrt(sum2 / 32);
    for (int l = 0; l < 32; ++l) weights[l] = av + std::fabs(x[32 * j + l]);
    scales[j] = makeQkx2(32, 15, x + 32 * j, weights, L + 32 * j, &mins[j], Laux, -1.f, 0.1f, 20);
    maxScale = std::max(maxScale, scales[j]);
    maxMin = std::max(maxMin, mins[j]);
  }
  const float invScale = maxScale > 0 ? 63.f / maxScale : 0.f, invMin = maxMin > 0 ? 63.f / maxMin : 0.f;
  uint8_t *sc = blk + 4;
  std::memset(sc, 0, 12);
  for (int j = 0; j < 8; ++j) {
    const uint8_t ls = uint8_t(std::min(63, nearestInt(invScale * scales[j])));
    const uint8_t lm = uint8_t(std::min(63, nearestInt(invMin * mins[j])));
    if (j < 4) { sc[j] = ls; sc[j + 4] = lm; }
    else { sc[j + 4] = uint8_t((ls & 0xF) | ((lm & 0xF) << 4)); sc[j - 4] |= uint8_t((ls >> 4) << 6); sc[j] |= uint8_t((lm >> 4) << 6); }
  }
  const uint16_t d16 = f2h(maxScale / 63.f), m16 = f2h(maxMin / 63.f);
  std::memcpy(blk, &d16, 2); std::memcpy(blk + 2, &m16, 2);
  for (int j = 0; j < 8; ++j) {
    uint8_t s, m; scaleMinK4(sc, j, s, m);
    const float d = h2f(d16) * s;
    if (!d) continue;
    const float dm = h2f(m16) * m;
    for (int i = 0; i < 32; ++i) L[32 * j + i] = uint8_t(std::clamp(nearestInt((x[32 * j + i] + dm) / d), 0, 15));
  }
  uint8_t *q = blk + 16;
  for (int j = 0; j < 256; j += 64, q += 32)
    for (int l = 0; l < 32; ++l) q[l] = uint8_t(L[j + l] | (L[j + l + 32] << 4));
}

float makeQx(int n, int nmax, const float *x, int8_t *L) {
  float mx = 0, amax = 0;
  for (int i = 0; i < n; ++i) { const float ax = std::fabs(x[i]); if (ax > amax) { amax = ax; mx = x[i]; } }
  if (amax < 1e-15f) { for (int i = 0; i < n; ++i) L[i] = 0; return 0.f; }
  float iscale = -float(nmax) / mx, sumLX = 0, sumL2 = 0;
  for (int i = 0; i < n; ++i) {
    const int l = std::clamp(nearestInt(iscale * x[i]), -nmax, nmax - 1);
    L[i] = int8_t(l + nmax);
    const float w = x[i] * x[i];
    sumLX += w * x[i] * l; sumL2 += w * l * l;
  }
  float scale = sumL2 ? sumLX / sumL2 : 0.f, best = scale * sumLX;
  for (int is = -9; is <= 9; ++is) {
    if (!is) continue;
    iscale = -(nmax + 0.1f * is) / mx;
    sumLX = sumL2 = 0;
    for (int i = 0; i < n; ++i) {
      const int l = std::clamp(nearestInt(iscale * x[i]), -nmax, nmax - 1);
      const float w = x[i] * x[i];
      sumLX += w * x[i] * l; sumL2 += w * l * l;
    }
    if (sumL2 > 0 && sumLX * sumLX > best * sumL2) {
      for (int i = 0; i < n; ++i) L[i] = int8_t(nmax + std::clamp(nearestInt(iscale * x[i]), -nmax, nmax - 1));
      scale = sumLX / sumL2; best = scale * sumLX;
    }
  }
  return scale;
}

void quantizeQ6K(const float *x, uint8_t *blk) {
  int8_t L[256];
  float scales[16], maxScale = 0, maxAbs = 0;
  for (int ib = 0; ib < 16; ++ib) {
    scales[ib] = makeQx(16, 32, x + 16 * ib, L + 16 * ib);
    if (std::fabs(scales[ib]) > maxAbs) { maxAbs = std::fabs(scales[ib]); maxScale = scales[ib]; }
  }
  std::memset(blk, 0, kQ6KBytes);
  if (maxAbs < 1e-15f) return;
  const float iscale = -128.f / maxScale;
  const uint16_t d16 = f2h(1 / iscale);
  std::memcpy(blk + kQ6KD, &d16, 2);
  int8_t *sc = reinterpret_cast<int8_t *>(blk + kQ6KScales);
  for (int ib = 0; ib < 16; ++ib) sc[ib] = int8_t(std::min(127, nearestInt(iscale * scales[ib])));
  for (int j = 0; j < 16; ++j) {
    const float d = h2f(d16) * sc[j];
    if (!d) continue;
    for (int i = 0; i < 16; ++i) L[16 * j + i] = int8_t(std::clamp(nearestInt(x[16 * j + i] / d), -32, 31) + 32);
  }
  uint8_t *ql = blk, *qh = blk + 128;
  for (int j = 0; j < 256; j += 128, ql += 64, qh += 32)
    for (int l = 0; l < 32; ++l) {
      const uint8_t q1 = L[j + l] & 0xF, q2 = L[j + l + 32] & 0xF, q3 = L[j + l + 64] & 0xF, q4 = L[j + l + 96] & 0xF;
      ql[l] = uint8_t(q1 | (q3 << 4));
      ql[l + 32] = uint8_t(q2 | (q4 << 4));
      qh[l] = uint8_t((L[j + l] >> 4) | ((L[j + l + 32] >> 4) << 2) | ((L[j + l + 64] >> 4) << 4) | ((L[j + l + 96] >> 4) << 6));
    }
}

template <class Scale>
void makeNativeWith(uint32_t fmt, uint32_t rows, uint32_t K, std::mt19937 &rng, uint8_t *native, Scale scale) {
  const size_t bytes = size_t(rows) * orc_row_bytes(fmt, K), bb = blockBytes(fmt);
  for (size_t i = 0; i < bytes; ++i) native[i] = uint8_t(rng());
  const uint32_t off = fmt == ORC_FMT_Q6K ? kQ6KD : fmt == ORC_FMT_Q3K ? kQ3KD : 0;
  for (size_t b = 0; b < bytes / bb; ++b) {
    uint8_t *blk = native + b * bb;
    const uint16_t d = scale();
    std::memcpy(blk + off, &d, 2);
    if (fmt == ORC_FMT_Q4K || fmt == ORC_FMT_Q5K) { const uint16_t m = scale(); std::memcpy(blk + off + 2, &m, 2); }
  }
}

} // namespace

extern "C" {

uint16_t orc_f2h(float f) { return f2h(f); }
float orc_h2f(uint16_t h) { return h2f(h); }
uint16_t orc_f2bf(float f) { return f2bf(f); }
float orc_bf2f(uint16_t b) { return bf2f(b); }

uint64_t orc_row_bytes(uint32_t fmt, uint32_t K) {
  const uint32_t bb = blockBytes(fmt);
  return bb && K % kBlock == 0 ? uint64_t(K / blockElements(fmt)) * bb : 0;
}

int orc_fixture(uint32_t fmt, uint32_t rows, uint32_t K, uint32_t seed, uint8_t *native) {
  if (!orc_row_bytes(fmt, K)) return -1;
  std::mt19937 rng(seed);
  makeNativeWith(fmt, rows, K, rng, native, [&] {
    uint16_t h;
    do h = uint16_t(rng()); while ((h & 0x7C00) == 0x7C00);
    return h;
  });
  return 0;
}

int orc_make_native(uint32_t fmt, uint32_t rows, uint32_t K, uint32_t seed, uint8_t *native) {
  if (!orc_row_bytes(fmt, K)) return -1;
  std::mt19937 rng(seed);
  // GgufFormatReference.hpp:295-323 scaleRange
  std::uniform_real_distribution<float> range = fmt == ORC_FMT_Q6K     ? std::uniform_real_distribution<float>(0.00002f, 0.0001f)
                                                : fmt == ORC_FMT_IQ4XS ? std::uniform_real_distribution<float>(0.00002f, 0.00015f)
                                                                       : std::uniform_real_distribution<float>(0.0005f, 0.004f);
  makeNativeWith(fmt, rows, K, rng, native, [&] { return f2h(range(rng)); });
  return 0;
}

int orc_dequant_rows(uint32_t fmt, const uint8_t *native, uint32_t rows, uint32_t K, float *out) {
  const uint64_t rb = orc_row_bytes(fmt, K);
  if (!rb) return -1;
  parallelFor(rows, 0, [&](uint32_t lo, uint32_t hi) {
    for (uint32_t r = lo; r < hi; ++r)
      for (uint32_t g = 0; g < K / 32; ++g) groupValues(fmt, native + r * rb, g, out + size_t(r) * K + 32 * g);
  });
  return 0;
}

int orc_quantize_rows(uint32_t fmt, const float *values, uint32_t rows, uint32_t K, uint8_t *native) {
  const uint64_t rb = orc_row_bytes(fmt, K);
  if (!rb || (fmt != ORC_FMT_Q4K && fmt != ORC_FMT_Q6K)) return -1;
  parallelFor(rows, 0, [&](uint32_t lo, uint32_t hi) {
    for (uint32_t r = lo; r < hi; ++r)
      for (uint32_t b = 0; b < K / kBlock; ++b) {
        const float *x = values + size_t(r) * K + size_t(b) * kBlock;
        uint8_t *blk = native + r * rb + size_t(b) * blockBytes(fmt);
        if (fmt == ORC_FMT_Q4K) quantizeQ4K(x, blk); else quantizeQ6K(x, blk);
      }
  });
  return 0;
}

int orc_gemm_staged(uint32_t fmt, const uint8_t *native, const uint16_t *x, uint32_t M, uint32_t K, uint32_t N,
                    double *exact, double *bound, float *staged, double *accumulation, int threads) {
  const uint64_t rb = orc_row_bytes(fmt, K);
  if (!rb) return -1;
  std::vector<float> xf(size_t(M) * K);
  for (size_t i = 0; i < xf.size(); ++i) xf[i] = bf2f(x[i]);
  parallelFor(N, threads, [&](uint32_t lo, uint32_t hi) {
    std::vector<float> w(K), w16(K);
    for (uint32_t n = lo; n < hi; ++n) {
      const uint8_t *row = native + n * rb;
      for (uint32_t g = 0; g < K / 32; ++g) groupValues(fmt, row, g, w.data() + 32 * g);
      for (uint32_t k = 0; k < K; ++k) w16[k] = h2f(f2h(w[k]));   // gguf_staged.h:12-19: rounded once to half
      for (uint32_t m = 0; m < M; ++m) {
        const float *xr = xf.data() + size_t(m) * K;
        // GgufFormatReference.hpp:717-742: dot and projectionBound(staged)
        double value = 0, magnitude = 0, inputs = 0, largest = 0, rounded = 0;
        for (uint32_t k = 0; k < K; ++k) {
          value += double(xr[k]) * w[k];
          magnitude += std::fabs(double(xr[k]) * w[k]);
          inputs += std::fabs(xr[k]);
          largest = std::max(largest, double(std::fabs(w[k])));
          rounded += double(xr[k]) * w16[k];
        }
        const size_t at = size_t(m) * N + n;
        const double chain = std::ldexp(inputs * largest, -16);
        if (exact) exact[at] = value;
        if (bound) bound[at] = chain + std::ldexp(magnitude, -11) + std::ldexp(inputs, -25);
        if (staged) staged[at] = float(rounded);
        if (accumulation) accumulation[at] = chain;
      }
    }
  });
  return 0;
}

// The column tile's projection (kernels/common/gguf_column_tile.h:25-68, kernels/decode/linear_gguf_column.metal:33-66):
// weights rounded once to half; per group of 32 one fp32 chain of its products in element order (each product of a
// half and a bf16 is exact in fp32, so every step rounds once), added to the sum of its part of K; part s of eight holds
// groups [s G / 8, (s + 1) G / 8); the parts are added in order. out[m][n] is that fp32 total, before any epilogue.
int orc_gemv_column(uint32_t fmt, const uint8_t *native, const uint16_t *x, uint32_t M, uint32_t K, uint32_t N, float *out,
                    int threads) {
  const uint64_t rb = orc_row_bytes(fmt, K);
  if (!rb) return -1;
  const uint32_t G = K / 32, kParts = 8;
  std::vector<float> xf(size_t(M) * K);
  for (size_t i = 0; i < xf.size(); ++i) xf[i] = bf2f(x[i]);
  parallelFor(N, threads, [&](uint32_t lo, uint32_t hi) {
    std::vector<float> w(K);
    for (uint32_t n = lo; n < hi; ++n) {
      const uint8_t *row = native + n * rb;
      for (uint32_t g = 0; g < G; ++g) groupValues(fmt, row, g, w.data() + 32 * g);
      for (uint32_t k = 0; k < K; ++k) w[k] = h2f(f2h(w[k]));
      for (uint32_t m = 0; m < M; ++m) {
        const float *xr = xf.data() + size_t(m) * K;
        float total = 0.0f;
        for (uint32_t s = 0; s < kParts; ++s) {
          float sums = 0.0f;
          for (uint32_t g = s * G / kParts; g < (s + 1) * G / kParts; ++g) {
            float sum = 0.0f;
            for (uint32_t i = 0; i < 32; ++i) {
              const float product = w[32 * g + i] * xr[32 * g + i];   // exact: 11 + 8 significant bits
              sum = sum + product;
            }
            sums += sum;
          }
          total += sums;
        }
        out[size_t(m) * N + n] = total;
      }
    }
  });
  return 0;
}

int orc_gemm(uint32_t fmt, const uint8_t *native, const uint16_t *x, uint32_t M, uint32_t K, uint32_t N,
             double *exact, double *bound, float *chain, int threads) {
  const uint64_t rb = orc_row_bytes(fmt, K);
  if (!rb) return -1;
  std::vector<float> xf(size_t(M) * K);
  for (size_t i = 0; i < xf.size(); ++i) xf[i] = bf2f(x[i]);
  // Per-row sums of 16 inputs in element order (the activation table's sums, kernels/common/gguf_sgmatrix.h).
  std::vector<float> sums16(size_t(M) * (K / 16));
  for (uint32_t m = 0; m < M; ++m)
    for (uint32_t h = 0; h < K / 16; ++h) {
      float s = 0;
      for (int k = 0; k < 16; ++k) s += xf[size_t(m) * K + 16 * h + k];
      sums16[size_t(m) * (K / 16) + h] = s;
    }
  parallelFor(N, threads, [&](uint32_t lo, uint32_t hi) {
    std::vector<float> w(K);
    Group grp;
    for (uint32_t n = lo; n < hi; ++n) {
      const uint8_t *row = native + n * rb;
      if (exact || bound)
        for (uint32_t g = 0; g < K / 32; ++g) groupValues(fmt, row, g, w.data() + 32 * g);
      for (uint32_t m = 0; m < M; ++m) {
        const float *xr = xf.data() + size_t(m) * K;
        if (exact || bound) {
          // GgufFormatReference.hpp:717-742 dot + projectionBound(register tile)
          double value = 0, inputs = 0, largest = 0;
          for (uint32_t k = 0; k < K; ++k) {
            value += double(xr[k]) * w[k];
            inputs += std::fabs(xr[k]);
            largest = std::max(largest, double(std::fabs(w[k])));
          }
          if (exact) exact[size_t(m) * N + n] = value;
          if (bound) bound[size_t(m) * N + n] = std::ldexp(inputs * largest, -16);
        }
        if (chain) {
          // linear_gguf_sgmatrix.metal:140-151, :199-288. Q4_K: one fp32 chain per 32 inputs over
          // operands 128 + code, closed by fma(dot, s, acc) and fma(sum32, m - 128 s, acc).
          // Q6_K: one chain per 16 inputs seeded with -160 * sum16 over operands 128 + code.
          float acc = 0;
          for (uint32_t g = 0; g < K / 32; ++g) {
            readGroup(fmt, row, g, grp);
            const float *s16 = sums16.data() + size_t(m) * (K / 16) + 2 * g;
            if (fmt == ORC_FMT_Q4K || fmt == ORC_FMT_Q5K) {
              float dot = 0;
              for (int k = 0; k < 32; ++k) dot = std::fma(xr[32 * g + k], float(128 + grp.code[k]), dot);
              acc = std::fma(dot, grp.s[0], acc);
              acc = std::fma(s16[0] + s16[1], grp.m - 128.f * grp.s[0], acc);
            } else if (fmt == ORC_FMT_Q80 || fmt == ORC_FMT_IQ4XS || fmt == ORC_FMT_IQ4NL) {
              // the operand is the int8 value itself (linear_gguf_sgmatrix.metal:96-98), or the codebook's
              // (:94-95), one scale a group, no min
              float dot = 0;
              for (int k = 0; k < 32; ++k) dot = std::fma(xr[32 * g + k], float(int(grp.code[k]) - 128), dot);
              acc = std::fma(dot, grp.s[0], acc);
            } else {
              for (int h = 0; h < 2; ++h) {
                float dot = -160.f * s16[h];
                for (int k = 0; k < 16; ++k) dot = std::fma(xr[32 * g + 16 * h + k], float(128 + grp.code[16 * h + k]), dot);
                acc = std::fma(dot, grp.s[h], acc);
              }
            }
          }
          chain[size_t(m) * N + n] = acc;
        }
      }
    }
  });
  return 0;
}

float orc_silu(float x) { return x / (1.f + std::exp2(-1.4426950408889634f * x)); }  // common/activation.h:8-16
uint16_t orc_epilogue_plain(float v) { return f2bf(v); }
uint16_t orc_epilogue_residual(float v, uint16_t residual) { return f2bf(v + bf2f(residual)); }
uint16_t orc_epilogue_swiglu(float gate, float up) {
  return f2bf(bf2f(f2bf(up)) * orc_silu(bf2f(f2bf(gate))));
}

} // extern "C"
