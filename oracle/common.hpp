// Shared helpers of the CPU oracle (test infrastructure only; see oracle.h).
#pragma once
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <functional>
#include <thread>
#include <vector>

namespace orc {

inline float bitsToFloat(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }
inline uint32_t floatBits(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }

// IEEE binary16 <-> binary32, round to nearest even, without compiler half types
// (the reference's f2h/h2f use __fp16: dev/tests/engine/GgufFormatReference.hpp:43-44).
inline float h2f(uint16_t h) {
  const uint32_t sign = uint32_t(h & 0x8000) << 16;
  uint32_t exp = (h >> 10) & 0x1F, man = h & 0x3FF;
  if (exp == 0) {
    if (!man) return bitsToFloat(sign);
    int e = -1;
    do { man <<= 1; ++e; } while (!(man & 0x400));
    return bitsToFloat(sign | uint32_t(127 - 15 - e) << 23 | (man & 0x3FF) << 13);
  }
  if (exp == 31) return bitsToFloat(sign | 0x7F800000u | man << 13);
  return bitsToFloat(sign | (exp + 112) << 23 | man << 13);
}
inline uint16_t f2h(float f) {
  const uint32_t u = floatBits(f);
  const uint16_t sign = uint16_t((u >> 16) & 0x8000);
  const uint32_t a = u & 0x7FFFFFFF;
  if (a >= 0x7F800000u) return uint16_t(sign | 0x7C00 | (a > 0x7F800000u ? 0x200 | ((a >> 13) & 0x3FF) : 0));
  if (a >= 0x477FF000u) return uint16_t(sign | 0x7C00);  // rounds to infinity
  if (a < 0x33000001u) return sign;                      // below half of the least subnormal
  int32_t exp = int32_t(a >> 23) - 127;
  uint32_t man = (a & 0x7FFFFF) | 0x800000;
  int shift = exp < -14 ? 13 + (-14 - exp) : 13;
  uint32_t halfMan = man >> shift;
  const uint32_t rem = man & ((1u << shift) - 1), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (halfMan & 1))) ++halfMan;
  if (exp < -14) return uint16_t(sign | halfMan);  // subnormal; a carry makes the least normal
  return uint16_t(sign | ((uint32_t(exp + 15) << 10) + (halfMan - 0x400)));
}
inline float bf2f(uint16_t b) { return bitsToFloat(uint32_t(b) << 16); }
inline uint16_t f2bf(float f) {
  uint32_t u = floatBits(f);
  if ((u & 0x7FFFFFFF) > 0x7F800000u) return uint16_t((u >> 16) | 0x40);
  u += 0x7FFF + ((u >> 16) & 1);
  return uint16_t(u >> 16);
}

inline void parallelFor(uint32_t n, int threads, const std::function<void(uint32_t, uint32_t)> &body) {
  uint32_t t = threads > 0 ? uint32_t(threads) : std::max(1u, std::thread::hardware_concurrency());
  t = std::min(t, std::max(1u, n));
  if (t <= 1) { body(0, n); return; }
  std::vector<std::thread> pool;
  for (uint32_t i = 0; i < t; ++i) {
    const uint32_t lo = uint64_t(n) * i / t, hi = uint64_t(n) * (i + 1) / t;
    pool.emplace_back([&body, lo, hi] { body(lo, hi); });
  }
  for (auto &th : pool) th.join();
}

} // namespace orc
