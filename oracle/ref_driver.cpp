// Builds the reference's own header-only CPU references into oracle/_ref/libref.so, from the
// headers where they lie under /root/reference (never copied). Test infrastructure only: it
// cross-checks the oracle's restatement in this container; the GPU box uses the prebuilt file
// when it is there and skips the cross-check when it is not.
#include "GgufFormatReference.hpp"
#include "Q8PageFormatReference.hpp"
#include "StateCodecReference.hpp"

#include <cstdint>
#include <random>
#include <vector>

using namespace gguf_reference;

extern "C" {

uint16_t ref_f2h(float f) { return f2h(f); }
float ref_h2f(uint16_t h) { return h2f(h); }

int ref_dequant_rows(uint32_t fmt, const uint8_t *native, uint32_t rows, uint32_t K, float *out) {
  const uint32_t rb = rowBytes(Fmt(fmt), K);
  for (uint32_t r = 0; r < rows; ++r) rowValues(Fmt(fmt), native + size_t(r) * rb, K, out + size_t(r) * K);
  return 0;
}

// dev/tests/engine/GgufFixtures.hpp:148-165 (that header needs Foundation; its scale draw is the lambda below).
int ref_fixture(uint32_t fmt, uint32_t rows, uint32_t K, uint32_t seed, uint8_t *out) {
  std::mt19937 rng(seed);
  const std::vector<uint8_t> v = makeNative(Fmt(fmt), rows, K, rng, [&] {
    uint16_t h;
    do h = static_cast<uint16_t>(rng());
    while ((h & 0x7C00) == 0x7C00);
    return h;
  });
  memcpy(out, v.data(), v.size());
  return 0;
}

int ref_make_native(uint32_t fmt, uint32_t rows, uint32_t K, uint32_t seed, uint8_t *out) {
  std::mt19937 rng(seed);
  const std::vector<uint8_t> v = makeNative(Fmt(fmt), rows, K, rng);
  memcpy(out, v.data(), v.size());
  return 0;
}

// dot + projectionBound of one (x row, weight row) pair.
void ref_dot_bound(const float *x, const float *w, uint32_t K, double *value, double *bound) {
  const Dot d = dot(x, w, K);
  *value = d.value;
  *bound = projectionBound(d, false);
}

// The staged tile's bound of the same pair.
void ref_dot_bound_staged(const float *x, const float *w, uint32_t K, double *value, double *bound) {
  const Dot d = dot(x, w, K);
  *value = d.value;
  *bound = projectionBound(d, true);
}

float ref_kv_scale(float maximum) { return splash::kv::reference_detail::storedScale(maximum); }
int ref_kv_code(float value, float maximum) { return splash::kv::reference_detail::quantize(value, maximum); }


// StateCodecReference.hpp:38-61
int ref_state_codes(const float *values, uint32_t rows, uint32_t columns, uint8_t *image) {
  const std::vector<uint8_t> v = splash::test::stateCodesReference(values, rows, columns);
  std::copy(v.begin(), v.end(), image);
  return 0;
}
}
