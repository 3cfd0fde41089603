// Device-side decode of the K-quant and Q8_0 weight images (abi/Gguf.h): every kernel that reads the
// image -- the projection tiles, the value dump of the bit-exactness test -- unpacks it through
// these functions, so the test of one covers the others.
#pragma once
#include "abi/Gguf.h"
#include "kernels/device_common.hpp"

namespace splash::kernels {

// The 6-bit scales and mins of a Q4_K super-block (llama.cpp get_scale_min_k4; the reference's
// quant_formats.h:105-118), four per word as bytes: scales of groups 0..3 and 4..7, mins likewise.
struct Q4KScales {
  uint32_t sc_lo, sc_hi, mn_lo, mn_hi;
  float d, dmin;
};
__device__ __forceinline__ Q4KScales q4k_scales(uint4 meta) {
  Q4KScales s;
  s.d = half_bits_to_float(meta.x & 0xFFFFu);
  s.dmin = half_bits_to_float(meta.x >> 16);
  s.sc_lo = meta.y & 0x3F3F3F3Fu;
  s.mn_lo = meta.z & 0x3F3F3F3Fu;
  s.sc_hi = (meta.w & 0x0F0F0F0Fu) | ((meta.y >> 2) & 0x30303030u);
  s.mn_hi = ((meta.w >> 4) & 0x0F0F0F0Fu) | ((meta.z >> 2) & 0x30303030u);
  return s;
}
__device__ __forceinline__ float byte_of(uint32_t word, uint32_t index) { return float((word >> (8u * index)) & 0xFFu); }

// Register j (0..3) of a group's bf16 operands 128 + code, from the two words that hold the
// lane's eight codes of that group in their low (high = false) or high nibbles.
// (a & mask) | base in one instruction: the mask rides the scalar bus, the base a register (on
// this ISA a three-operand vector instruction takes no literal, so the compiler would emit two).
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t base) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(base));
  return r;
}
template <bool High> __device__ __forceinline__ uint4 q4_operands(uint32_t wa, uint32_t wb) {
  constexpr uint32_t kMask = 0x000F000Fu, kBase = 0x43004300u;  // bf16 0x4300 = 128, ulp 1
  constexpr uint32_t s = High ? 4u : 0u;
  uint4 r;
  r.x = and_or(s ? wa >> s : wa, kMask, kBase);
  r.y = and_or(wa >> (s + 8u), kMask, kBase);
  r.z = and_or(s ? wb >> s : wb, kMask, kBase);
  r.w = and_or(wb >> (s + 8u), kMask, kBase);
  return r;
}
// The same for Q6_K: the low nibbles as Q4_K's, then the 2-bit high fields of pair v0..v0+3 of
// the high-bits word (abi/Gguf.h) at bits 4..5 of each half.
template <bool High, uint32_t V0> __device__ __forceinline__ uint4 q6_operands(uint32_t wa, uint32_t wb, uint32_t hw) {
  constexpr uint32_t kHigh = 0x00300030u;
  uint4 r = q4_operands<High>(wa, wb);
  auto with = [&](uint32_t v, uint32_t low) -> uint32_t {
    return and_or(2u * v > 4u ? hw >> (2u * v - 4u) : 2u * v < 4u ? hw << (4u - 2u * v) : hw, kHigh, low);
  };
  r.x = with(V0, r.x);
  r.y = with(V0 + 1, r.y);
  r.z = with(V0 + 2, r.z);
  r.w = with(V0 + 3, r.w);
  return r;
}

// The same for Q5_K: the low nibbles as Q4_K's, then the fifth bits of registers R0 .. R0 + 3 of the record
// half's fifth-bits word (abi/Gguf.h: bit r the low half's, bit 16 + r the high half's) at bit 4 of each half.
template <bool High, uint32_t R0> __device__ __forceinline__ uint4 q5_operands(uint32_t wa, uint32_t wb, uint32_t hw) {
  constexpr uint32_t kFifth = 0x00100010u;
  uint4 r = q4_operands<High>(wa, wb);
  auto with = [&](uint32_t reg, uint32_t low) -> uint32_t {
    return and_or(reg > 4u ? hw >> (reg - 4u) : reg < 4u ? hw << (4u - reg) : hw, kFifth, low);
  };
  r.x = with(R0, r.x);
  r.y = with(R0 + 1, r.y);
  r.z = with(R0 + 2, r.z);
  r.w = with(R0 + 3, r.w);
  return r;
}
// Q8_0: the bf16 operands 128 + value of a group from the words of its inputs 4 kq .. 4 kq + 3 (wa) and
// 16 + 4 kq .. + 3 (wb). value + 128 is the byte with its sign bit flipped; an integer up to 255 is exact in
// fp32 and in bf16, whose bits are the fp32's upper half.
// The operands of a group from its bytes 0..255 themselves: a the inputs 4 kq .. 4 kq + 3, b the inputs 16 + 4 kq .. + 3.
__device__ __forceinline__ uint4 byte_operands(uint32_t a, uint32_t b) {
  auto pair = [](uint32_t first, uint32_t second) -> uint32_t {  // bf16(first) in the low half, bf16(second) in the high
    return __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, float(second)), __builtin_bit_cast(uint32_t, float(first)), 0x07060302u);
  };
  uint4 r;
  r.x = pair(a & 0xFFu, (a >> 16) & 0xFFu);
  r.y = pair((a >> 8) & 0xFFu, a >> 24);
  r.z = pair(b & 0xFFu, (b >> 16) & 0xFFu);
  r.w = pair((b >> 8) & 0xFFu, b >> 24);
  return r;
}
__device__ __forceinline__ uint4 q8_operands(uint32_t wa, uint32_t wb) { return byte_operands(wa ^ 0x80808080u, wb ^ 0x80808080u); }

// IQ4_XS and IQ4_NL: 128 + the codebook value of each of four codes (one a byte, 0..15), by two byte permutes over the
// codebook's halves and a select on the codes' bit 3. The codebook (ggml's kvalues_iq4nl):
// -127 -104 -83 -65 -49 -35 -22 -10 1 13 25 38 53 69 89 113.
__device__ __forceinline__ uint32_t iq4_bytes(uint32_t codes) {
  constexpr uint32_t kT0 = 0x3F2D1801u, kT1 = 0x766A5D4Fu, kT2 = 0xA6998D81u, kT3 = 0xF1D9C5B5u;  // 128 + value, code 0 lowest
  const uint32_t index = codes & 0x07070707u;
  const uint32_t low = __builtin_amdgcn_perm(kT1, kT0, index), high = __builtin_amdgcn_perm(kT3, kT2, index);
  const uint32_t upper = ((codes >> 3) & 0x01010101u) * 0xFFu;  // 0xFF in the bytes of codes 8..15
  return (high & upper) | (low & ~upper);
}
// The operands of a group from the word of the lane's eight codes (abi/Gguf.h): low nibbles inputs 4 kq .. + 3, high
// nibbles inputs 16 + 4 kq .. + 3.
__device__ __forceinline__ uint4 iq4_operands(uint32_t word) {
  return byte_operands(iq4_bytes(word & 0x0F0F0F0Fu), iq4_bytes((word >> 4) & 0x0F0F0F0Fu));
}

// The code (0..15, or 0..63 for Q6_K) in half `half` of operand register `reg`.
__device__ __forceinline__ uint32_t operand_code(uint32_t reg, uint32_t half) { return (reg >> (16u * half)) & 0x7Fu; }

} // namespace splash::kernels
