#include "ops/GgufImage.hpp"

#include <cstring>
#include <stdexcept>
#include <string>
#include <thread>

namespace splash::ops {

namespace {

void requireShape(uint32_t formatId, uint32_t rows, uint32_t inputSize) {
  if (!gguf_record_bytes(formatId)) throw std::invalid_argument("no weight image for format " + std::to_string(formatId));
  if (!rows || rows % GGUF_TILE_COLUMNS) throw std::invalid_argument("a weight image holds whole tiles of 16 rows");
  if (!inputSize || inputSize % GGUF_BLOCK) throw std::invalid_argument("a weight image holds whole super-blocks of 256 inputs");
}

// Q6_K: the 6-bit code of input k (0..255) of a native block (llama.cpp dequantize_row_q6_K order).
inline uint32_t q6Code(const uint8_t *blk, uint32_t k) {
  const uint32_t n = k / 128, r = (k % 128) / 32, e = k % 32;
  const uint32_t l4 = (blk[64 * n + e + 32 * (r & 1)] >> (4 * (r >> 1))) & 15u;
  const uint32_t h2 = (blk[128 + 32 * n + e] >> (2 * r)) & 3u;
  return l4 | (h2 << 4);
}
inline void q6SetCode(uint8_t *blk, uint32_t k, uint32_t code) {
  const uint32_t n = k / 128, r = (k % 128) / 32, e = k % 32;
  uint8_t &low = blk[64 * n + e + 32 * (r & 1)];
  low = uint8_t((low & ~(0xFu << (4 * (r >> 1)))) | ((code & 15u) << (4 * (r >> 1))));
  uint8_t &high = blk[128 + 32 * n + e];
  high = uint8_t((high & ~(0x3u << (2 * r))) | ((code >> 4) << (2 * r)));
}

template <class Body> void forTiles(uint32_t tiles, Body body) {
  const uint32_t workers = std::min<uint32_t>(std::max(1u, std::thread::hardware_concurrency()), std::max(1u, tiles / 8));
  if (workers <= 1) { for (uint32_t t = 0; t < tiles; ++t) body(t); return; }
  std::vector<std::thread> pool;
  for (uint32_t w = 0; w < workers; ++w)
    pool.emplace_back([=] { for (uint32_t t = w; t < tiles; t += workers) body(t); });
  for (auto &th : pool) th.join();
}

// The nibble part of a record: lane (c, kq), half h, word w (0..3) holds, in its low nibbles, the
// codes of group 4 h + 2 (w / 2) and, in its high nibbles, of group 4 h + 2 (w / 2) + 1, for inputs
// 16 (w % 2) + 4 kq + 0..3 of each group, one byte per input.
inline uint32_t nibbleOffset(uint32_t c, uint32_t kq, uint32_t h, uint32_t w) { return 1024 * h + 16 * (kq * 16 + c) + 4 * w; }

} // namespace

void packGgufImage(uint32_t formatId, const uint8_t *native, uint32_t rows, uint32_t inputSize, uint8_t *image) {
  requireShape(formatId, rows, inputSize);
  const uint32_t blocks = inputSize / GGUF_BLOCK, nb = gguf_native_bytes(formatId), rb = gguf_record_bytes(formatId);
  const size_t rowBytes = size_t(blocks) * nb;
  forTiles(rows / GGUF_TILE_COLUMNS, [&](uint32_t tile) {
    for (uint32_t b = 0; b < blocks; ++b) {
      uint8_t *rec = image + (size_t(tile) * blocks + b) * rb;
      std::memset(rec, 0, rb);
      for (uint32_t c = 0; c < 16; ++c) {
        const uint8_t *blk = native + size_t(16 * tile + c) * rowBytes + size_t(b) * nb;
        if (formatId == GGUF_FMT_Q4K) {
          // Native qs byte 32 p + i holds input i of groups 2 p (low) and 2 p + 1 (high): the
          // record's words are native words, moved.
          const uint8_t *qs = blk + 16;
          for (uint32_t kq = 0; kq < 4; ++kq)
            for (uint32_t h = 0; h < 2; ++h)
              for (uint32_t w = 0; w < 4; ++w)
                std::memcpy(rec + nibbleOffset(c, kq, h, w), qs + 64 * h + 32 * (w / 2) + 16 * (w % 2) + 4 * kq, 4);
          std::memcpy(rec + 2048 + 16 * c, blk, 16);
        } else if (formatId == GGUF_FMT_Q5K) {
          // Native: d, dmin, 12 scale bytes, qh[32] (bit j of byte i: the fifth bit of input i of group j), qs[128] as Q4_K's.
          const uint8_t *qh = blk + 16, *qs = blk + 48;
          for (uint32_t kq = 0; kq < 4; ++kq) {
            for (uint32_t h = 0; h < 2; ++h) {
              for (uint32_t w = 0; w < 4; ++w)
                std::memcpy(rec + nibbleOffset(c, kq, h, w), qs + 64 * h + 32 * (w / 2) + 16 * (w % 2) + 4 * kq, 4);
              uint32_t word = 0;
              for (uint32_t gi = 0; gi < 4; ++gi)
                for (uint32_t j = 0; j < 4; ++j)
                  for (uint32_t half = 0; half < 2; ++half) {
                    const uint32_t group = 4 * h + gi, input = gguf_operand_input(kq, 2 * j + half);
                    word |= ((qh[input] >> group) & 1u) << (4 * gi + j + 16 * half);
                  }
              std::memcpy(rec + GGUF_Q5K_HIGH + 8 * (kq * 16 + c) + 4 * h, &word, 4);
            }
          }
          std::memcpy(rec + GGUF_Q5K_META + 16 * c, blk, 16);
        } else if (formatId == GGUF_FMT_IQ4XS || formatId == GGUF_FMT_IQ4NL) {
          // Native IQ4_XS: d, scales_h, scales_l[4], qs[128]; IQ4_NL: eight blocks of (fp16 d, qs[16]). Byte j of a
          // group's 16 holds inputs j (low nibble) and 16 + j (high): the record's words are native words, moved.
          const bool xs = formatId == GGUF_FMT_IQ4XS;
          for (uint32_t group = 0; group < 8; ++group) {
            const uint8_t *qs = xs ? blk + 8 + 16 * group : blk + 18 * group + 2;
            for (uint32_t kq = 0; kq < 4; ++kq) std::memcpy(rec + nibbleOffset(c, kq, group / 4, group % 4), qs + 4 * kq, 4);
            if (!xs) std::memcpy(rec + GGUF_IQ4_SCALES + 16 * c + 2 * group, blk + 18 * group, 2);
          }
          if (xs) std::memcpy(rec + GGUF_IQ4_SCALES + 8 * c, blk, 8);
        } else if (formatId == GGUF_FMT_Q80) {
          // Native: eight blocks of (fp16 d, 32 int8).
          for (uint32_t group = 0; group < 8; ++group) {
            const uint8_t *q = blk + 34 * group + 2;
            for (uint32_t kq = 0; kq < 4; ++kq) {
              uint8_t *mine = rec + 1024 * (group / 2) + 16 * (kq * 16 + c) + 8 * (group % 2);
              std::memcpy(mine, q + 4 * kq, 4);
              std::memcpy(mine + 4, q + 16 + 4 * kq, 4);
            }
            std::memcpy(rec + GGUF_Q80_SCALES + 16 * c + 2 * group, blk + 34 * group, 2);
          }
        } else {
          for (uint32_t kq = 0; kq < 4; ++kq) {
            for (uint32_t h = 0; h < 2; ++h)
              for (uint32_t w = 0; w < 4; ++w)
                for (uint32_t i = 0; i < 4; ++i) {
                  const uint32_t group = 4 * h + 2 * (w / 2), input = 16 * (w % 2) + 4 * kq + i;
                  const uint32_t low = q6Code(blk, 32 * group + input) & 15u, high = q6Code(blk, 32 * (group + 1) + input) & 15u;
                  rec[nibbleOffset(c, kq, h, w) + i] = uint8_t(low | (high << 4));
                }
            // High bits: word i covers groups 2 i, 2 i + 1; pair v = register v % 4 of group
            // 2 i + v / 4; element e = 2 (v % 4) + half; fields at bits 2 v and 16 + 2 v.
            for (uint32_t i = 0; i < 4; ++i) {
              uint32_t word = 0;
              for (uint32_t v = 0; v < 8; ++v)
                for (uint32_t half = 0; half < 2; ++half) {
                  const uint32_t group = 2 * i + v / 4, e = 2 * (v % 4) + half;
                  const uint32_t code = q6Code(blk, 32 * group + gguf_operand_input(kq, e));
                  word |= (code >> 4) << (2 * v + 16 * half);
                }
              std::memcpy(rec + GGUF_Q6K_HIGH + 16 * (kq * 16 + c) + 4 * i, &word, 4);
            }
          }
          std::memcpy(rec + GGUF_Q6K_SCALES + 16 * c, blk + 192, 16);
          std::memcpy(rec + GGUF_Q6K_D + 2 * c, blk + 208, 2);
        }
      }
    }
  });
}

std::vector<uint8_t> packGgufImage(uint32_t formatId, const std::vector<uint8_t> &native, uint32_t rows, uint32_t inputSize) {
  requireShape(formatId, rows, inputSize);
  if (native.size() != gguf_image_bytes(formatId, rows, inputSize))
    throw std::invalid_argument("native rows do not match the tensor's shape");
  std::vector<uint8_t> image(native.size());
  packGgufImage(formatId, native.data(), rows, inputSize, image.data());
  return image;
}

void unpackGgufImage(uint32_t formatId, const uint8_t *image, uint32_t rows, uint32_t inputSize, uint8_t *native) {
  requireShape(formatId, rows, inputSize);
  const uint32_t blocks = inputSize / GGUF_BLOCK, nb = gguf_native_bytes(formatId), rb = gguf_record_bytes(formatId);
  const size_t rowBytes = size_t(blocks) * nb;
  forTiles(rows / GGUF_TILE_COLUMNS, [&](uint32_t tile) {
    for (uint32_t b = 0; b < blocks; ++b) {
      const uint8_t *rec = image + (size_t(tile) * blocks + b) * rb;
      for (uint32_t c = 0; c < 16; ++c) {
        uint8_t *blk = native + size_t(16 * tile + c) * rowBytes + size_t(b) * nb;
        std::memset(blk, 0, nb);
        if (formatId == GGUF_FMT_Q4K) {
          for (uint32_t kq = 0; kq < 4; ++kq)
            for (uint32_t h = 0; h < 2; ++h)
              for (uint32_t w = 0; w < 4; ++w)
                std::memcpy(blk + 16 + 64 * h + 32 * (w / 2) + 16 * (w % 2) + 4 * kq, rec + nibbleOffset(c, kq, h, w), 4);
          std::memcpy(blk, rec + 2048 + 16 * c, 16);
        } else if (formatId == GGUF_FMT_Q5K) {
          uint8_t *qh = blk + 16, *qs = blk + 48;
          for (uint32_t kq = 0; kq < 4; ++kq)
            for (uint32_t h = 0; h < 2; ++h) {
              for (uint32_t w = 0; w < 4; ++w)
                std::memcpy(qs + 64 * h + 32 * (w / 2) + 16 * (w % 2) + 4 * kq, rec + nibbleOffset(c, kq, h, w), 4);
              uint32_t word;
              std::memcpy(&word, rec + GGUF_Q5K_HIGH + 8 * (kq * 16 + c) + 4 * h, 4);
              for (uint32_t gi = 0; gi < 4; ++gi)
                for (uint32_t j = 0; j < 4; ++j)
                  for (uint32_t half = 0; half < 2; ++half) {
                    const uint32_t group = 4 * h + gi, input = gguf_operand_input(kq, 2 * j + half);
                    qh[input] = uint8_t(qh[input] | (((word >> (4 * gi + j + 16 * half)) & 1u) << group));
                  }
            }
          std::memcpy(blk, rec + GGUF_Q5K_META + 16 * c, 16);
        } else if (formatId == GGUF_FMT_IQ4XS || formatId == GGUF_FMT_IQ4NL) {
          const bool xs = formatId == GGUF_FMT_IQ4XS;
          for (uint32_t group = 0; group < 8; ++group) {
            uint8_t *qs = xs ? blk + 8 + 16 * group : blk + 18 * group + 2;
            for (uint32_t kq = 0; kq < 4; ++kq) std::memcpy(qs + 4 * kq, rec + nibbleOffset(c, kq, group / 4, group % 4), 4);
            if (!xs) std::memcpy(blk + 18 * group, rec + GGUF_IQ4_SCALES + 16 * c + 2 * group, 2);
          }
          if (xs) std::memcpy(blk, rec + GGUF_IQ4_SCALES + 8 * c, 8);
        } else if (formatId == GGUF_FMT_Q80) {
          for (uint32_t group = 0; group < 8; ++group) {
            uint8_t *q = blk + 34 * group + 2;
            for (uint32_t kq = 0; kq < 4; ++kq) {
              const uint8_t *mine = rec + 1024 * (group / 2) + 16 * (kq * 16 + c) + 8 * (group % 2);
              std::memcpy(q + 4 * kq, mine, 4);
              std::memcpy(q + 16 + 4 * kq, mine + 4, 4);
            }
            std::memcpy(blk + 34 * group, rec + GGUF_Q80_SCALES + 16 * c + 2 * group, 2);
          }
        } else {
          for (uint32_t kq = 0; kq < 4; ++kq) {
            uint32_t highWords[4];
            std::memcpy(highWords, rec + GGUF_Q6K_HIGH + 16 * (kq * 16 + c), 16);
            for (uint32_t group = 0; group < 8; ++group)
              for (uint32_t e = 0; e < 8; ++e) {
                const uint32_t input = gguf_operand_input(kq, e);
                // low nibble: word w = 2 ((group % 4) / 2) + input / 16 of half group / 4, byte input % 4 ... of lane kq
                const uint32_t h = group / 4, w = 2 * ((group % 4) / 2) + input / 16, i = input % 4;
                const uint8_t byte = rec[nibbleOffset(c, kq, h, w) + i];
                const uint32_t low = group % 2 ? byte >> 4 : byte & 15u;
                const uint32_t v = 4 * (group % 2) + e / 2, half = e % 2;
                const uint32_t high = (highWords[group / 2] >> (2 * v + 16 * half)) & 3u;
                q6SetCode(blk, 32 * group + input, low | (high << 4));
              }
          }
          std::memcpy(blk + 192, rec + GGUF_Q6K_SCALES + 16 * c, 16);
          std::memcpy(blk + 208, rec + GGUF_Q6K_D + 2 * c, 2);
        }
      }
    }
  });
}

namespace {
constexpr uint32_t kGgmlQ4_0 = 2, kGgmlQ5_0 = 6, kGgmlQ3_K = 11;
constexpr uint32_t kQ3KBytes = 110, kQ40Bytes = 18, kQ50Bytes = 22, kQ80Bytes = 34;
constexpr NativeRewrite kQ3KRewrite{GGUF_FMT_Q6K, kQ3KBytes}, kQ40Rewrite{GGUF_FMT_Q80, 8 * kQ40Bytes}, kQ50Rewrite{GGUF_FMT_Q80, 8 * kQ50Bytes};

void q3kAsQ6K(const uint8_t *q3k, uint64_t blocks, uint8_t *q6k) {
  constexpr uint32_t kScales3 = 96, kD3 = 108, kHigh6 = 128, kScales6 = 192, kD6 = 208;
  for (uint64_t b = 0; b < blocks; ++b, q3k += kQ3KBytes, q6k += GGUF_Q6K_NATIVE) {
    std::memset(q6k, 0, GGUF_Q6K_NATIVE);
    const uint8_t *mask = q3k, *codes = q3k + 32, *packed = q3k + kScales3;
    for (uint32_t i = 0; i < 16; ++i) {
      const int low = i < 8 ? packed[i] & 15 : packed[i - 8] >> 4, high = (packed[8 + i % 4] >> (2 * (i / 4))) & 3;
      q6k[kScales6 + i] = uint8_t(int8_t((low | (high << 4)) - 32));
    }
    // Value 32 j + k: Q3_K keeps its two bits at bit 2 (j % 4) of codes[32 (j / 4) + k] and its mask bit at bit j of
    // mask[k]; Q6_K keeps the low nibble at nibble j % 4 / 2 of ql[64 (j / 4) + 32 (j % 2) + k] and the high two bits at
    // bit 2 (j % 4) of qh[32 (j / 4) + k].
    for (uint32_t j = 0; j < 8; ++j)
      for (uint32_t k = 0; k < 32; ++k) {
        const int two = (codes[32 * (j / 4) + k] >> (2 * (j % 4))) & 3, set = (mask[k] >> j) & 1;
        const uint32_t q = uint32_t(two - (set ? 0 : 4) + 32), r = j % 4;
        q6k[64 * (j / 4) + 32 * (r & 1) + k] |= uint8_t((q & 15) << (4 * (r >> 1)));
        q6k[kHigh6 + 32 * (j / 4) + k] |= uint8_t((q >> 4) << (2 * r));
      }
    std::memcpy(q6k + kD6, q3k + kD3, 2);
  }
}

// Groups of 32 values: byte k of the sixteen holds value k in its low nibble and value 16 + k in its high one; Q5_0's
// fifth bit of value k is bit k of the four bytes after d.
void legacyAsQ80(bool five, const uint8_t *source, uint64_t groups, uint8_t *q80) {
  const uint32_t bytes = five ? kQ50Bytes : kQ40Bytes;
  for (uint64_t g = 0; g < groups; ++g, source += bytes, q80 += kQ80Bytes) {
    const uint8_t *high = source + 2, *nibbles = source + (five ? 6 : 2);
    std::memcpy(q80, source, 2);
    for (uint32_t k = 0; k < 32; ++k) {
      const int low = k < 16 ? nibbles[k] & 15 : nibbles[k - 16] >> 4;
      const int q = five ? (low | (((high[k / 8] >> (k % 8)) & 1) << 4)) - 16 : low - 8;
      q80[2 + k] = uint8_t(int8_t(q));
    }
  }
}
} // namespace

const NativeRewrite *nativeRewriteOf(uint32_t ggmlType) noexcept {
  return ggmlType == kGgmlQ3_K ? &kQ3KRewrite : ggmlType == kGgmlQ4_0 ? &kQ40Rewrite : ggmlType == kGgmlQ5_0 ? &kQ50Rewrite : nullptr;
}

void rewriteNative(uint32_t ggmlType, const uint8_t *source, uint64_t superBlocks, uint8_t *out) {
  if (ggmlType == kGgmlQ3_K) return q3kAsQ6K(source, superBlocks, out);
  if (ggmlType == kGgmlQ4_0 || ggmlType == kGgmlQ5_0) return legacyAsQ80(ggmlType == kGgmlQ5_0, source, superBlocks * 8, out);
  throw std::invalid_argument("ggml type " + std::to_string(ggmlType) + " is not read through another format's blocks");
}

} // namespace splash::ops
