// Load-time re-tiling of native GGUF K-quant rows into the weight image of abi/Gguf.h (the
// counterpart of the reference's repack into planes: runtime/model/GgufPreparation.cpp,
// kernels/shared/gguf_repack.metal). Host code; the image's bytes equal the native rows'.
#pragma once
#include "abi/Gguf.h"

#include <cstdint>
#include <vector>

namespace splash::ops {

// The image of `rows` native rows of `inputSize` values (rows a multiple of 16, inputSize of 256).
// Throws std::invalid_argument for another format or shape.
void packGgufImage(uint32_t formatId, const uint8_t *native, uint32_t rows, uint32_t inputSize, uint8_t *image);
[[nodiscard]] std::vector<uint8_t> packGgufImage(uint32_t formatId, const std::vector<uint8_t> &native, uint32_t rows,
                                                 uint32_t inputSize);
// The inverse: native rows of an image (decode(retile(native)) == decode(native) follows from
// unpack(pack(native)) == native, which the CPU tests check).
void unpackGgufImage(uint32_t formatId, const uint8_t *image, uint32_t rows, uint32_t inputSize, uint8_t *native);


// ggml's Q3_K (super-blocks of 110 bytes: 32 of mask bits, 64 of two-bit codes, sixteen 6-bit scales in 12, a half d;
// value = d (scale - 32) (code - 4 [mask bit clear])) has no kernels of its own. Its blocks are rewritten at load time
// as Q6_K blocks of the same values: the same d, the scale of each sixteen values less 32 as Q6_K's signed byte, and
// the code's value q in [-4, 3] as Q6_K's six-bit q + 32. Both formats evaluate d * scale * q in that order, so every
// value, and with it every projection, is bit for bit the Q3_K block's; the image holds 210 bytes a block for 110.
inline constexpr uint32_t kQ3KNativeBytes = 110;
void transcodeQ3KToQ6K(const uint8_t *q3k, uint64_t blocks, uint8_t *q6k);

} // namespace splash::ops
