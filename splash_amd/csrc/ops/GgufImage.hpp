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


// ggml types that have no kernels of their own and are rewritten at load time as blocks of a format that has, with the
// same values bit for bit (the formats evaluate scale * integer products in the same order, and the integers fit):
// * Q3_K (type 11; super-blocks of 110 bytes: 32 of mask bits, 64 of two-bit codes, sixteen 6-bit scales in 12, a half
//   d; value = d (scale - 32) (code - 4 [mask bit clear])) as Q6_K: the same d, the scale of each sixteen values less 32
//   as Q6_K's signed byte, and the code's value q in [-4, 3] as Q6_K's six-bit q + 32; 210 bytes for 110.
// * Q4_0 (type 2; 32 values: a half d, sixteen bytes of nibbles; value = d (code - 8)) and Q5_0 (type 6; d, 32 fifth
//   bits, sixteen bytes of nibbles; value = d (code - 16)) as Q8_0: the same d and code - 8 or code - 16 as its signed
//   byte; 34 bytes for 18 or 22.
struct NativeRewrite final {
  uint32_t imageFormat;   // GGUF_FMT_* of the blocks written
  uint32_t sourceBytes;   // bytes of 256 values of the source
};
// nullptr for a type read as it is (or not at all).
[[nodiscard]] const NativeRewrite *nativeRewriteOf(uint32_t ggmlType) noexcept;
// `superBlocks` times 256 values of `source` as gguf_native_bytes(imageFormat) bytes each. Throws std::invalid_argument for
// a type with no rewrite.
void rewriteNative(uint32_t ggmlType, const uint8_t *source, uint64_t superBlocks, uint8_t *out);

} // namespace splash::ops
