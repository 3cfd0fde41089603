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

} // namespace splash::ops
