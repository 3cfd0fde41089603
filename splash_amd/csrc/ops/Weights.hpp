// Quantized projection weights as the operators see them (the reference's runtime/ops/Weights.hpp:
// QuantizedSegment :108-160, BlockWeights :162-164, Projection :170-225): a projection is a list of
// column segments, each one tensor's weight image in HBM (abi/Gguf.h).
#pragma once
#include "abi/Gguf.h"
#include "hip/Backend.hpp"

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

namespace splash::ops {

enum class FloatOutput : uint8_t { BFloat16, Float32 };

struct QuantizedSegment final {
  // The image of an [outputSize, inputSize] tensor of formatId (gguf_image_bytes).
  [[nodiscard]] static QuantizedSegment ofImage(uint32_t formatId, uint32_t outputSize, uint32_t inputSize,
                                              hip::Buffer image, uint32_t columnOffset = 0) {
    if (!gguf_record_bytes(formatId)) throw std::invalid_argument("no weight image for format " + std::to_string(formatId));
    QuantizedSegment s;
    s.image = std::move(image);
    s.outputSize = outputSize;
    s.inputSize = inputSize;
    s.columnOffset = columnOffset;
    s.formatId = formatId;
    return s;
  }
  hip::Buffer image;
  uint32_t outputSize = 0;
  uint32_t inputSize = 0;
  uint32_t columnOffset = 0;
  uint32_t formatId = GGUF_FMT_Q4K;
  // The kernel name token of its format (the reference's kQuantFormats[].name).
  [[nodiscard]] const char *name() const noexcept { return gguf_format_name(formatId); }
};

// Weights kept as rows of floats, [outputSize][inputSize] F32 or BF16 as their file stores them, which the fp32
// projection reads (the reference's float segments, Weights.hpp:108-160 isFloat; a MoE router, the GDN alpha/beta
// gates of a GGUF that keeps them F32).
struct FloatRows final {
  hip::Buffer rows;
  uint32_t outputSize = 0;
  uint32_t inputSize = 0;
  bool bfloat16 = false;
  [[nodiscard]] explicit operator bool() const noexcept { return static_cast<bool>(rows); }
  [[nodiscard]] uint64_t weightBytes() const noexcept { return uint64_t{outputSize} * inputSize * (bfloat16 ? 2 : 4); }
};

struct BlockWeights final {
  std::vector<QuantizedSegment> segments;
};

// A projection of outputSize x inputSize whose segments tile its leading output columns in order
// (Weights.hpp:170-186 in the reference, same checks).
class Projection final {
public:
  Projection() = default;
  Projection(uint32_t output, uint32_t input, BlockWeights weights)
      : outputSize(output), inputSize(input), weights_(std::move(weights)) {
    if (weights_.segments.empty()) throw std::invalid_argument("block projection has no segments");
    uint32_t covered = 0;
    for (const QuantizedSegment &s : weights_.segments) {
      if (s.inputSize != input || s.columnOffset != covered || !s.outputSize || s.outputSize > output - covered)
        throw std::invalid_argument("block segments do not tile the projection");
      covered += s.outputSize;
    }
  }
  [[nodiscard]] const BlockWeights &blocks() const noexcept { return weights_; }
  // Rows [first, first + count) of a projection's weights (Weights.hpp:193-204 in the reference).
  struct RowRange final {
    uint32_t first = 0;
    uint32_t count = 0;
  };
  // A view of a projection of one tensor over the rows of `ranges`, whole 16-row tiles of them (an empty range holds
  // none), which become its output columns in order: segments over slices of the same image (an image is rows of
  // sixteen columns, so a range of whole tiles is contiguous in it), no copy. The draft's head over a subset of the
  // vocabulary (DraftVocabulary::rows) and its context writers' key and value rows are such views.
  [[nodiscard]] Projection rows(std::initializer_list<RowRange> ranges) const {
    if (weights_.segments.size() != 1) throw std::invalid_argument("a row view is of a projection of one tensor");
    const QuantizedSegment &whole = weights_.segments.front();
    BlockWeights view;
    uint32_t covered = 0;
    for (const RowRange &range : ranges) {
      if (range.first % GGUF_TILE_COLUMNS || range.count % GGUF_TILE_COLUMNS || range.first > outputSize || range.count > outputSize - range.first)
        throw std::invalid_argument("a row view takes whole 16-row tiles inside the projection");
      if (!range.count) continue;
      view.segments.push_back(QuantizedSegment::ofImage(whole.formatId, range.count, inputSize,
                                                        whole.image.slice(gguf_image_bytes(whole.formatId, range.first, inputSize),
                                                                          gguf_image_bytes(whole.formatId, range.count, inputSize)),
                                                        covered));
      covered += range.count;
    }
    Projection result(covered, inputSize, std::move(view));
    result.destination = destination;
    return result;
  }
  // Native bytes of its weights: what one pass over it streams from HBM.
  [[nodiscard]] uint64_t weightBytes() const noexcept {
    uint64_t bytes = 0;
    for (const QuantizedSegment &s : weights_.segments) bytes += gguf_image_bytes(s.formatId, s.outputSize, s.inputSize);
    return bytes;
  }
  uint32_t outputSize = 0;
  uint32_t inputSize = 0;
  // fp32 only for plain plans (the LM head's logits).
  FloatOutput destination = FloatOutput::BFloat16;

private:
  BlockWeights weights_;
};

} // namespace splash::ops
