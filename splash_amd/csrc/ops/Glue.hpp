// Glue operators of the verify path: ops::Normalization (runtime/ops/Normalization.cpp:16-40),
// ops::Embedding (runtime/ops/Embedding.cpp:20-47) and ops::RoPE (runtime/ops/RoPE.hpp:33-37) of the
// reference, over kernels/glue.hip. Each validates its buffers and throws std::invalid_argument
// before it adds a dispatch.
#pragma once
#include "abi/Glue.h"
#include "hip/Backend.hpp"
#include "ops/Linear.hpp"

#include <vector>

namespace splash::ops {

class Normalization final {
public:
  // output = bf16((x * rsqrt(mean x^2 + 1e-6)) * weight) over `rows` rows of `width`.
  static void addRms(hip::CommandGraph &graph, const hip::Buffer &input, const hip::Buffer &weight, const hip::Buffer &output,
                     uint32_t width, uint32_t rows);
  // The same, and the projection activation table of the normalized rows in scratch.input; returns
  // what the table then describes (the reference's norm_rms_table16_decode producer).
  static PreparedInput addRmsTable(hip::CommandGraph &graph, const hip::Buffer &input, const hip::Buffer &weight,
                                   const hip::Buffer &output, const LinearScratch &scratch, uint32_t width, uint32_t rows);
};

// A token table's rows as stored: native K-quant blocks, gathered, never multiplied (Weights.hpp:227-260).
struct EmbeddingTable final {
  hip::Buffer rows;
  uint32_t formatId = GGUF_FMT_Q4K;
  uint32_t vocabulary = 0;
  uint32_t hidden = 0;
};
class Embedding final {
public:
  static void add(hip::CommandGraph &graph, const EmbeddingTable &table, const hip::Buffer &tokens, const hip::Buffer &output,
                  uint32_t rows);
};

// The fp32 projection of weights kept as rows (the reference's addGgufFloat, LinearGguf.cpp:545-612): output row r's
// columns [outOffset, outOffset + N) of outStride = sum_k x[r][k] W[n][k], fp32 or rounded to bf16.
class FloatProjection final {
public:
  static void add(hip::CommandGraph &graph, const hip::Buffer &input, const FloatRows &weights, const hip::Buffer &output,
                  uint32_t rows, uint32_t outStride, uint32_t outOffset, FloatOutput type);
};

// output = bf16(up * silu(gate)) over rows of bf16 values: the SwiGLU of rows whose gate and up were projected apart
// (a prompt chunk under the prefill tile, which has no gate/up epilogue); the arithmetic of LinearEpilogue::GateUp.
class SwiGlu final {
public:
  static void add(hip::CommandGraph &graph, const hip::Buffer &gate, const hip::Buffer &up, const hip::Buffer &output, uint64_t count);
};

struct RopeSequence final {
  uint32_t firstRow = 0, rows = 0, anchor = 0;
};
class RoPE final {
public:
  // cos/sin of (anchor + depth[row]) * inverseFrequency[pair] per packed row.
  static void addTreeTables(hip::CommandGraph &graph, const hip::Buffer &inverseFrequency, const hip::Buffer &depth,
                            const hip::Buffer &cosines, const hip::Buffer &sines, uint32_t pairs,
                            const std::vector<RopeSequence> &sequences);
};

// Rows of `stride` bf16 values from row `row` of a buffer, of which a copy reads or writes the values
// from `column` on (RowCopy.hpp:9-15 in the reference).
struct RowRegion final {
  uint32_t row = 0, stride = 0, column = 0;
};
// Copies rows of bf16 values between two row regions: a capture layer's output rows into their slot
// of the draft's captured target hidden rows (RowCopy.hpp:17-28, QwenTarget.cpp addCapture).
class RowCopy final {
public:
  static void add(hip::CommandGraph &graph, const hip::Buffer &source, RowRegion from, const hip::Buffer &destination, RowRegion to,
                  uint32_t rows, uint32_t width);
};

} // namespace splash::ops
