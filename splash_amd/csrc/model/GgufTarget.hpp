// A dense decoder's weights from a GGUF file: the counterpart, for the dense verify driver, of the reference's
// GgufTargetLoader and planImages (runtime/model/GgufTarget.hpp:24-75, GgufImage.cpp:474-520, :696-713): the
// geometry from the file's metadata, each layer's projections as weight images (q|k|v one projection of three segments,
// each of its tensor's format), the norms as bf16, the token table as native rows and the head, tied to the token table
// when the file holds no output.weight.
#pragma once
#include "model/DenseVerify.hpp"
#include "model/GgufFile.hpp"

namespace splash::model {

// The geometry the file's metadata names (<architecture>.block_count, .embedding_length, .feed_forward_length,
// .attention.head_count, .attention.head_count_kv, .attention.key_length, .rope.freq_base; the vocabulary is the token
// table's rows). Throws GgufError for a missing key, an RMS epsilon other than 1e-6 or a geometry the kernels do not
// take.
[[nodiscard]] DenseDimensions ggufDenseDimensions(const GgufFile &file);
// Loads every weight of `verify` (built with ggufDenseDimensions(file)) from the file. Throws GgufError naming every
// tensor that is missing, of a type or shape the path does not read, or that the file holds and the loader does not
// read (biases, for one).
void loadGgufDenseWeights(hip::Backend &backend, const GgufFile &file, DenseVerify &verify);

} // namespace splash::model
