// Header parser for llama.cpp GGUF files (version 3) and the step from a file's tensor to what the
// operators take: the counterpart of the reference's runtime/model/GgufFile.hpp:24-150 (GgufFile,
// GgufTensor, GgufMetadata) and of the image preparation in GgufImage.cpp, scoped to the formats
// the projections read (Q4_K, Q5_K, Q6_K, Q8_0) and the 16/32-bit vectors of the norms. The file is
// mapped read-only; tensor data is read in place.
#pragma once
#include "hip/Backend.hpp"

#include <cstdint>
#include <map>
#include <optional>
#include <stdexcept>
#include <string>
#include <string_view>
#include <vector>

namespace splash::model {

class GgufError : public std::runtime_error {
public:
  using std::runtime_error::runtime_error;
};

// ggml type ids as GGUF tensor infos store them (ggml-common.h; GgufFile.hpp:35-66 in the reference).
namespace ggml {
inline constexpr uint32_t kF32 = 0, kF16 = 1, kQ4_0 = 2, kQ5_0 = 6, kQ8_0 = 8, kQ3_K = 11, kQ4_K = 12, kQ5_K = 13, kQ6_K = 14, kIQ4_NL = 20, kIQ4_XS = 23, kBF16 = 30;
}
struct GgmlTypeTraits {
  const char *name;
  uint32_t blockElements;
  uint32_t blockBytes;
};
// nullptr for a type this parser cannot size.
[[nodiscard]] const GgmlTypeTraits *ggmlTypeTraits(uint32_t type) noexcept;
// The weight-image format (abi/Gguf.h) of a ggml type, if the projections read it. Q3_K is read as Q6_K and Q4_0 and
// Q5_0 as Q8_0: the loader rewrites their blocks as blocks of the same values (ops::rewriteNative).
[[nodiscard]] std::optional<uint32_t> imageFormat(uint32_t ggmlType) noexcept;

struct GgufTensor {
  std::string name;
  uint32_t type = 0;
  std::vector<uint64_t> dims;  // dims[0] is the fastest (row length)
  uint64_t offset = 0;         // in the tensor data of the file that holds it
  uint64_t bytes = 0;
  uint32_t file = 0;           // which part of a split GGUF holds it (GgufFile.hpp:74 in the reference)
  [[nodiscard]] uint64_t columns() const noexcept { return dims.empty() ? 0 : dims[0]; }
  [[nodiscard]] uint64_t rows() const noexcept;
  [[nodiscard]] uint64_t elements() const noexcept { return columns() * rows(); }
};

// Scalar metadata by key: every integer and boolean as unsigned (a negative one as its two's
// complement), every float as a double, and the strings (GgufFile.hpp:95-107).
struct GgufMetadata {
  std::map<std::string, uint64_t, std::less<>> unsigneds;
  std::map<std::string, double, std::less<>> floats;
  std::map<std::string, std::string, std::less<>> strings;
  [[nodiscard]] std::optional<uint64_t> unsignedValue(std::string_view key) const;
  [[nodiscard]] std::optional<double> floatValue(std::string_view key) const;
  [[nodiscard]] std::optional<std::string> stringValue(std::string_view key) const;
};

class GgufFile final {
public:
  // Maps the file and parses its header; throws GgufError on a malformed or truncated file.
  explicit GgufFile(const std::string &path);
  // The parts of a split GGUF in split order (GgufFile.hpp:118-124, GgufFile.cpp:167-201 in the reference): the first
  // part's metadata is kept, and its split.count and split.tensors.count, where it states them, must describe the parts
  // read (a part read alone is refused); a later part's split.no must be its place; a part of no tensors may end at
  // its header. One path is the single file.
  explicit GgufFile(const std::vector<std::string> &paths);
  ~GgufFile();
  GgufFile(const GgufFile &) = delete;
  GgufFile &operator=(const GgufFile &) = delete;

  [[nodiscard]] const GgufMetadata &metadata() const noexcept { return metadata_; }
  [[nodiscard]] const std::vector<GgufTensor> &tensors() const noexcept { return tensors_; }
  [[nodiscard]] const GgufTensor *find(std::string_view name) const noexcept;
  [[nodiscard]] const GgufTensor &require(std::string_view name) const;
  // The tensor's bytes in the mapped file.
  [[nodiscard]] const uint8_t *data(const GgufTensor &tensor) const;
  [[nodiscard]] size_t parts() const noexcept { return parts_.size(); }

private:
  struct Part {
    const uint8_t *base = nullptr;
    uint64_t size = 0;
    uint64_t dataStart = 0;
  };
  void parse(const std::string &path, uint32_t file);
  void unmap() noexcept;
  std::vector<Part> parts_;
  GgufMetadata metadata_;
  std::vector<GgufTensor> tensors_;
  std::map<std::string, size_t, std::less<>> index_;
};

// A projection tensor's weight image in device memory.
struct LoadedImage {
  uint32_t formatId = 0;
  uint32_t rows = 0;       // output size
  uint32_t inputSize = 0;  // K
  hip::Buffer image;
};
// Packs rows [firstRow, firstRow + rows) of a 2-D tensor of an image format (whole 16-row tiles of
// whole 256-input super-blocks) and uploads them; rows = 0 takes all.
[[nodiscard]] LoadedImage loadImage(hip::Backend &backend, const GgufFile &file, const GgufTensor &tensor, uint32_t firstRow = 0,
                                    uint32_t rows = 0);
// A projection tensor's native rows in device memory, in the format imageFormat names (what the token gather decodes).
[[nodiscard]] hip::Buffer loadNativeRows(hip::Backend &backend, const GgufFile &file, const GgufTensor &tensor, const char *label);
// The rows of a tensor an image, a table of float rows or a vector takes, in the order it takes them: runs of source
// rows one after the other (the reference's TensorRows with its RowOrder, GgufImage.hpp:29-38). All rows when empty.
struct RowRun final {
  uint64_t first = 0, rows = 0;
};
using RowRuns = std::vector<RowRun>;
// Value heads of `headRows` rows from row `from` on, which llama.cpp stores tiled (value head j of key head h at
// j * keyHeads + h) and these kernels group by key head (h * valueHeadsPerKey + j): the runs that put `rows` rows of a
// tensor in grouped order (GgufImage.hpp:29-38, GgufImage.cpp:410-413); rows below `from` keep their order.
[[nodiscard]] RowRuns groupedHeadRows(uint64_t rows, uint64_t from, uint32_t headRows, uint32_t keyHeads, uint32_t valueHeadsPerKey);
// The weight image of `runs` of a tensor of an image format (any rank: its rows are those of all its outer
// dimensions), columns [firstColumn, firstColumn + columns) of each (whole super-blocks; columns 0: all), the runs'
// rows whole 16-row tiles in all.
[[nodiscard]] LoadedImage loadImageRows(hip::Backend &backend, const GgufFile &file, const GgufTensor &tensor, const RowRuns &runs,
                                        uint64_t firstColumn = 0, uint64_t columns = 0);
// The same on the host: `images` images one after the other, image i of images[i]'s rows.
struct PackedImages {
  uint32_t formatId = 0, rows = 0, inputSize = 0;
  std::vector<uint8_t> bytes;
};
[[nodiscard]] PackedImages packImagesOfRows(const GgufFile &file, const GgufTensor &tensor, const std::vector<RowRuns> &images,
                                            uint64_t firstColumn = 0, uint64_t columns = 0);
// `count` images one after the other in one buffer, image i of runs[i] (a layer's experts, each expert's rows an image).
[[nodiscard]] LoadedImage loadImagesOfRows(hip::Backend &backend, const GgufFile &file, const GgufTensor &tensor,
                                           const std::vector<RowRuns> &images, uint64_t firstColumn = 0, uint64_t columns = 0);
// Rows of an F32, BF16 or F16 tensor as the fp32 projection reads them: F32 and BF16 as stored, F16 widened to F32
// (GgufImage.cpp:353-366, :372-386). bfloat16: whether the rows are BF16.
struct LoadedFloatRows {
  hip::Buffer rows;
  uint32_t outputSize = 0, inputSize = 0;
  bool bfloat16 = false;
};
[[nodiscard]] LoadedFloatRows loadFloatRows(hip::Backend &backend, const GgufFile &file, const std::vector<const GgufTensor *> &tensors,
                                            const RowRuns &runs = {});
// The values of `runs` of an F32, F16 or BF16 tensor (rows of its first dimension) as fp32, or narrowed to bf16.
[[nodiscard]] hip::Buffer loadFloat32Values(hip::Backend &backend, const GgufFile &file, const GgufTensor &tensor, const RowRuns &runs = {});
[[nodiscard]] hip::Buffer loadBf16Values(hip::Backend &backend, const GgufFile &file, const GgufTensor &tensor, const RowRuns &runs = {});
// A 1-D F32, F16 or BF16 tensor as bf16 in device memory (the norms' weights).
[[nodiscard]] hip::Buffer loadBf16Vector(hip::Backend &backend, const GgufFile &file, const GgufTensor &tensor);

} // namespace splash::model
