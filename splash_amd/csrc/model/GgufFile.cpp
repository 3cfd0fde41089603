#include "model/GgufFile.hpp"

#include "abi/Gguf.h"
#include "ops/GgufImage.hpp"

#include <array>
#include <cmath>
#include <cstring>
#include <set>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

namespace splash::model {

namespace {

constexpr std::array<std::pair<uint32_t, GgmlTypeTraits>, 14> kTypes{{
    {0, {"F32", 1, 4}},        {1, {"F16", 1, 2}},        {2, {"Q4_0", 32, 18}},    {3, {"Q4_1", 32, 20}},
    {6, {"Q5_0", 32, 22}},     {8, {"Q8_0", 32, 34}},     {10, {"Q2_K", 256, 84}},   {11, {"Q3_K", 256, 110}}, {12, {"Q4_K", 256, 144}},
    {13, {"Q5_K", 256, 176}},  {14, {"Q6_K", 256, 210}},  {20, {"IQ4_NL", 32, 18}},   {23, {"IQ4_XS", 256, 136}},
    {30, {"BF16", 1, 2}},
}};

// GGUF metadata value types.
enum : uint32_t { kU8, kI8, kU16, kI16, kU32, kI32, kF32, kBool, kString, kArray, kU64, kI64, kF64 };

struct Reader {
  const uint8_t *base;
  uint64_t size, at = 0;
  void need(uint64_t bytes) const {
    if (bytes > size - at) throw GgufError("GGUF header is truncated");
  }
  template <class T> T take() {
    need(sizeof(T));
    T v;
    std::memcpy(&v, base + at, sizeof(T));
    at += sizeof(T);
    return v;
  }
  std::string string() {
    const uint64_t n = take<uint64_t>();
    if (n > (1u << 24)) throw GgufError("GGUF string is too long");
    need(n);
    std::string s(reinterpret_cast<const char *>(base + at), n);
    at += n;
    return s;
  }
  void skipValue(uint32_t type) {
    static constexpr uint32_t kBytes[] = {1, 1, 2, 2, 4, 4, 4, 1, 0, 0, 8, 8, 8};
    if (type == kString) { (void)string(); return; }
    if (type == kArray) {
      const uint32_t inner = take<uint32_t>();
      const uint64_t n = take<uint64_t>();
      if (inner == kArray || inner > kF64) throw GgufError("unsupported GGUF array");
      if (inner == kString) { for (uint64_t i = 0; i < n; ++i) (void)string(); return; }
      if (n > (size - at) / kBytes[inner]) throw GgufError("GGUF header is truncated");
      at += n * kBytes[inner];
      return;
    }
    if (type > kF64) throw GgufError("unknown GGUF metadata type");
    need(kBytes[type]);
    at += kBytes[type];
  }
};

float halfToFloat(uint16_t h) {
  const uint32_t sign = uint32_t(h & 0x8000u) << 16, exponent = (h >> 10) & 31u, mantissa = h & 0x3FFu;
  uint32_t bits;
  if (exponent == 31) bits = sign | 0x7F800000u | (mantissa << 13);
  else if (exponent) bits = sign | ((exponent + 112u) << 23) | (mantissa << 13);
  else if (!mantissa) bits = sign;
  else {
    int shift = 0;
    uint32_t m = mantissa;
    while (!(m & 0x400u)) { m <<= 1; ++shift; }
    bits = sign | ((113u - shift) << 23) | ((m & 0x3FFu) << 13);
  }
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}
uint16_t floatToBf16(float f) {  // nearest, ties to even
  uint32_t v;
  std::memcpy(&v, &f, 4);
  if ((v & 0x7FFFFFFFu) > 0x7F800000u) return uint16_t((v >> 16) | 0x40u);
  return uint16_t((v + 0x7FFFu + ((v >> 16) & 1u)) >> 16);
}

} // namespace

const GgmlTypeTraits *ggmlTypeTraits(uint32_t type) noexcept {
  for (const auto &[id, traits] : kTypes)
    if (id == type) return &traits;
  return nullptr;
}

std::optional<uint32_t> imageFormat(uint32_t ggmlType) noexcept {
  switch (ggmlType) {
    case ggml::kQ4_K: return GGUF_FMT_Q4K;
    case ggml::kQ5_K: return GGUF_FMT_Q5K;
    case ggml::kQ6_K: return GGUF_FMT_Q6K;
    case ggml::kQ3_K: case ggml::kQ4_0: case ggml::kQ5_0: return ops::nativeRewriteOf(ggmlType)->imageFormat;
    case ggml::kQ8_0: return GGUF_FMT_Q80;
    case ggml::kIQ4_XS: return GGUF_FMT_IQ4XS;
    case ggml::kIQ4_NL: return GGUF_FMT_IQ4NL;
    default: return std::nullopt;
  }
}

uint64_t GgufTensor::rows() const noexcept {
  uint64_t n = dims.empty() ? 0 : 1;
  for (size_t i = 1; i < dims.size(); ++i) n *= dims[i];
  return n;
}

std::optional<uint64_t> GgufMetadata::unsignedValue(std::string_view key) const {
  const auto it = unsigneds.find(key);
  return it == unsigneds.end() ? std::nullopt : std::optional<uint64_t>(it->second);
}
std::optional<double> GgufMetadata::floatValue(std::string_view key) const {
  const auto it = floats.find(key);
  return it == floats.end() ? std::nullopt : std::optional<double>(it->second);
}
std::optional<std::string> GgufMetadata::stringValue(std::string_view key) const {
  const auto it = strings.find(key);
  return it == strings.end() ? std::nullopt : std::optional<std::string>(it->second);
}

GgufFile::GgufFile(const std::string &path) : GgufFile(std::vector<std::string>{path}) {}

GgufFile::GgufFile(const std::vector<std::string> &paths) {
  if (paths.empty()) throw GgufError("a GGUF has at least one file");
  try {
    for (size_t file = 0; file < paths.size(); ++file) parse(paths[file], uint32_t(file));
    if (metadata_.unsignedValue("split.count").value_or(1) != parts_.size())
      throw GgufError("the GGUF's split.count does not match its " + std::to_string(parts_.size()) + " file(s)");
    if (metadata_.unsignedValue("split.tensors.count").value_or(tensors_.size()) != tensors_.size())
      throw GgufError("the GGUF's files hold another number of tensors than split.tensors.count");
  } catch (...) {
    unmap();
    throw;
  }
}

void GgufFile::parse(const std::string &path, uint32_t file) {
  const int fd = ::open(path.c_str(), O_RDONLY);
  if (fd < 0) throw GgufError("cannot open " + path);
  struct stat st {};
  if (::fstat(fd, &st) != 0 || st.st_size < 24) {
    ::close(fd);
    throw GgufError("not a GGUF file: " + path);
  }
  Part part;
  part.size = uint64_t(st.st_size);
  void *mapped = ::mmap(nullptr, part.size, PROT_READ, MAP_PRIVATE, fd, 0);
  ::close(fd);
  if (mapped == MAP_FAILED) throw GgufError("cannot map " + path);
  part.base = static_cast<const uint8_t *>(mapped);
  parts_.push_back(part);   // unmapped with the others if the header is refused
  Reader r{part.base, part.size};
  if (r.take<uint32_t>() != 0x46554747u) throw GgufError("not a GGUF file: " + path);  // "GGUF"
  const uint32_t version = r.take<uint32_t>();
  if (version != 3) throw GgufError("unsupported GGUF version " + std::to_string(version));
  const uint64_t tensorCount = r.take<uint64_t>(), valueCount = r.take<uint64_t>();
  if (tensorCount > 16384 || valueCount > 16384) throw GgufError("implausible GGUF header counts");
  // Only the first part's metadata is kept: a later part repeats split.* alone, whose split.no must be its place.
  GgufMetadata later;
  GgufMetadata &metadata = file ? later : metadata_;
  std::set<std::string, std::less<>> keys;   // a key holds one value (GgufFile.cpp:191-194 of the reference)
  for (uint64_t i = 0; i < valueCount; ++i) {
    const std::string key = r.string();
    if (!keys.insert(key).second) throw GgufError("duplicate GGUF metadata key: " + key);
    const uint32_t type = r.take<uint32_t>();
    if (file && key == "split.no" && type != kU16 && type != kU32) throw GgufError("invalid split.no in " + path);
    switch (type) {
      case kU8: metadata.unsigneds[key] = r.take<uint8_t>(); break;
      case kI8: metadata.unsigneds[key] = uint64_t(int64_t(r.take<int8_t>())); break;
      case kU16: metadata.unsigneds[key] = r.take<uint16_t>(); break;
      case kI16: metadata.unsigneds[key] = uint64_t(int64_t(r.take<int16_t>())); break;
      case kU32: metadata.unsigneds[key] = r.take<uint32_t>(); break;
      case kI32: metadata.unsigneds[key] = uint64_t(int64_t(r.take<int32_t>())); break;
      case kBool: metadata.unsigneds[key] = r.take<uint8_t>() != 0; break;
      case kU64: metadata.unsigneds[key] = r.take<uint64_t>(); break;
      case kI64: metadata.unsigneds[key] = uint64_t(r.take<int64_t>()); break;
      case kF32: metadata.floats[key] = r.take<float>(); break;
      case kF64: metadata.floats[key] = r.take<double>(); break;
      case kString: metadata.strings[key] = r.string(); break;
      default: r.skipValue(type); break;  // arrays (tokenizer tables) are not kept
    }
  }
  if (file && later.unsignedValue("split.no").value_or(file) != file) throw GgufError("GGUF split file " + path + " is out of order");
  // the first part's alignment holds for every part: a later part's metadata is read for its split.no alone
  const uint64_t alignment = metadata_.unsignedValue("general.alignment").value_or(32);
  if (alignment < 8 || alignment > 65536 || (alignment & (alignment - 1))) throw GgufError("invalid GGUF alignment");
  const size_t firstTensor = tensors_.size();
  tensors_.reserve(firstTensor + tensorCount);
  for (uint64_t i = 0; i < tensorCount; ++i) {
    GgufTensor t;
    t.name = r.string();
    t.file = file;
    const uint32_t dimensions = r.take<uint32_t>();
    if (!dimensions || dimensions > 4) throw GgufError("tensor has an unsupported rank: " + t.name);
    for (uint32_t d = 0; d < dimensions; ++d) t.dims.push_back(r.take<uint64_t>());
    t.type = r.take<uint32_t>();
    t.offset = r.take<uint64_t>();
    const GgmlTypeTraits *traits = ggmlTypeTraits(t.type);
    if (!traits) throw GgufError("tensor " + t.name + " has unknown ggml type " + std::to_string(t.type));
    if (!t.columns() || t.columns() % traits->blockElements) throw GgufError("tensor rows do not hold whole blocks: " + t.name);
    if (t.rows() && t.columns() / traits->blockElements > UINT64_MAX / traits->blockBytes / t.rows())
      throw GgufError("tensor is too large: " + t.name);
    t.bytes = t.columns() / traits->blockElements * traits->blockBytes * t.rows();
    if (t.offset % alignment) throw GgufError("tensor data is misaligned: " + t.name);
    if (!index_.emplace(t.name, tensors_.size()).second) throw GgufError("duplicate tensor " + t.name);
    tensors_.push_back(std::move(t));
  }
  Part &mine = parts_.back();
  mine.dataStart = (r.at + alignment - 1) / alignment * alignment;
  for (size_t i = firstTensor; i < tensors_.size(); ++i) {
    const GgufTensor &t = tensors_[i];
    if (mine.dataStart > mine.size || t.offset > mine.size - mine.dataStart || t.bytes > mine.size - mine.dataStart - t.offset)
      throw GgufError("tensor data lies past the end of the file: " + t.name);
  }
}

void GgufFile::unmap() noexcept {
  for (const Part &part : parts_)
    if (part.base) ::munmap(const_cast<uint8_t *>(part.base), part.size);
  parts_.clear();
}

GgufFile::~GgufFile() { unmap(); }

const GgufTensor *GgufFile::find(std::string_view name) const noexcept {
  const auto it = index_.find(name);
  return it == index_.end() ? nullptr : &tensors_[it->second];
}
const GgufTensor &GgufFile::require(std::string_view name) const {
  if (const GgufTensor *t = find(name)) return *t;
  throw GgufError("missing tensor " + std::string(name));
}
const uint8_t *GgufFile::data(const GgufTensor &tensor) const {
  const Part &part = parts_.at(tensor.file);
  return part.base + part.dataStart + tensor.offset;
}

LoadedImage loadImage(hip::Backend &backend, const GgufFile &file, const GgufTensor &tensor, uint32_t firstRow, uint32_t rows) {
  const std::optional<uint32_t> format = imageFormat(tensor.type);
  if (!format) throw std::invalid_argument("tensor " + tensor.name + " is not of a projection format");
  if (tensor.dims.size() != 2) throw std::invalid_argument("a projection tensor has two dimensions: " + tensor.name);
  const uint64_t all = tensor.rows(), columns = tensor.columns();
  if (!rows) rows = uint32_t(all - std::min<uint64_t>(all, firstRow));
  if (!rows || uint64_t{firstRow} + rows > all || rows % GGUF_TILE_COLUMNS || firstRow % GGUF_TILE_COLUMNS || columns % GGUF_BLOCK ||
      columns > UINT32_MAX)
    throw std::invalid_argument("a weight image holds whole 16-row tiles of whole 256-input super-blocks: " + tensor.name);
  std::vector<uint8_t> rewritten;
  const uint8_t *native;
  if (const ops::NativeRewrite *rewrite = ops::nativeRewriteOf(tensor.type)) {
    const uint64_t blocks = columns / GGUF_BLOCK * rows;
    rewritten.resize(blocks * gguf_native_bytes(*format));
    ops::rewriteNative(tensor.type, file.data(tensor) + uint64_t{firstRow} * (columns / GGUF_BLOCK * rewrite->sourceBytes), blocks, rewritten.data());
    native = rewritten.data();
  } else {
    native = file.data(tensor) + uint64_t{firstRow} * (columns / GGUF_BLOCK * gguf_native_bytes(*format));
  }
  std::vector<uint8_t> image(gguf_image_bytes(*format, rows, uint32_t(columns)));
  ops::packGgufImage(*format, native, rows, uint32_t(columns), image.data());
  LoadedImage out;
  out.formatId = *format;
  out.rows = rows;
  out.inputSize = uint32_t(columns);
  out.image = backend.allocateBuffer(image.size(), hip::BufferStorage::Private, tensor.name.c_str());
  out.image.upload(image.data(), image.size());
  return out;
}

hip::Buffer loadNativeRows(hip::Backend &backend, const GgufFile &file, const GgufTensor &tensor, const char *label) {
  const ops::NativeRewrite *rewrite = ops::nativeRewriteOf(tensor.type);
  if (!rewrite) {
    hip::Buffer rows = backend.allocateBuffer(tensor.bytes, hip::BufferStorage::Private, label);
    rows.upload(file.data(tensor), tensor.bytes);
    return rows;
  }
  const uint64_t blocks = tensor.bytes / rewrite->sourceBytes;
  std::vector<uint8_t> rewritten(blocks * gguf_native_bytes(rewrite->imageFormat));
  ops::rewriteNative(tensor.type, file.data(tensor), blocks, rewritten.data());
  hip::Buffer rows = backend.allocateBuffer(rewritten.size(), hip::BufferStorage::Private, label);
  rows.upload(rewritten.data(), rewritten.size());
  return rows;
}

RowRuns groupedHeadRows(uint64_t rows, uint64_t from, uint32_t headRows, uint32_t keyHeads, uint32_t valueHeadsPerKey) {
  if (!headRows || !keyHeads || !valueHeadsPerKey || from > rows || (rows - from) != uint64_t{keyHeads} * valueHeadsPerKey * headRows)
    throw std::invalid_argument("the rows past `from` are the value heads' rows");
  RowRuns runs;
  if (from) runs.push_back({0, from});
  for (uint32_t h = 0; h < keyHeads; ++h)
    for (uint32_t j = 0; j < valueHeadsPerKey; ++j) runs.push_back({from + (uint64_t{j} * keyHeads + h) * headRows, headRows});
  return runs;
}

namespace {
uint64_t runRows(const RowRuns &runs, uint64_t all) {
  if (runs.empty()) return all;
  uint64_t rows = 0;
  for (const RowRun &run : runs) {
    if (!run.rows || run.first > all || run.rows > all - run.first) throw std::invalid_argument("a run of rows lies past the tensor");
    rows += run.rows;
  }
  return rows;
}
// The native rows of `runs`, columns [firstColumn, firstColumn + columns) of each, one after the other.
std::vector<uint8_t> gatherNative(const GgufFile &file, const GgufTensor &tensor, uint32_t format, const RowRuns &runs, uint64_t firstColumn,
                                  uint64_t columns) {
  const uint64_t all = tensor.rows(), width = tensor.columns();
  const ops::NativeRewrite *rewrite = ops::nativeRewriteOf(tensor.type);
  const uint64_t blockBytes = rewrite ? rewrite->sourceBytes : gguf_native_bytes(format), rowBytes = width / GGUF_BLOCK * blockBytes;
  const uint64_t piece = columns / GGUF_BLOCK * blockBytes, skip = firstColumn / GGUF_BLOCK * blockBytes;
  std::vector<uint8_t> native(runRows(runs, all) * piece);
  const uint8_t *data = file.data(tensor);
  uint64_t at = 0;
  auto take = [&](uint64_t first, uint64_t rows) {
    for (uint64_t r = 0; r < rows; ++r, at += piece) std::memcpy(native.data() + at, data + (first + r) * rowBytes + skip, piece);
  };
  if (runs.empty()) take(0, all);
  for (const RowRun &run : runs) take(run.first, run.rows);
  if (rewrite) {
    std::vector<uint8_t> rewritten(native.size() / rewrite->sourceBytes * gguf_native_bytes(format));
    ops::rewriteNative(tensor.type, native.data(), native.size() / rewrite->sourceBytes, rewritten.data());
    return rewritten;
  }
  return native;
}
} // namespace

PackedImages packImagesOfRows(const GgufFile &file, const GgufTensor &tensor, const std::vector<RowRuns> &images, uint64_t firstColumn,
                              uint64_t columns) {
  const std::optional<uint32_t> format = imageFormat(tensor.type);
  if (!format) throw std::invalid_argument("tensor " + tensor.name + " is not of a projection format");
  if (images.empty()) throw std::invalid_argument("no rows to load of " + tensor.name);
  const uint64_t width = tensor.columns();
  if (!columns) columns = width - std::min(width, firstColumn);
  if (!columns || firstColumn % GGUF_BLOCK || columns % GGUF_BLOCK || firstColumn + columns > width || columns > UINT32_MAX)
    throw std::invalid_argument("a weight image holds whole 256-input super-blocks: " + tensor.name);
  const uint64_t rows = runRows(images.front(), tensor.rows());
  if (!rows || rows % GGUF_TILE_COLUMNS || rows > UINT32_MAX) throw std::invalid_argument("a weight image holds whole 16-row tiles: " + tensor.name);
  const uint64_t imageBytes = gguf_image_bytes(*format, uint32_t(rows), uint32_t(columns));
  std::vector<uint8_t> packed(imageBytes * images.size());
  for (size_t i = 0; i < images.size(); ++i) {
    if (runRows(images[i], tensor.rows()) != rows) throw std::invalid_argument("the images of " + tensor.name + " hold the same rows each");
    const std::vector<uint8_t> native = gatherNative(file, tensor, *format, images[i], firstColumn, columns);
    ops::packGgufImage(*format, native.data(), uint32_t(rows), uint32_t(columns), packed.data() + i * imageBytes);
  }
  return {*format, uint32_t(rows), uint32_t(columns), std::move(packed)};
}

LoadedImage loadImagesOfRows(hip::Backend &backend, const GgufFile &file, const GgufTensor &tensor, const std::vector<RowRuns> &images,
                             uint64_t firstColumn, uint64_t columns) {
  const PackedImages packed = packImagesOfRows(file, tensor, images, firstColumn, columns);
  LoadedImage out;
  out.formatId = packed.formatId;
  out.rows = packed.rows;
  out.inputSize = packed.inputSize;
  out.image = backend.allocateBuffer(packed.bytes.size(), hip::BufferStorage::Private, tensor.name.c_str());
  out.image.upload(packed.bytes.data(), packed.bytes.size());
  return out;
}

LoadedImage loadImageRows(hip::Backend &backend, const GgufFile &file, const GgufTensor &tensor, const RowRuns &runs, uint64_t firstColumn,
                          uint64_t columns) {
  return loadImagesOfRows(backend, file, tensor, {runs}, firstColumn, columns);
}

namespace {
bool floatTensor(uint32_t type) { return type == ggml::kF32 || type == ggml::kF16 || type == ggml::kBF16; }
uint32_t elementBytes(uint32_t type) { return type == ggml::kF32 ? 4 : 2; }
float floatAt(const uint8_t *data, uint32_t type, uint64_t i) {
  if (type == ggml::kF32) {
    float f;
    std::memcpy(&f, data + 4 * i, 4);
    return f;
  }
  uint16_t h;
  std::memcpy(&h, data + 2 * i, 2);
  if (type == ggml::kF16) return halfToFloat(h);
  const uint32_t bits = uint32_t{h} << 16;
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}
// The fp32 values of `runs` of a float tensor.
std::vector<float> gatherFloats(const GgufFile &file, const GgufTensor &tensor, const RowRuns &runs) {
  if (!floatTensor(tensor.type)) throw std::invalid_argument("tensor " + tensor.name + " does not hold 16- or 32-bit floats");
  // a vector's runs are runs of its values
  const bool vector = tensor.dims.size() == 1;
  const uint64_t all = vector ? tensor.columns() : tensor.rows(), width = vector ? 1 : tensor.columns();
  std::vector<float> values;
  values.reserve(runRows(runs, all) * width);
  const uint8_t *data = file.data(tensor);
  auto take = [&](uint64_t first, uint64_t rows) {
    for (uint64_t i = first * width; i < (first + rows) * width; ++i) values.push_back(floatAt(data, tensor.type, i));
  };
  if (runs.empty()) take(0, all);
  for (const RowRun &run : runs) take(run.first, run.rows);
  return values;
}
} // namespace

LoadedFloatRows loadFloatRows(hip::Backend &backend, const GgufFile &file, const std::vector<const GgufTensor *> &tensors, const RowRuns &runs) {
  if (tensors.empty() || !tensors.front()) throw std::invalid_argument("no float rows to load");
  const uint64_t width = tensors.front()->columns();
  bool bfloat16 = true;
  for (const GgufTensor *t : tensors) {
    if (!t || !floatTensor(t->type) || t->columns() != width) throw std::invalid_argument("float rows of one width");
    bfloat16 = bfloat16 && t->type == ggml::kBF16;
  }
  LoadedFloatRows out;
  out.inputSize = uint32_t(width);
  out.bfloat16 = bfloat16;
  std::vector<uint8_t> bytes;
  for (const GgufTensor *t : tensors) {
    const std::vector<float> values = gatherFloats(file, *t, runs);
    out.outputSize += uint32_t(values.size() / width);
    for (float v : values) {
      if (bfloat16) {
        const uint16_t b = floatToBf16(v);  // exact: the value is a bf16's
        bytes.insert(bytes.end(), reinterpret_cast<const uint8_t *>(&b), reinterpret_cast<const uint8_t *>(&b) + 2);
      } else {
        bytes.insert(bytes.end(), reinterpret_cast<const uint8_t *>(&v), reinterpret_cast<const uint8_t *>(&v) + 4);
      }
    }
  }
  out.rows = backend.allocateBuffer(std::max<uint64_t>(bytes.size(), 16), hip::BufferStorage::Private, tensors.front()->name.c_str());
  out.rows.upload(bytes.data(), bytes.size());
  return out;
}

hip::Buffer loadFloat32Values(hip::Backend &backend, const GgufFile &file, const GgufTensor &tensor, const RowRuns &runs) {
  const std::vector<float> values = gatherFloats(file, tensor, runs);
  hip::Buffer out = backend.allocateBuffer(std::max<uint64_t>(values.size() * 4, 16), hip::BufferStorage::Private, tensor.name.c_str());
  out.upload(values.data(), values.size() * 4);
  return out;
}

hip::Buffer loadBf16Values(hip::Backend &backend, const GgufFile &file, const GgufTensor &tensor, const RowRuns &runs) {
  const std::vector<float> values = gatherFloats(file, tensor, runs);
  std::vector<uint16_t> bits(values.size());
  for (size_t i = 0; i < values.size(); ++i) bits[i] = floatToBf16(values[i]);
  hip::Buffer out = backend.allocateBuffer(std::max<uint64_t>(bits.size() * 2, 16), hip::BufferStorage::Private, tensor.name.c_str());
  out.upload(bits.data(), bits.size() * 2);
  return out;
}

hip::Buffer loadBf16Vector(hip::Backend &backend, const GgufFile &file, const GgufTensor &tensor) {
  if (tensor.type != ggml::kF32 && tensor.type != ggml::kF16 && tensor.type != ggml::kBF16)
    throw std::invalid_argument("tensor " + tensor.name + " is not a 16- or 32-bit float vector");
  const uint64_t n = tensor.elements();
  std::vector<uint16_t> bits(n);
  const uint8_t *data = file.data(tensor);
  for (uint64_t i = 0; i < n; ++i) {
    if (tensor.type == ggml::kBF16) std::memcpy(&bits[i], data + 2 * i, 2);
    else if (tensor.type == ggml::kF16) {
      uint16_t h;
      std::memcpy(&h, data + 2 * i, 2);
      bits[i] = floatToBf16(halfToFloat(h));
    } else {
      float f;
      std::memcpy(&f, data + 4 * i, 4);
      bits[i] = floatToBf16(f);
    }
  }
  hip::Buffer out = backend.allocateBuffer(std::max<uint64_t>(n * 2, 16), hip::BufferStorage::Private, tensor.name.c_str());
  out.upload(bits.data(), n * 2);
  return out;
}

} // namespace splash::model
