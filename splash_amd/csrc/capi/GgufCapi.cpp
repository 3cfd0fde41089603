// The C entry points of include/splash_gguf.h over model::GgufFile.
#include "splash_gguf.h"
#include "capi/Guard.hpp"
#include "capi/Handles.hpp"
#include "model/GgufFile.hpp"

#include <algorithm>
#include <cstring>
#include <memory>

using namespace splash;

struct spg_file {
  std::unique_ptr<model::GgufFile> file;
};

namespace splash::capi {
const model::GgufFile &ggufOf(const spg_file *file) {
  require(file, "file");
  return *file->file;
}
} // namespace splash::capi

namespace {
size_t copyOut(const std::string &text, char *out, size_t capacity) {
  if (out && capacity) {
    const size_t n = std::min(capacity - 1, text.size());
    std::memcpy(out, text.data(), n);
    out[n] = 0;
  }
  return text.size() + 1;
}
const model::GgufTensor &tensorOf(const spg_file *file, uint64_t index) {
  capi::require(file, "file");
  if (index >= file->file->tensors().size()) throw std::invalid_argument("no such tensor");
  return file->file->tensors()[index];
}
sp_buffer *handOver(const hip::Buffer &buffer) {
  sp_buffer_retain(buffer.handle());  // the caller's reference; the wrapper drops its own
  return buffer.handle();
}
} // namespace

extern "C" {

sp_status spg_open(const char *path, spg_file **out) {
  return capi::guard([&] {
    capi::require(path && out, "path or result");
    auto holder = std::make_unique<spg_file>();
    holder->file = std::make_unique<model::GgufFile>(path);
    *out = holder.release();
  });
}
sp_status spg_open_parts(const char *const *paths, uint32_t count, spg_file **out) {
  return capi::guard([&] {
    capi::require(paths && count && out, "paths or result");
    std::vector<std::string> parts;
    for (uint32_t i = 0; i < count; ++i) {
      capi::require(paths[i], "a part's path");
      parts.emplace_back(paths[i]);
    }
    auto holder = std::make_unique<spg_file>();
    holder->file = std::make_unique<model::GgufFile>(parts);
    *out = holder.release();
  });
}
void spg_close(spg_file *file) { delete file; }

int spg_metadata_unsigned(const spg_file *file, const char *key, uint64_t *value) {
  if (!file || !key) return 0;
  const auto v = file->file->metadata().unsignedValue(key);
  if (v && value) *value = *v;
  return v.has_value();
}
int spg_metadata_float(const spg_file *file, const char *key, double *value) {
  if (!file || !key) return 0;
  const auto v = file->file->metadata().floatValue(key);
  if (v && value) *value = *v;
  return v.has_value();
}
size_t spg_metadata_string(const spg_file *file, const char *key, char *out, size_t capacity) {
  if (!file || !key) return 0;
  const auto v = file->file->metadata().stringValue(key);
  return v ? copyOut(*v, out, capacity) : 0;
}

uint64_t spg_tensor_count(const spg_file *file) { return file ? file->file->tensors().size() : 0; }
size_t spg_tensor_name(const spg_file *file, uint64_t index, char *out, size_t capacity) {
  if (!file || index >= file->file->tensors().size()) return 0;
  return copyOut(file->file->tensors()[index].name, out, capacity);
}
sp_status spg_tensor_info(const spg_file *file, uint64_t index, spg_tensor *out) {
  return capi::guard([&] {
    capi::require(out, "result");
    const model::GgufTensor &t = tensorOf(file, index);
    *out = spg_tensor{};
    out->ggml_type = t.type;
    out->dimensions = uint32_t(t.dims.size());
    for (size_t d = 0; d < t.dims.size(); ++d) out->dims[d] = t.dims[d];
    out->bytes = t.bytes;
    out->format = model::imageFormat(t.type).value_or(0xFFFFFFFFu);
  });
}
int64_t spg_find(const spg_file *file, const char *name) {
  if (!file || !name) return -1;
  const model::GgufTensor *t = file->file->find(name);
  return t ? int64_t(t - file->file->tensors().data()) : -1;
}
const void *spg_tensor_data(const spg_file *file, uint64_t index) {
  if (!file || index >= file->file->tensors().size()) return nullptr;
  return file->file->data(file->file->tensors()[index]);
}

sp_status spg_load_image(sp_backend *backend, const spg_file *file, uint64_t index, uint32_t first_row, uint32_t rows,
                         sp_buffer **image, uint32_t *format, uint32_t *out_rows, uint32_t *input_size) {
  return capi::guard([&] {
    capi::require(backend && image && format && out_rows && input_size, "backend or results");
    hip::Backend borrowed(backend);
    const model::LoadedImage loaded = model::loadImage(borrowed, *file->file, tensorOf(file, index), first_row, rows);
    *image = handOver(loaded.image);
    *format = loaded.formatId;
    *out_rows = loaded.rows;
    *input_size = loaded.inputSize;
  });
}
sp_status spg_load_bf16(sp_backend *backend, const spg_file *file, uint64_t index, sp_buffer **out, uint64_t *elements) {
  return capi::guard([&] {
    capi::require(backend && out, "backend or result");
    hip::Backend borrowed(backend);
    const model::GgufTensor &t = tensorOf(file, index);
    *out = handOver(model::loadBf16Vector(borrowed, *file->file, t));
    if (elements) *elements = t.elements();
  });
}

} // extern "C"
