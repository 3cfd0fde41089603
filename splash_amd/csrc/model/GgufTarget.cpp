#include "model/GgufTarget.hpp"

#include <cmath>
#include <set>

namespace splash::model {
namespace {

uint32_t requireUnsigned(const GgufFile &file, const std::string &key) {
  const std::optional<uint64_t> value = file.metadata().unsignedValue(key);
  if (!value || !*value || *value > UINT32_MAX) throw GgufError("GGUF metadata lacks " + key);
  return uint32_t(*value);
}
std::string architectureOf(const GgufFile &file) {
  const std::optional<std::string> name = file.metadata().stringValue("general.architecture");
  if (!name || name->empty()) throw GgufError("GGUF metadata lacks general.architecture");
  return *name;
}
std::string prefix(uint32_t layer) { return "blk." + std::to_string(layer) + "."; }

// Collects what the file lacks or the path does not read, so that one error names all of it.
struct Problems {
  std::string text;
  void add(const std::string &problem) { text += (text.empty() ? "" : "; ") + problem; }
};

struct Loader {
  hip::Backend &backend;
  const GgufFile &file;
  Problems &problems;
  std::set<std::string> read;

  const GgufTensor *tensor(const std::string &name, uint64_t rows, uint64_t columns) {
    read.insert(name);
    const GgufTensor *t = file.find(name);
    if (!t) {
      problems.add(name + " is missing");
      return nullptr;
    }
    if (t->dims.empty() || t->dims[0] != columns || t->rows() != rows) {
      problems.add(name + " is not " + std::to_string(rows) + " x " + std::to_string(columns));
      return nullptr;
    }
    return t;
  }
  // A projection tensor as one segment of a projection, `offset` output columns in.
  std::optional<ops::QuantizedSegment> segment(const std::string &name, uint32_t rows, uint32_t columns, uint32_t offset = 0) {
    const GgufTensor *t = tensor(name, rows, columns);
    if (!t) return std::nullopt;
    if (!imageFormat(t->type)) {
      problems.add(name + " is of a type the projections do not read");
      return std::nullopt;
    }
    LoadedImage image = loadImage(backend, file, *t);
    return ops::QuantizedSegment::ofImage(image.formatId, rows, columns, std::move(image.image), offset);
  }
  ops::Projection projection(const std::string &name, uint32_t rows, uint32_t columns) {
    std::optional<ops::QuantizedSegment> s = segment(name, rows, columns);
    return s ? ops::Projection(rows, columns, ops::BlockWeights{{std::move(*s)}}) : ops::Projection{};
  }
  hip::Buffer norm(const std::string &name, uint32_t size) {
    const GgufTensor *t = tensor(name, 1, size);
    if (!t) return {};
    if (t->type != ggml::kF32 && t->type != ggml::kF16 && t->type != ggml::kBF16) {
      problems.add(name + " is not a float vector");
      return {};
    }
    return loadBf16Vector(backend, file, *t);
  }
};

} // namespace

// The architectures whose dense decoder tensors, head geometry and RoPE pairing (dimension i with i + pairs, GGML's
// "neox" rotation) these kernels compute: the Qwen families the reference targets (requireMetadata,
// runtime/model/GgufImage.cpp:874-916, takes its model's own architecture and nothing else). A llama-architecture
// file permutes its query and key rows for the interleaved rotation: it would load and give wrong logits.
bool denseArchitecture(const std::string &name) {
  static const std::set<std::string> known = {"qwen2", "qwen3", "qwen35"};
  return known.count(name) != 0;
}

DenseDimensions ggufDenseDimensions(const GgufFile &file) {
  const std::string name = architectureOf(file);
  if (!denseArchitecture(name))
    throw GgufError("GGUF architecture " + name + " is not one the dense driver computes (qwen2, qwen3, qwen35)");
  const std::string a = name + ".";
  // What the metadata names and the kernels do not do, collected so that one error names all of it.
  Problems problems;
  DenseDimensions d;
  d.layers = requireUnsigned(file, a + "block_count");
  d.hidden = requireUnsigned(file, a + "embedding_length");
  d.ffn = requireUnsigned(file, a + "feed_forward_length");
  d.qHeads = requireUnsigned(file, a + "attention.head_count");
  d.kvHeads = requireUnsigned(file, a + "attention.head_count_kv");
  const std::optional<uint64_t> keyLength = file.metadata().unsignedValue(a + "attention.key_length");
  d.headDimension = keyLength ? uint32_t(*keyLength) : d.hidden / d.qHeads;
  const std::optional<uint64_t> valueLength = file.metadata().unsignedValue(a + "attention.value_length");
  if (valueLength && *valueLength != d.headDimension) problems.add("keys and values of different lengths are not supported");
  const std::optional<uint64_t> rotary = file.metadata().unsignedValue(a + "rope.dimension_count");
  if (rotary && *rotary != d.headDimension) problems.add("a partial rotary embedding is not supported by the dense driver");
  d.rotaryPairs = d.headDimension / 2;
  const std::optional<double> base = file.metadata().floatValue(a + "rope.freq_base");
  if (!base || !(*base > 0)) problems.add("GGUF metadata lacks " + a + "rope.freq_base");
  d.ropeTheta = float(base.value_or(0.0));
  if (const std::optional<std::string> scaling = file.metadata().stringValue(a + "rope.scaling.type"); scaling && *scaling != "none")
    problems.add("rope.scaling.type " + *scaling + " is not computed (expected none)");
  const double epsilon = file.metadata().floatValue(a + "attention.layer_norm_rms_epsilon").value_or(1e-6);
  if (std::fabs(epsilon - 1e-6) > 1e-12) problems.add("the norms' epsilon is 1e-6 in these kernels; the file names another");
  if (!problems.text.empty()) throw GgufError("GGUF metadata this build cannot follow: " + problems.text);
  const GgufTensor &table = file.require("token_embd.weight");
  if (table.dims.size() != 2 || table.dims[0] != d.hidden) throw GgufError("token_embd.weight is not vocabulary x hidden");
  d.vocabulary = uint32_t(table.dims[1]);
  // Per-head query and key norms when the file holds them (Qwen3), none otherwise.
  d.normalizeHeads = file.find("blk.0.attn_q_norm.weight") != nullptr;
  return d;
}

void loadGgufDenseWeights(hip::Backend &backend, const GgufFile &file, DenseVerify &verify) {
  const DenseDimensions &d = verify.dimensions();
  Problems problems;
  Loader load{backend, file, problems, {}};
  DenseWeights &w = verify.weights();
  const uint32_t D = d.headDimension, kvWidth = d.kvHeads * D, qWidth = d.qHeads * D;
  for (uint32_t layer = 0; layer < d.layers; ++layer) {
    const std::string p = prefix(layer);
    DenseLayer out;
    out.inputNorm = load.norm(p + "attn_norm.weight", d.hidden);
    std::vector<ops::QuantizedSegment> qkv;
    const std::pair<const char *, uint32_t> parts[3] = {{"attn_q.weight", qWidth}, {"attn_k.weight", kvWidth}, {"attn_v.weight", kvWidth}};
    uint32_t offset = 0;
    for (const auto &[name, rows] : parts) {
      std::optional<ops::QuantizedSegment> s = load.segment(p + name, rows, d.hidden, offset);
      if (s) qkv.push_back(std::move(*s));
      offset += rows;
    }
    if (qkv.size() == 3) out.qkv = ops::Projection(d.qkvWidth(), d.hidden, ops::BlockWeights{std::move(qkv)});
    if (d.normalizeHeads) {
      out.queryNorm = load.norm(p + "attn_q_norm.weight", D);
      out.keyNorm = load.norm(p + "attn_k_norm.weight", D);
    }
    out.output = load.projection(p + "attn_output.weight", d.hidden, qWidth);
    out.postNorm = load.norm(p + "ffn_norm.weight", d.hidden);
    out.gate = load.projection(p + "ffn_gate.weight", d.ffn, d.hidden);
    out.up = load.projection(p + "ffn_up.weight", d.ffn, d.hidden);
    out.down = load.projection(p + "ffn_down.weight", d.hidden, d.ffn);
    w.layers.at(layer) = std::move(out);
  }
  w.finalNorm = load.norm("output_norm.weight", d.hidden);
  // The token table stays in its native rows (the gather decodes them); a tied head reads the same tensor as an image.
  const GgufTensor *table = load.tensor("token_embd.weight", d.vocabulary, d.hidden);
  if (table) {
    const std::optional<uint32_t> format = imageFormat(table->type);
    if (!format) problems.add("token_embd.weight is of a type the token gather does not read");
    else {
      hip::Buffer rows = backend.allocateBuffer(table->bytes, hip::BufferStorage::Private, "token table");
      rows.upload(file.data(*table), table->bytes);
      w.embedding = {std::move(rows), *format, d.vocabulary, d.hidden};
    }
  }
  w.head = load.projection(file.find("output.weight") ? "output.weight" : "token_embd.weight", d.vocabulary, d.hidden);
  w.head.destination = ops::FloatOutput::Float32;
  // What the file holds beside: rope_freqs (long-context factors) and biases would change the result if ignored.
  for (const GgufTensor &t : file.tensors())
    if (!load.read.count(t.name)) problems.add(t.name + " is not read by the dense driver");
  if (!problems.text.empty()) throw GgufError("GGUF tensors this build cannot load: " + problems.text);
}

} // namespace splash::model
