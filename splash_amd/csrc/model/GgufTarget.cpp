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
      hip::Buffer rows = loadNativeRows(backend, file, *table, "token table");
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

namespace {
bool floatType(uint32_t type) { return type == ggml::kF32 || type == ggml::kF16 || type == ggml::kBF16; }
uint64_t optionalUnsigned(const GgufFile &file, const std::string &key, uint64_t otherwise = 0) {
  return file.metadata().unsignedValue(key).value_or(otherwise);
}
// Whether `name` is a tensor of a block blk.N. with N >= first (the multi-token prediction blocks after the target's).
bool inLaterBlocks(const std::string &name, uint32_t first) {
  if (name.rfind("blk.", 0) != 0) return false;
  const size_t dot = name.find('.', 4);
  if (dot == std::string::npos) return false;
  try {
    return std::stoul(name.substr(4, dot - 4)) >= first;
  } catch (...) {
    return false;
  }
}
} // namespace

HybridDimensions ggufHybridDimensions(const GgufFile &file) {
  const std::string name = architectureOf(file);
  if (name != "qwen35" && name != "qwen35moe")
    throw GgufError("GGUF architecture " + name + " is not one the hybrid driver computes (qwen35, qwen35moe)");
  const std::string a = name + ".";
  Problems problems;
  HybridDimensions d;
  const uint32_t blocks = requireUnsigned(file, a + "block_count");
  const uint64_t extra = optionalUnsigned(file, a + "nextn_predict_layers");
  if (extra >= blocks) throw GgufError("GGUF metadata names no layer before its prediction blocks");
  d.layers = blocks - uint32_t(extra);
  d.hidden = requireUnsigned(file, a + "embedding_length");
  d.qHeads = requireUnsigned(file, a + "attention.head_count");
  d.kvHeads = requireUnsigned(file, a + "attention.head_count_kv");
  d.headDimension = requireUnsigned(file, a + "attention.key_length");
  if (optionalUnsigned(file, a + "attention.value_length", d.headDimension) != d.headDimension)
    problems.add("keys and values of different lengths are not supported");
  const uint64_t rotary = optionalUnsigned(file, a + "rope.dimension_count", d.headDimension);
  if (!rotary || rotary % 2 || rotary > d.headDimension) problems.add("rope.dimension_count is not an even part of a head");
  d.rotaryPairs = uint32_t(rotary / 2);
  const std::optional<double> base = file.metadata().floatValue(a + "rope.freq_base");
  if (!base || !(*base > 0)) problems.add("GGUF metadata lacks " + a + "rope.freq_base");
  d.ropeTheta = float(base.value_or(0.0));
  if (const std::optional<std::string> scaling = file.metadata().stringValue(a + "rope.scaling.type"); scaling && *scaling != "none")
    problems.add("rope.scaling.type " + *scaling + " is not computed (expected none)");
  const double epsilon = file.metadata().floatValue(a + "attention.layer_norm_rms_epsilon").value_or(1e-6);
  if (std::fabs(epsilon - 1e-6) > 1e-12) problems.add("the norms' epsilon is 1e-6 in these kernels; the file names another");
  d.attentionInterval = requireUnsigned(file, a + "full_attention_interval");
  d.gdnKeyHeads = requireUnsigned(file, a + "ssm.group_count");
  d.gdnValueHeads = requireUnsigned(file, a + "ssm.time_step_rank");
  if (requireUnsigned(file, a + "ssm.state_size") != GDN_HEAD_DIMENSION) problems.add("ssm.state_size is 128 in these kernels");
  if (requireUnsigned(file, a + "ssm.conv_kernel") != GDN_CONVOLUTION_TAPS) problems.add("ssm.conv_kernel is 4 in these kernels");
  if (requireUnsigned(file, a + "ssm.inner_size") != uint64_t{d.gdnValueHeads} * GDN_HEAD_DIMENSION)
    problems.add("ssm.inner_size is not ssm.time_step_rank heads of 128");
  if (d.gdnKeyHeads && d.gdnValueHeads % d.gdnKeyHeads) problems.add("the value heads are not whole groups of the key heads");
  const uint32_t packed = (2 * d.gdnKeyHeads + 2 * d.gdnValueHeads) * GDN_HEAD_DIMENSION + 2 * d.gdnValueHeads;
  d.gdnPackedWidth = (packed + GGUF_TILE_COLUMNS * 4 - 1) / (GGUF_TILE_COLUMNS * 4) * (GGUF_TILE_COLUMNS * 4);  // whole 64-column groups
  d.experts = uint32_t(optionalUnsigned(file, a + "expert_count"));
  if (d.experts) {
    d.topK = requireUnsigned(file, a + "expert_used_count");
    d.expertFfn = requireUnsigned(file, a + "expert_feed_forward_length");
    const uint64_t shared = optionalUnsigned(file, a + "expert_shared_feed_forward_length");
    if (shared % d.expertFfn) problems.add("the shared expert is not whole slices of the routed experts' width");
    d.sharedSlices = uint32_t(shared / d.expertFfn);
    d.sharedGate = file.find("blk.0.ffn_gate_inp_shexp.weight") != nullptr;
  } else {
    d.denseFfn = requireUnsigned(file, a + "feed_forward_length");
  }
  if (!problems.text.empty()) throw GgufError("GGUF metadata this build cannot follow: " + problems.text);
  const GgufTensor &table = file.require("token_embd.weight");
  if (table.dims.size() != 2 || table.dims[0] != d.hidden) throw GgufError("token_embd.weight is not vocabulary x hidden");
  d.vocabulary = uint32_t(table.dims[1]);
  // The first attention layer tells what every attention layer holds: head norms, and queries with their gates.
  const std::string first = prefix(d.attentionInterval - 1);
  d.normalizeHeads = file.find(first + "attn_q_norm.weight") != nullptr;
  if (const GgufTensor *q = file.find(first + "attn_q.weight"))
    d.gatedAttention = q->rows() == 2ull * d.qHeads * d.headDimension;
  return d;
}

void loadGgufHybridWeights(hip::Backend &backend, const GgufFile &file, HybridVerify &verify) {
  const HybridDimensions &d = verify.dimensions();
  Problems problems;
  Loader load{backend, file, problems, {}};
  HybridWeights &w = verify.weights();
  const uint32_t D = d.headDimension, H = d.hidden, KH = d.gdnKeyHeads, VH = d.gdnValueHeads, perKey = KH ? VH / KH : 0;
  const uint32_t keyRows = 2 * KH * GDN_HEAD_DIMENSION, valueRows = VH * GDN_HEAD_DIMENSION, convolution = keyRows + valueRows;
  // a float tensor of `rows` x `columns` (a vector: columns values), or nullptr with the problem noted
  auto floats = [&](const std::string &name, uint64_t rows, uint64_t columns) -> const GgufTensor * {
    load.read.insert(name);
    const GgufTensor *t = file.find(name);
    if (!t) {
      problems.add(name + " is missing");
      return nullptr;
    }
    if (!floatType(t->type)) {
      problems.add(name + " is not of 16- or 32-bit floats");
      return nullptr;
    }
    if (t->elements() != rows * columns || t->columns() != columns) {
      problems.add(name + " is not " + std::to_string(rows) + " x " + std::to_string(columns));
      return nullptr;
    }
    return t;
  };
  // a projection tensor (any rank) of `rows` rows of `columns` inputs of an image format
  auto quantized = [&](const std::string &name, uint64_t rows, uint64_t columns) -> const GgufTensor * {
    load.read.insert(name);
    const GgufTensor *t = file.find(name);
    if (!t) {
      problems.add(name + " is missing");
      return nullptr;
    }
    if (t->rows() != rows || t->columns() != columns) {
      problems.add(name + " is not " + std::to_string(rows) + " x " + std::to_string(columns));
      return nullptr;
    }
    if (!imageFormat(t->type)) {
      problems.add(name + " is of a type the projections do not read");
      return nullptr;
    }
    return t;
  };
  auto segmentOf = [&](const GgufTensor &t, const RowRuns &runs, uint32_t rows, uint32_t offset) {
    LoadedImage image = loadImageRows(backend, file, t, runs);
    return ops::QuantizedSegment::ofImage(image.formatId, rows, uint32_t(t.columns()), std::move(image.image), offset);
  };
  for (uint32_t layer = 0; layer < d.layers; ++layer) {
    const std::string p = prefix(layer);
    HybridLayer out;
    out.inputNorm = load.norm(p + "attn_norm.weight", H);
    out.postNorm = load.norm(p + "post_attention_norm.weight", H);
    if (d.attends(layer)) {
      const uint32_t qRows = (d.gatedAttention ? 2 : 1) * d.qHeads * D, kvRows = d.kvHeads * D;
      std::vector<ops::QuantizedSegment> qkv;
      const std::pair<const char *, uint32_t> parts[3] = {{"attn_q.weight", qRows}, {"attn_k.weight", kvRows}, {"attn_v.weight", kvRows}};
      uint32_t offset = 0;
      for (const auto &[name, rows] : parts) {
        if (std::optional<ops::QuantizedSegment> s = load.segment(p + name, rows, H, offset)) qkv.push_back(std::move(*s));
        offset += rows;
      }
      if (qkv.size() == 3) out.mixerInput = ops::Projection(d.qkvWidth(), H, ops::BlockWeights{std::move(qkv)});
      if (d.normalizeHeads) {
        out.queryNorm = load.norm(p + "attn_q_norm.weight", D);
        out.keyNorm = load.norm(p + "attn_k_norm.weight", D);
      }
      out.mixerOutput = load.projection(p + "attn_output.weight", H, d.qHeads * D);
    } else {
      // q | k | v: the value heads' rows regrouped by key head; z likewise; beta | alpha as rows of floats
      const GgufTensor *qkv = quantized(p + "attn_qkv.weight", convolution, H), *z = quantized(p + "attn_gate.weight", valueRows, H);
      if (qkv && z) {
        std::vector<ops::QuantizedSegment> segments;
        segments.push_back(segmentOf(*qkv, groupedHeadRows(convolution, keyRows, GDN_HEAD_DIMENSION, KH, perKey), convolution, 0));
        segments.push_back(segmentOf(*z, groupedHeadRows(valueRows, 0, GDN_HEAD_DIMENSION, KH, perKey), valueRows, convolution));
        out.mixerInput = ops::Projection(d.gdnPackedWidth, H, ops::BlockWeights{std::move(segments)});
      }
      const GgufTensor *beta = floats(p + "ssm_beta.weight", VH, H), *alpha = floats(p + "ssm_alpha.weight", VH, H);
      if (beta && alpha) {
        LoadedFloatRows rows = loadFloatRows(backend, file, {beta, alpha}, groupedHeadRows(VH, 0, 1, KH, perKey));
        out.gateRows = {std::move(rows.rows), rows.outputSize, rows.inputSize, rows.bfloat16};
      }
      if (const GgufTensor *t = floats(p + "ssm_conv1d.weight", convolution, GDN_CONVOLUTION_TAPS))
        out.convolutionWeights = loadBf16Values(backend, file, *t, groupedHeadRows(convolution, keyRows, GDN_HEAD_DIMENSION, KH, perKey));
      if (const GgufTensor *t = floats(p + "ssm_a", 1, VH)) out.decay = loadFloat32Values(backend, file, *t, groupedHeadRows(VH, 0, 1, KH, perKey));
      if (const GgufTensor *t = floats(p + "ssm_dt.bias", 1, VH)) out.timeBias = loadBf16Values(backend, file, *t, groupedHeadRows(VH, 0, 1, KH, perKey));
      if (const GgufTensor *t = floats(p + "ssm_norm.weight", 1, GDN_HEAD_DIMENSION)) {
        out.mixerNorm = loadFloat32Values(backend, file, *t);   // read unrounded, as the reference reads a GGUF's norms
        out.mixerNormFloat = true;
      }
      out.mixerOutput = load.projection(p + "ssm_out.weight", H, valueRows);
    }
    if (d.dense()) {
      out.ffnGate = load.projection(p + "ffn_gate.weight", d.denseFfn, H);
      out.ffnUp = load.projection(p + "ffn_up.weight", d.denseFfn, H);
      out.ffnDown = load.projection(p + "ffn_down.weight", H, d.denseFfn);
    } else {
      const uint32_t E = d.experts, F = d.expertFfn, S = d.sharedSlices;
      if (const GgufTensor *t = floats(p + "ffn_gate_inp.weight", E, H)) {
        LoadedFloatRows rows = loadFloatRows(backend, file, {t});
        out.routerRows = {std::move(rows.rows), rows.outputSize, rows.inputSize, rows.bfloat16};
      }
      // an expert's rows an image; the shared slices' images after the routed experts'
      auto expertRuns = [&](uint64_t experts, uint64_t rows, uint64_t stride, uint64_t first) {
        std::vector<RowRuns> images;
        for (uint64_t e = 0; e < experts; ++e) images.push_back({{first + e * stride, rows}});
        return images;
      };
      struct Side {
        PackedImages routed, shared;
        bool whole = false;
      };
      auto upload = [&](Side &side, const char *label) -> hip::Buffer {
        if (!side.whole) return {};
        std::vector<uint8_t> &bytes = side.routed.bytes;
        bytes.insert(bytes.end(), side.shared.bytes.begin(), side.shared.bytes.end());
        hip::Buffer buffer = backend.allocateBuffer(bytes.size(), hip::BufferStorage::Private, label);
        buffer.upload(bytes.data(), bytes.size());
        return buffer;
      };
      Side gate, up, down;
      const std::string fused = p + "ffn_gate_up_exps.weight";
      if (file.find(fused)) {
        // expert e's gate rows are rows 2 e F .. of the fused tensor, its up rows the next F (GgufImage.cpp:231-246)
        if (const GgufTensor *t = quantized(fused, 2ull * E * F, H)) {
          gate.routed = packImagesOfRows(file, *t, expertRuns(E, F, 2ull * F, 0));
          up.routed = packImagesOfRows(file, *t, expertRuns(E, F, 2ull * F, F));
          gate.whole = up.whole = true;
        }
      } else {
        if (const GgufTensor *t = quantized(p + "ffn_gate_exps.weight", uint64_t{E} * F, H)) {
          gate.routed = packImagesOfRows(file, *t, expertRuns(E, F, F, 0));
          gate.whole = true;
        }
        if (const GgufTensor *t = quantized(p + "ffn_up_exps.weight", uint64_t{E} * F, H)) {
          up.routed = packImagesOfRows(file, *t, expertRuns(E, F, F, 0));
          up.whole = true;
        }
      }
      if (const GgufTensor *t = quantized(p + "ffn_down_exps.weight", uint64_t{E} * H, F)) {
        down.routed = packImagesOfRows(file, *t, expertRuns(E, H, H, 0));
        down.whole = true;
      }
      if (S) {
        // the shared expert: gate and up of S slices of F rows; down's S column windows of F inputs (GgufImage.cpp:254-260)
        const GgufTensor *sg = quantized(p + "ffn_gate_shexp.weight", uint64_t{S} * F, H), *su = quantized(p + "ffn_up_shexp.weight", uint64_t{S} * F, H);
        const GgufTensor *sd = quantized(p + "ffn_down_shexp.weight", H, uint64_t{S} * F);
        auto sameFormat = [&](const GgufTensor *t, const Side &side, const char *what) {
          if (t && side.whole && *imageFormat(t->type) != side.routed.formatId) {
            problems.add(p + what + " is not of the routed experts' format");
            return false;
          }
          return t && side.whole;
        };
        if (sameFormat(sg, gate, "ffn_gate_shexp.weight")) gate.shared = packImagesOfRows(file, *sg, expertRuns(S, F, F, 0));
        else gate.whole = false;
        if (sameFormat(su, up, "ffn_up_shexp.weight")) up.shared = packImagesOfRows(file, *su, expertRuns(S, F, F, 0));
        else up.whole = false;
        if (sameFormat(sd, down, "ffn_down_shexp.weight")) {
          for (uint32_t s = 0; s < S; ++s) {
            const PackedImages window = packImagesOfRows(file, *sd, {RowRuns{}}, uint64_t{s} * F, F);
            down.shared.bytes.insert(down.shared.bytes.end(), window.bytes.begin(), window.bytes.end());
          }
        } else down.whole = false;
        if (d.sharedGate)
          if (const GgufTensor *t = floats(p + "ffn_gate_inp_shexp.weight", 1, H)) out.sharedScalarGate = loadFloat32Values(backend, file, *t);
      }
      if (gate.whole && up.whole && gate.routed.formatId != up.routed.formatId) {
        problems.add(p + "ffn_up_exps.weight is not of ffn_gate_exps.weight's format");
        gate.whole = false;
      }
      out.experts.format = gate.routed.formatId;
      out.experts.downFormat = down.routed.formatId;
      out.experts.gate = upload(gate, "expert gate images");
      out.experts.up = upload(up, "expert up images");
      out.experts.down = upload(down, "expert down images");
    }
    w.layers.at(layer) = std::move(out);
  }
  w.finalNorm = load.norm("output_norm.weight", H);
  const GgufTensor *table = load.tensor("token_embd.weight", d.vocabulary, H);
  if (table) {
    const std::optional<uint32_t> format = imageFormat(table->type);
    if (!format) problems.add("token_embd.weight is of a type the token gather does not read");
    else {
      hip::Buffer rows = loadNativeRows(backend, file, *table, "token table");
      w.embedding = {std::move(rows), *format, d.vocabulary, H};
    }
  }
  w.head = load.projection(file.find("output.weight") ? "output.weight" : "token_embd.weight", d.vocabulary, H);
  w.head.destination = ops::FloatOutput::Float32;
  for (const GgufTensor &t : file.tensors())
    if (!load.read.count(t.name) && !inLaterBlocks(t.name, d.layers)) problems.add(t.name + " is not read by the hybrid driver");
  if (!problems.text.empty()) throw GgufError("GGUF tensors this build cannot load: " + problems.text);
  verify.setTiledGdnHeads(true);
}

} // namespace splash::model
