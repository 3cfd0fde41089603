// C entry points of model::HybridVerify (include/splash_ops.h).
#include "splash_ops.h"
#include "capi/Guard.hpp"
#include "capi/Handles.hpp"
#include "capi/Policies.hpp"
#include "model/GgufTarget.hpp"
#include "model/HybridVerify.hpp"
#include "splash_gguf.h"
#include "model/StepResults.hpp"

#include <array>
#include <memory>

using namespace splash;

struct spo_hybrid_verify {
  std::unique_ptr<hip::Backend> backend;  // a borrowed wrapper of the caller's backend
  std::unique_ptr<model::HybridVerify> verify;
};

namespace {
hip::Buffer B(sp_buffer *b) { return hip::Buffer::share(b); }
std::vector<model::HybridLane> lanesOf(const spo_hybrid_lane *lanes, uint32_t count) {
  capi::require(lanes && count, "lanes");
  std::vector<model::HybridLane> out;
  for (uint32_t i = 0; i < count; ++i) {
    const spo_verify_lane &b = lanes[i].block;
    out.push_back({{b.rows, b.committed, b.table_first,
                    ops::SamplingPolicy{b.temperature, b.min_p, b.top_k, b.top_p > 0.0f ? b.top_p : 1.0f}, b.remaining},
                   lanes[i].pending_path,
                   lanes[i].parity});
  }
  return out;
}
} // namespace

extern "C" {

sp_status spo_hybrid_verify_create(sp_backend *backend, const spo_hybrid_dimensions *d, uint32_t max_lanes, uint32_t physical_pages,
                                   uint32_t page_table_entries, spo_hybrid_verify **out) {
  return spo_hybrid_verify_create_chunked(backend, d, max_lanes, physical_pages, page_table_entries, 0, out);
}
sp_status spo_hybrid_verify_create_chunked(sp_backend *backend, const spo_hybrid_dimensions *d, uint32_t max_lanes, uint32_t physical_pages,
                                           uint32_t page_table_entries, uint32_t prefill_rows, spo_hybrid_verify **out) {
  return capi::guard([&] {
    capi::require(backend && d && out, "backend, dimensions or result");
    auto holder = std::make_unique<spo_hybrid_verify>();
    holder->backend = std::make_unique<hip::Backend>(backend);
    model::HybridDimensions dims;
    dims.hidden = d->hidden;
    dims.vocabulary = d->vocabulary;
    dims.layers = d->layers;
    dims.attentionInterval = d->attention_interval;
    dims.qHeads = d->q_heads;
    dims.kvHeads = d->kv_heads;
    dims.headDimension = d->head_dim;
    dims.rotaryPairs = d->rotary_pairs;
    dims.normalizeHeads = d->normalize_heads != 0;
    dims.gatedAttention = d->gated_attention != 0;
    dims.ropeTheta = d->rope_theta;
    dims.gdnKeyHeads = d->gdn_key_heads;
    dims.gdnValueHeads = d->gdn_value_heads;
    dims.gdnPackedWidth = d->gdn_packed_width;
    dims.experts = d->experts;
    dims.topK = d->top_k;
    dims.expertFfn = d->expert_ffn;
    dims.sharedSlices = d->shared_slices;
    dims.sharedGate = d->shared_gate != 0;
    dims.denseFfn = d->dense_ffn;
    holder->verify = std::make_unique<model::HybridVerify>(*holder->backend, dims, max_lanes, physical_pages, page_table_entries, prefill_rows);
    *out = holder.release();
  });
}
void spo_hybrid_verify_destroy(spo_hybrid_verify *verify) { delete verify; }

sp_status spo_hybrid_verify_set_capture(spo_hybrid_verify *verify, const uint32_t *layers, uint32_t count, sp_buffer *destination) {
  return capi::guard([&] {
    capi::require(verify && (layers || !count), "verify or layers");
    verify->verify->setCapture(std::vector<uint32_t>(layers, layers + count), B(destination));
  });
}

sp_status spo_hybrid_verify_set_penalties(spo_hybrid_verify *verify, uint32_t lane, float repetition, float presence, float frequency) {
  return capi::guard([&] {
    capi::require(verify, "verify");
    verify->verify->setPenalties(lane, {repetition, presence, frequency});
  });
}

sp_status spo_hybrid_verify_set_admission(spo_hybrid_verify *verify, uint32_t lane, uint32_t constrained, uint32_t excludes_stop_tokens) {
  return capi::guard([&] {
    capi::require(verify, "verify");
    verify->verify->setAdmission(lane, constrained != 0, excludes_stop_tokens != 0);
  });
}
sp_status spo_hybrid_verify_set_stop_tokens(spo_hybrid_verify *verify, const uint32_t *stop_tokens) {
  return capi::guard([&] {
    capi::require(verify, "verify");
    std::array<uint32_t, SAMPLING_STOP_TOKENS> stops{SAMPLING_NO_TOKEN, SAMPLING_NO_TOKEN, SAMPLING_NO_TOKEN, SAMPLING_NO_TOKEN};
    if (stop_tokens) for (size_t i = 0; i < stops.size(); ++i) stops[i] = stop_tokens[i];
    verify->verify->setStopTokens(stops);
  });
}
sp_status spo_hybrid_verify_set_thinking_cutoff(spo_hybrid_verify *verify, uint32_t lane, const spo_thinking_cutoff *cutoff) {
  return capi::guard([&] {
    capi::require(verify, "verify");
    verify->verify->setThinkingCutoff(lane, capi::cutoffOf(cutoff));
  });
}

sp_status spg_hybrid_dimensions(const spg_file *file, spo_hybrid_dimensions *out) {
  return capi::guard([&] {
    capi::require(out, "result");
    const model::HybridDimensions d = model::ggufHybridDimensions(capi::ggufOf(file));
    *out = {};
    out->hidden = d.hidden;
    out->vocabulary = d.vocabulary;
    out->layers = d.layers;
    out->attention_interval = d.attentionInterval;
    out->q_heads = d.qHeads;
    out->kv_heads = d.kvHeads;
    out->head_dim = d.headDimension;
    out->rotary_pairs = d.rotaryPairs;
    out->normalize_heads = d.normalizeHeads;
    out->gated_attention = d.gatedAttention;
    out->rope_theta = d.ropeTheta;
    out->gdn_key_heads = d.gdnKeyHeads;
    out->gdn_value_heads = d.gdnValueHeads;
    out->gdn_packed_width = d.gdnPackedWidth;
    out->experts = d.experts;
    out->top_k = d.topK;
    out->expert_ffn = d.expertFfn;
    out->shared_slices = d.sharedSlices;
    out->shared_gate = d.sharedGate;
    out->dense_ffn = d.denseFfn;
  });
}
sp_status spo_hybrid_verify_load_gguf(spo_hybrid_verify *verify, const spg_file *file) {
  return capi::guard([&] {
    capi::require(verify, "verify");
    model::loadGgufHybridWeights(*verify->backend, capi::ggufOf(file), *verify->verify);
  });
}

sp_status spo_hybrid_verify_set_layer(spo_hybrid_verify *verify, uint32_t layer, const spo_hybrid_layer *l) {
  return capi::guard([&] {
    capi::require(verify && l && l->mixer_input && l->mixer_output, "verify, layer or projections");
    const bool dense = verify->verify->dimensions().dense();
    capi::require(dense ? (l->ffn_gate && l->ffn_up && l->ffn_down) : l->router != nullptr, "the layer's FFN");
    model::HybridWeights &w = verify->verify->weights();
    if (layer >= w.layers.size()) throw std::invalid_argument("no such layer");
    model::HybridLayer out;
    out.mixerInput = capi::projectionOf(l->mixer_input);
    out.mixerOutput = capi::projectionOf(l->mixer_output);
    out.inputNorm = B(l->input_norm);
    out.postNorm = B(l->post_norm);
    out.queryNorm = B(l->query_norm);
    out.keyNorm = B(l->key_norm);
    out.convolutionWeights = B(l->convolution_weights);
    out.decay = B(l->decay_weights);
    out.timeBias = B(l->time_bias);
    out.mixerNorm = B(l->mixer_norm);
    if (dense) {
      out.ffnGate = capi::projectionOf(l->ffn_gate);
      out.ffnUp = capi::projectionOf(l->ffn_up);
      out.ffnDown = capi::projectionOf(l->ffn_down);
    } else {
      out.router = capi::projectionOf(l->router);
      out.router.destination = ops::FloatOutput::Float32;
      out.experts = {B(l->gate_images), B(l->up_images), B(l->down_images), l->expert_format, l->expert_down_format};
    }
    if (l->shared_scalar_gate) out.sharedScalarGate = B(l->shared_scalar_gate);
    w.layers[layer] = std::move(out);
  });
}
sp_status spo_hybrid_verify_set_head(spo_hybrid_verify *verify, uint32_t embedding_format, sp_buffer *embedding_rows, sp_buffer *final_norm,
                                     const spo_projection *head) {
  return capi::guard([&] {
    capi::require(verify && head, "verify or head");
    model::HybridWeights &w = verify->verify->weights();
    const model::HybridDimensions &d = verify->verify->dimensions();
    w.embedding = {B(embedding_rows), embedding_format, d.vocabulary, d.hidden};
    w.finalNorm = B(final_norm);
    w.head = capi::projectionOf(head);
    w.head.destination = ops::FloatOutput::Float32;
  });
}
sp_status spo_hybrid_verify_results(spo_hybrid_verify *verify, const spo_hybrid_lane *lanes, uint32_t count, uint32_t *tokens,
                                    uint32_t *retained, uint32_t *accepted, uint32_t *retained_rows) {
  return capi::guard([&] {
    capi::require(verify && lanes && count && tokens && retained && accepted && retained_rows, "verify, lanes or results");
    model::HybridVerify &v = *verify->verify;
    std::vector<model::StepLane> list;
    uint32_t first = 0;
    for (uint32_t i = 0; i < count; ++i) { list.push_back({first, lanes[i].block.rows, lanes[i].block.remaining}); first += lanes[i].block.rows; }
    model::readStepResults(list, v.tokens(), v.retained(), v.acceptedCount(), v.retainedRows(), v.dimensions().vocabulary, tokens, retained,
                           accepted, retained_rows);
  });
}
sp_status spo_hybrid_verify_buffer(spo_hybrid_verify *verify, uint32_t which, uint32_t index, sp_buffer **out) {
  return capi::guard([&] {
    capi::require(verify && out, "verify or result");
    model::HybridVerify &v = *verify->verify;
    hip::Buffer b;
    switch (which) {
    case SPO_VERIFY_INPUT_TOKENS: b = v.inputTokens(); break;
    case SPO_VERIFY_TREE_ROWS: b = v.treeRows(); break;
    case SPO_VERIFY_DEPTHS: b = v.depths(); break;
    case SPO_VERIFY_UNIFORMS: b = v.uniforms(); break;
    case SPO_VERIFY_TOKENS: b = v.tokens(); break;
    case SPO_VERIFY_RETAINED: b = v.retained(); break;
    case SPO_VERIFY_ACCEPTED: b = v.acceptedCount(); break;
    case SPO_VERIFY_RETAINED_ROWS: b = v.retainedRows(); break;
    case SPO_VERIFY_PAGE_TABLE: b = v.pageTable(); break;
    case SPO_VERIFY_KV_POOL: b = v.kvPool(index); break;
    case SPO_VERIFY_LOGITS: b = v.logits(); break;
    case SPO_VERIFY_DRAFT_PROBABILITIES: b = v.draftProbabilities(); break;
    case SPO_VERIFY_HIDDEN: b = v.hidden(index); break;
    case SPO_VERIFY_PENALTY_WORDS: b = v.penaltyWords(); break;
    case SPO_VERIFY_TOKEN_MASK: b = v.tokenMask(); break;
    case SPO_VERIFY_GDN_STATES: b = v.gdnStates(); break;
    case SPO_VERIFY_GDN_TAPE: b = v.gdnTape(); break;
    default: throw std::invalid_argument("no such verify buffer");
    }
    sp_buffer_retain(b.handle());
    *out = b.handle();
  });
}
sp_status spo_hybrid_verify_layout(const spo_hybrid_verify *verify, uint64_t *page_bytes, uint64_t *cell_bytes, uint64_t *tape_layer_bytes,
                                   spo_gdn_state_strides *strides) {
  return capi::guard([&] {
    capi::require(verify, "verify");
    const model::HybridVerify &v = *verify->verify;
    if (page_bytes) *page_bytes = v.pageBytes();
    if (cell_bytes) *cell_bytes = v.gdnCellBytes();
    if (tape_layer_bytes) *tape_layer_bytes = v.gdnTapeLayerBytes();
    if (strides) *strides = {v.gdnStrides().convolutionLayerBytes, v.gdnStrides().recurrentLayerBytes, v.gdnStrides().convolutionStateBytes};
  });
}
uint64_t spo_hybrid_verify_step_bytes(const spo_hybrid_verify *verify, const spo_hybrid_lane *lanes, uint32_t count) {
  uint64_t bytes = 0;
  capi::guard([&] { capi::require(verify, "verify"); bytes = verify->verify->stepBytes(lanesOf(lanes, count)); });
  return bytes;
}
sp_status spo_hybrid_verify_encode(spo_hybrid_verify *verify, spo_graph *graph, const spo_hybrid_lane *lanes, uint32_t count, int commit) {
  return capi::guard([&] {
    capi::require(verify && graph, "verify or graph");
    verify->verify->encode(capi::graphOf(graph), lanesOf(lanes, count), commit != 0);
  });
}
sp_status spo_hybrid_verify_encode_part(spo_hybrid_verify *verify, spo_graph *graph, uint32_t part, uint32_t index,
                                        const spo_hybrid_lane *lanes, uint32_t count) {
  return capi::guard([&] {
    capi::require(verify && graph, "verify or graph");
    const std::vector<model::HybridLane> list = lanesOf(lanes, count);
    uint32_t rows = 0;
    for (const model::HybridLane &l : list) rows += l.block.rows;
    if (part == 0) verify->verify->encodeEmbedding(capi::graphOf(graph), rows);
    else if (part == 1) verify->verify->encodeLayer(capi::graphOf(graph), index, list);
    else if (part == 2) verify->verify->encodeHead(capi::graphOf(graph), rows);
    else throw std::invalid_argument("no such part of the step");
  });
}

sp_status spo_hybrid_verify_encode_prefill(spo_hybrid_verify *verify, spo_graph *graph, uint32_t lane, uint32_t table_first,
                                           uint32_t committed, uint32_t tokens, uint32_t parity, uint32_t first_layer, uint32_t layer_count) {
  return capi::guard([&] {
    capi::require(verify && graph, "verify or graph");
    verify->verify->encodePrefill(capi::graphOf(graph), lane, table_first, committed, tokens, parity, first_layer, layer_count);
  });
}

} // extern "C"
