// C entry points of ops::DraftAttention (include/splash_ops.h).
#include "splash_ops.h"
#include "capi/Guard.hpp"
#include "capi/Handles.hpp"
#include "ops/DraftAttention.hpp"

#include <span>

using namespace splash;

namespace {
hip::Buffer B(sp_buffer *b) { return hip::Buffer::share(b); }
ops::DraftAttentionPlan planOf(uint32_t hidden, uint32_t lanes) { return ops::DraftAttention::plan(ops::DraftAttentionShape::of(hidden), lanes); }
} // namespace

sp_status spo_draft_attention_workspace(uint32_t hidden, uint32_t lanes, uint64_t sizes[5]) {
  return capi::guard([&] {
    capi::require(sizes, "sizes");
    const ops::DraftAttentionWorkspace w = planOf(hidden, lanes).workspace();
    sizes[0] = w.convolutionBytes;
    sizes[1] = w.qkvBytes;
    sizes[2] = w.groupedQueriesBytes;
    sizes[3] = w.queryKeysBytes;
    sizes[4] = w.queryValuesBytes;
  });
}

sp_status spo_draft_attention_add_convolution(spo_graph *graph, sp_buffer *input, sp_buffer *dynamic, sp_buffer *weights, sp_buffer *residual,
                                              sp_buffer *output, uint32_t hidden, uint32_t lanes, uint32_t finish) {
  return capi::guard([&] {
    capi::require(graph, "graph");
    ops::DraftAttention::addConvolution(capi::graphOf(graph), {B(input), B(dynamic), B(weights), B(residual), B(output)}, planOf(hidden, lanes),
                                        finish ? ops::DraftConvolutionStage::Residual : ops::DraftConvolutionStage::Prepare);
  });
}

sp_status spo_draft_attention_add_prepare(spo_graph *graph, sp_buffer *qkv, sp_buffer *grouped_queries, sp_buffer *query_norm,
                                          sp_buffer *key_norm, sp_buffer *rope_cos, sp_buffer *rope_sin, sp_buffer *query_keys,
                                          sp_buffer *query_values, uint32_t hidden, uint32_t lanes) {
  return capi::guard([&] {
    capi::require(graph, "graph");
    ops::DraftAttention::addPrepare(capi::graphOf(graph),
                                    {B(qkv), B(grouped_queries), B(query_norm), B(key_norm), B(rope_cos), B(rope_sin), B(query_keys), B(query_values)},
                                    planOf(hidden, lanes));
  });
}

sp_status spo_draft_attention_add_decode(spo_graph *graph, sp_buffer *grouped_queries, sp_buffer *rings, const uint64_t *keys,
                                         const uint64_t *values, sp_buffer *query_keys, sp_buffer *query_values,
                                         const uint32_t *cache_lengths, uint32_t hidden, uint32_t lanes) {
  return capi::guard([&] {
    capi::require(graph && keys && values && cache_lengths, "graph, rings or cache lengths");
    ops::DraftAttention::addDecode(capi::graphOf(graph),
                                   {B(grouped_queries), {B(rings), std::span(keys, lanes), std::span(values, lanes)}, B(query_keys), B(query_values)},
                                   std::span(cache_lengths, lanes), planOf(hidden, lanes));
  });
}

sp_status spo_draft_attention_add_context_prefill(spo_graph *graph, sp_buffer *context_kv, sp_buffer *key_norm, sp_buffer *rope_cos,
                                                  sp_buffer *rope_sin, sp_buffer *rings, uint64_t keys, uint64_t values, uint32_t tokens,
                                                  uint32_t start_position, uint32_t hidden) {
  return capi::guard([&] {
    capi::require(graph, "graph");
    ops::DraftAttention::addContextPrefill(capi::graphOf(graph), B(context_kv), B(key_norm), B(rope_cos), B(rope_sin), B(rings), keys, values,
                                           tokens, start_position, ops::DraftAttentionShape::of(hidden));
  });
}

sp_status spo_draft_attention_add_context_commit(spo_graph *graph, sp_buffer *context_kv, sp_buffer *key_norm, sp_buffer *rope_cos,
                                                 sp_buffer *rope_sin, sp_buffer *rings, const uint64_t *keys, const uint64_t *values,
                                                 sp_buffer *retained_rows, sp_buffer *lane_rows, const uint32_t *start_positions,
                                                 uint32_t lanes, uint32_t rows, uint32_t lane_cap, uint32_t hidden) {
  return capi::guard([&] {
    capi::require(graph && keys && values && start_positions, "graph, rings or start positions");
    ops::DraftAttention::addContextCommit(capi::graphOf(graph), B(context_kv), B(key_norm), B(rope_cos), B(rope_sin),
                                          {B(rings), std::span(keys, lanes), std::span(values, lanes)}, B(retained_rows), B(lane_rows),
                                          std::span(start_positions, lanes), {lanes, rows, lane_cap}, ops::DraftAttentionShape::of(hidden));
  });
}

sp_status spo_draft_context_window_bytes(uint32_t width, uint64_t *bytes) {
  return capi::guard([&] {
    capi::require(bytes, "result");
    *bytes = ops::DraftAttention::contextWindowBytes(width);
  });
}

sp_status spo_draft_attention_add_window_store(spo_graph *graph, sp_buffer *context, sp_buffer *window, uint32_t rows, uint32_t start_position,
                                               uint32_t width) {
  return capi::guard([&] {
    capi::require(graph, "graph");
    ops::DraftAttention::addWindowStore(capi::graphOf(graph), B(context), B(window), rows, start_position, width);
  });
}

sp_status spo_draft_attention_add_window_commit(spo_graph *graph, sp_buffer *context, sp_buffer *window, sp_buffer *retained,
                                                sp_buffer *lane_rows, uint32_t context_rows, uint32_t rows, uint32_t start_position,
                                                uint32_t width) {
  return capi::guard([&] {
    capi::require(graph, "graph");
    ops::DraftAttention::addWindowCommit(capi::graphOf(graph), B(context), B(window), B(retained), B(lane_rows), context_rows, rows,
                                         start_position, width);
  });
}

sp_status spo_draft_attention_add_window_load(spo_graph *graph, sp_buffer *window, sp_buffer *context, uint32_t rows, uint32_t start_position,
                                              uint32_t width) {
  return capi::guard([&] {
    capi::require(graph, "graph");
    ops::DraftAttention::addWindowLoad(capi::graphOf(graph), B(window), B(context), rows, start_position, width);
  });
}

sp_status spo_draft_attention_add_mask_rows(spo_graph *graph, sp_buffer *mask, sp_buffer *rows, uint32_t width, uint32_t lanes) {
  return capi::guard([&] {
    capi::require(graph, "graph");
    ops::DraftAttention::addMaskRows(capi::graphOf(graph), B(mask), B(rows), width, lanes);
  });
}

// ---- model::DFlashDraft ----
#include "model/DFlashDraft.hpp"

#include <memory>
#include <optional>

struct spo_dflash_draft {
  std::unique_ptr<hip::Backend> backend;  // a borrowed wrapper of the caller's backend
  std::unique_ptr<ops::Linear> linear;
  model::DFlashDraftWeights weights;
  ops::Projection head;
  std::optional<model::DFlashDraft> draft;  // built by the first encode, once every weight is set
  uint32_t maxLanes = 0, contextRows = 0;
  model::DFlashDecodeBuffers decode;
  model::DFlashContextBuffers context;
  std::vector<model::DFlashLaneState> lanes;

  model::DFlashDraft &ready() {
    if (!draft) {
      draft.emplace(weights, *linear, head);
      const ops::LinearScratchSize size = draft->scratchSize(std::max(maxLanes * DRAFT_ATTENTION_QUERY_ROWS, contextRows));
      auto device = [&](uint64_t bytes, const char *label) {
        return backend->allocateBuffer(std::max<uint64_t>(bytes, 16), hip::BufferStorage::Private, label);
      };
      decode.scratch = {device(size.input, "draft linear table"), device(size.partials, "draft linear partials"),
                        device(size.counters, "draft linear counters")};
      context.scratch = decode.scratch;
    }
    return *draft;
  }
};

namespace {
const ops::Projection &P(const spo_projection *p, const char *what) {
  capi::require(p, what);
  return p->projection;
}
} // namespace

sp_status spo_dflash_draft_create(sp_backend *backend, const spo_dflash_layout *l, uint32_t max_lanes, uint32_t context_rows,
                                  spo_dflash_draft **out) {
  return capi::guard([&] {
    capi::require(backend && l && out, "backend, layout or result");
    if (!max_lanes || max_lanes > DRAFT_ATTENTION_MAXIMUM_LANES) throw std::invalid_argument("invalid draft batch width");
    auto holder = std::make_unique<spo_dflash_draft>();
    holder->backend = std::make_unique<hip::Backend>(backend);
    holder->linear = std::make_unique<ops::Linear>(holder->backend->deviceInfo());
    model::DFlashDraftLayout &layout = holder->weights.layout;
    layout = {l->layers, l->hidden, l->vocabulary, l->intermediate, l->target_layers};
    if (!layout.layers || !layout.hiddenSize || layout.hiddenSize % DRAFT_CONTEXT_GROUP || !layout.vocabularySize || !layout.intermediateSize ||
        !layout.targetLayerCount)
      throw std::invalid_argument("DFlash draft layout contains a zero dimension");
    (void)ops::DraftAttention::plan(layout.attentionShape(), max_lanes);
    holder->weights.layers.resize(layout.layers);
    holder->maxLanes = max_lanes;
    holder->contextRows = std::max(context_rows, max_lanes * DRAFT_ATTENTION_ROPE_LANE_ROWS);
    if (holder->contextRows > ops::kMaximumDispatchRows) throw std::invalid_argument("a draft context call takes up to 256 rows");
    const hip::Backend &b = *holder->backend;
    auto device = [&](uint64_t bytes, const char *label) { return b.allocateBuffer(std::max<uint64_t>(bytes, 16), hip::BufferStorage::Private, label); };
    const uint64_t rows = uint64_t{max_lanes} * DRAFT_ATTENTION_QUERY_ROWS, hidden = layout.hiddenSize;
    const ops::DraftAttentionWorkspace w = ops::DraftAttention::plan(layout.attentionShape(), max_lanes).workspace();
    model::DFlashDecodeBuffers &d = holder->decode;
    d.hidden = {device(rows * hidden * 2, "draft hidden 0"), device(rows * hidden * 2, "draft hidden 1")};
    d.normalized = device(rows * hidden * 2, "draft normalized");
    d.dynamic = device(rows * layout.dynamicSize() * 2, "draft dynamic");
    d.convolved = device(w.convolutionBytes, "draft convolved");
    d.proposalQkv = device(w.qkvBytes, "draft q|k|v");
    d.attention = device(w.groupedQueriesBytes, "draft attention");
    d.projected = device(rows * hidden * 2, "draft projected");
    d.residual = device(rows * hidden * 2, "draft residual");
    d.intermediate = device(rows * layout.intermediateSize * 2, "draft intermediate");
    d.finalHidden = device(rows * hidden * 2, "draft final hidden");
    d.logits = device(rows * layout.vocabularySize * 4, "draft logits");
    d.selectorHidden = device(rows * DRAFT_SELECTOR_RANK * 2, "draft selector hidden");
    d.queryKeys = device(w.queryKeysBytes, "draft query keys");
    d.queryValues = device(w.queryValuesBytes, "draft query values");
    const uint64_t ropeBytes = uint64_t{max_lanes} * DRAFT_ATTENTION_ROPE_LANE_ROWS * DRAFT_ATTENTION_ROPE_PAIRS * 4;
    d.ropeCos = device(ropeBytes, "draft RoPE cosine");
    d.ropeSin = device(ropeBytes, "draft RoPE sine");
    d.rings = device(uint64_t{max_lanes} * layout.ringBytes(), "draft rings");
    model::DFlashContextBuffers &c = holder->context;
    const uint64_t contextRows = holder->contextRows;
    c.capturedTargetHidden = device(contextRows * layout.targetHiddenSize() * 2, "draft captured target hidden");
    c.projected = device(contextRows * hidden * 2, "draft context projected");
    c.hidden = device(contextRows * hidden * 2, "draft context hidden");
    c.contextKv = device(contextRows * layout.contextKvSize() * 2, "draft context k/v");
    c.ropeCos = device(contextRows * DRAFT_ATTENTION_ROPE_PAIRS * 4, "draft context RoPE cosine");
    c.ropeSin = device(contextRows * DRAFT_ATTENTION_ROPE_PAIRS * 4, "draft context RoPE sine");
    c.rings = d.rings;
    c.windows = device(uint64_t{max_lanes} * layout.windowBytes(), "draft context windows");
    for (uint32_t lane = 0; lane < max_lanes; ++lane) holder->lanes.push_back({lane * layout.ringBytes(), lane * layout.windowBytes()});
    *out = holder.release();
  });
}

void spo_dflash_draft_destroy(spo_dflash_draft *draft) { delete draft; }

sp_status spo_dflash_draft_set_layer(spo_dflash_draft *draft, uint32_t layer, const spo_dflash_layer *w) {
  return capi::guard([&] {
    capi::require(draft && w, "draft or weights");
    if (layer >= draft->weights.layers.size() || draft->draft) throw std::invalid_argument("no such draft layer, or the draft has already encoded");
    model::DFlashDraftLayerWeights &to = draft->weights.layers[layer];
    to.inputNorm = B(w->input_norm);
    to.attentionConvolution = B(w->attention_convolution);
    to.attentionDynamic = P(w->attention_dynamic, "attention-dynamic");
    to.qkvProjection = P(w->qkv, "qkv");
    to.queryNorm = B(w->query_norm);
    to.keyNorm = B(w->key_norm);
    to.outputProjection = P(w->output, "attention-output");
    to.postAttentionNorm = B(w->post_attention_norm);
    to.mlpConvolution = B(w->mlp_convolution);
    to.mlpDynamic = P(w->mlp_dynamic, "mlp-dynamic");
    to.gateProjection = P(w->gate, "mlp-gate");
    to.upProjection = P(w->up, "mlp-up");
    to.downProjection = P(w->down, "mlp-down");
    to.contextKvProjection = model::projectionRowsFrom(to.qkvProjection, DRAFT_ATTENTION_WIDTH);
  });
}

sp_status spo_dflash_draft_set_model(spo_dflash_draft *draft, const spo_projection *context_projection, sp_buffer *hidden_norm,
                                     sp_buffer *final_norm, const spo_projection *selector, sp_buffer *mask_embedding,
                                     const spo_projection *head) {
  return capi::guard([&] {
    capi::require(draft, "draft");
    if (draft->draft) throw std::invalid_argument("the draft has already encoded");
    draft->weights.contextProjection = P(context_projection, "context projection");
    draft->weights.hiddenNorm = B(hidden_norm);
    draft->weights.finalNorm = B(final_norm);
    draft->weights.selectorProjection = P(selector, "selector projection");
    draft->weights.maskEmbedding = B(mask_embedding);
    draft->head = P(head, "vocabulary head");
  });
}

sp_status spo_dflash_draft_buffer(spo_dflash_draft *draft, spo_dflash_buffer which, uint32_t index, sp_buffer **out) {
  return capi::guard([&] {
    capi::require(draft && out, "draft or result");
    const hip::Buffer *buffer = nullptr;
    switch (which) {
    case SPO_DFLASH_HIDDEN: buffer = &draft->decode.hidden[index & 1]; break;
    case SPO_DFLASH_LOGITS: buffer = &draft->decode.logits; break;
    case SPO_DFLASH_SELECTOR_HIDDEN: buffer = &draft->decode.selectorHidden; break;
    case SPO_DFLASH_FINAL_HIDDEN: buffer = &draft->decode.finalHidden; break;
    case SPO_DFLASH_ROPE_COS: buffer = &draft->decode.ropeCos; break;
    case SPO_DFLASH_ROPE_SIN: buffer = &draft->decode.ropeSin; break;
    case SPO_DFLASH_RINGS: buffer = &draft->decode.rings; break;
    case SPO_DFLASH_WINDOWS: buffer = &draft->context.windows; break;
    case SPO_DFLASH_CAPTURED_TARGET_HIDDEN: buffer = &draft->context.capturedTargetHidden; break;
    case SPO_DFLASH_CONTEXT_ROPE_COS: buffer = &draft->context.ropeCos; break;
    case SPO_DFLASH_CONTEXT_ROPE_SIN: buffer = &draft->context.ropeSin; break;
    case SPO_DFLASH_CONTEXT_HIDDEN: buffer = &draft->context.hidden; break;
    }
    if (!buffer || !*buffer) throw std::invalid_argument("no such draft buffer");
    sp_buffer *raw = buffer->handle();
    sp_buffer_retain(raw);
    *out = raw;
  });
}

sp_status spo_dflash_draft_encode_decode(spo_dflash_draft *draft, spo_graph *graph, const uint32_t *cache_lengths, uint32_t lanes) {
  return capi::guard([&] {
    capi::require(draft && graph && cache_lengths, "draft, graph or cache lengths");
    if (!lanes || lanes > draft->maxLanes) throw std::invalid_argument("invalid draft decode batch");
    model::DFlashDraft &model = draft->ready();
    model.addMaskRows(capi::graphOf(graph), draft->decode.hidden[0], lanes);
    model.addDecode(capi::graphOf(graph), draft->decode, std::span(draft->lanes.data(), lanes), std::span(cache_lengths, lanes));
  });
}

sp_status spo_dflash_draft_encode_context_prefill(spo_dflash_draft *draft, spo_graph *graph, uint32_t lane, uint32_t rows,
                                                  uint32_t start_position, int rebuild) {
  return capi::guard([&] {
    capi::require(draft && graph, "draft or graph");
    if (lane >= draft->maxLanes || rows > draft->contextRows) throw std::invalid_argument("invalid draft context prefill");
    model::DFlashDraft &model = draft->ready();
    if (rebuild) model.addContextRebuild(capi::graphOf(graph), draft->context, draft->lanes[lane], rows, start_position);
    else model.addContextPrefill(capi::graphOf(graph), draft->context, draft->lanes[lane], rows, start_position);
  });
}

sp_status spo_dflash_draft_encode_context_commit(spo_dflash_draft *draft, spo_graph *graph, sp_buffer *retained_rows, sp_buffer *lane_rows,
                                                 const uint32_t *start_positions, uint32_t lanes, uint32_t rows, uint32_t lane_cap) {
  return capi::guard([&] {
    capi::require(draft && graph && start_positions, "draft, graph or start positions");
    if (!lanes || lanes > draft->maxLanes || rows > draft->contextRows) throw std::invalid_argument("invalid draft context batch");
    draft->ready().addContextCommit(capi::graphOf(graph), draft->context, std::span(draft->lanes.data(), lanes), B(retained_rows), B(lane_rows),
                                    std::span(start_positions, lanes), {lanes, rows, lane_cap});
  });
}
