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
