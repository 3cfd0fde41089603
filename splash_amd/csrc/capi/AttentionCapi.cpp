// C entry points of ops::PagedAttention (include/splash_ops.h).
#include "splash_ops.h"
#include "capi/Guard.hpp"
#include "capi/Handles.hpp"
#include "ops/PagedAttention.hpp"

using namespace splash;


namespace {
ops::KvPages pagesOf(sp_buffer *table, sp_buffer *pool, uint64_t pageBytes) {
  return {hip::Buffer::share(table), hip::Buffer::share(pool), pageBytes};
}
} // namespace

extern "C" {

uint64_t spo_kv_page_bytes(uint32_t kv_heads, uint32_t head_dim) { return attention_page_bytes(kv_heads, head_dim); }
uint64_t spo_kv_key_index(uint32_t head, uint32_t token, uint32_t dim, uint32_t head_dim) {
  return attention_key_index(head, token, dim, head_dim);
}
uint64_t spo_kv_value_index(uint32_t head, uint32_t token, uint32_t dim, uint32_t head_dim) {
  return attention_value_index(head, token, dim, head_dim);
}

sp_status spo_attention_plan_create(const spo_attention_geometry *geometry, const spo_attention_rows *sequences, uint32_t count,
                                    spo_attention_plan **out) {
  return capi::guard([&] {
    capi::require(geometry && sequences && out, "geometry, sequences or result");
    std::vector<ops::AttentionRows> rows;
    for (uint32_t i = 0; i < count; ++i)
      rows.push_back({sequences[i].first_row, sequences[i].rows, sequences[i].committed, sequences[i].table_first});
    const ops::AttentionGeometry g{geometry->q_heads, geometry->kv_heads, geometry->head_dim, geometry->rotary_pairs,
                                   geometry->normalize != 0, geometry->gated != 0, geometry->int8_queries != 0};
    *out = new spo_attention_plan{ops::PagedAttention::plan(g, std::move(rows))};
  });
}
void spo_attention_plan_destroy(spo_attention_plan *plan) { delete plan; }
uint32_t spo_attention_plan_splits(const spo_attention_plan *plan) { return plan ? plan->plan.splits() : 0; }
sp_status spo_attention_workspace(const spo_attention_plan *plan, uint64_t sizes[4]) {
  return capi::guard([&] {
    capi::require(plan && sizes, "plan or result");
    const ops::AttentionWorkspaceSize w = plan->plan.workspace();
    sizes[0] = w.queries; sizes[1] = w.querySums; sizes[2] = w.partials; sizes[3] = w.partialSums;
  });
}
sp_status spo_attention_add_projection(spo_graph *graph, const spo_attention_plan *plan, sp_buffer *qkv, sp_buffer *query_norm,
                                       sp_buffer *key_norm, sp_buffer *rope_cos, sp_buffer *rope_sin, sp_buffer *queries,
                                       sp_buffer *query_sums, sp_buffer *page_table, sp_buffer *pool, uint64_t page_bytes) {
  return capi::guard([&] {
    capi::require(graph && plan, "graph or plan");
    ops::AttentionProjectionBuffers b{hip::Buffer::share(qkv), hip::Buffer::share(query_norm), hip::Buffer::share(key_norm),
                                      hip::Buffer::share(rope_cos), hip::Buffer::share(rope_sin)};
    ops::AttentionWorkspace w{hip::Buffer::share(queries), hip::Buffer::share(query_sums), {}, {}};
    ops::PagedAttention::addProjection(capi::graphOf(graph), plan->plan, b, w, pagesOf(page_table, pool, page_bytes));
  });
}
sp_status spo_attention_add_attention(spo_graph *graph, const spo_attention_plan *plan, sp_buffer *queries, sp_buffer *query_sums,
                                      sp_buffer *partials, sp_buffer *partial_sums, sp_buffer *tree_rows, sp_buffer *page_table,
                                      sp_buffer *pool, uint64_t page_bytes, sp_buffer *output, sp_buffer *output_table,
                                      sp_buffer *packed_qkv) {
  return capi::guard([&] {
    capi::require(graph && plan, "graph or plan");
    ops::AttentionWorkspace w{hip::Buffer::share(queries), hip::Buffer::share(query_sums), hip::Buffer::share(partials),
                              hip::Buffer::share(partial_sums)};
    ops::PagedAttention::addAttention(capi::graphOf(graph), plan->plan, w, hip::Buffer::share(tree_rows),
                                      pagesOf(page_table, pool, page_bytes), hip::Buffer::share(output),
                                      hip::Buffer::share(output_table), hip::Buffer::share(packed_qkv));
  });
}
sp_status spo_attention_add_path_commit(spo_graph *graph, const spo_attention_plan *plan, sp_buffer *retained,
                                        sp_buffer *page_table, sp_buffer *pool, uint64_t page_bytes) {
  return capi::guard([&] {
    capi::require(graph && plan, "graph or plan");
    ops::PagedAttention::addPathCommit(capi::graphOf(graph), plan->plan, hip::Buffer::share(retained),
                                       pagesOf(page_table, pool, page_bytes));
  });
}

sp_status spo_attention_chunk_plan_create(const spo_attention_geometry *geometry, const spo_attention_chunk *chunks, uint32_t count,
                                          spo_attention_chunk_plan **out) {
  return capi::guard([&] {
    capi::require(geometry && chunks && out, "geometry, chunks or result");
    std::vector<ops::AttentionChunk> list;
    for (uint32_t i = 0; i < count; ++i) list.push_back({chunks[i].first_row, chunks[i].tokens, chunks[i].committed, chunks[i].table_first});
    const ops::AttentionGeometry g{geometry->q_heads, geometry->kv_heads, geometry->head_dim, geometry->rotary_pairs,
                                   geometry->normalize != 0, geometry->gated != 0, geometry->int8_queries != 0};
    *out = new spo_attention_chunk_plan{ops::PagedAttention::planChunks(g, list)};
  });
}
void spo_attention_chunk_plan_destroy(spo_attention_chunk_plan *plan) { delete plan; }
uint32_t spo_attention_chunk_plan_dispatches(const spo_attention_chunk_plan *plan) {
  return plan ? uint32_t(plan->plan.dispatches().size()) : 0;
}
sp_status spo_attention_chunk_workspace(const spo_attention_chunk_plan *plan, uint64_t sizes[4]) {
  return capi::guard([&] {
    capi::require(plan && sizes, "plan or result");
    const ops::AttentionWorkspaceSize w = plan->plan.workspace();
    sizes[0] = w.queries; sizes[1] = w.querySums; sizes[2] = w.partials; sizes[3] = w.partialSums;
  });
}
sp_status spo_attention_add_chunk_projection(spo_graph *graph, const spo_attention_chunk_plan *plan, sp_buffer *qkv, sp_buffer *query_norm,
                                             sp_buffer *key_norm, sp_buffer *rope_cos, sp_buffer *rope_sin, sp_buffer *queries,
                                             sp_buffer *query_sums, sp_buffer *page_table, sp_buffer *pool, uint64_t page_bytes) {
  return capi::guard([&] {
    capi::require(graph && plan, "graph or plan");
    ops::AttentionProjectionBuffers b{hip::Buffer::share(qkv), hip::Buffer::share(query_norm), hip::Buffer::share(key_norm),
                                      hip::Buffer::share(rope_cos), hip::Buffer::share(rope_sin)};
    ops::AttentionWorkspace w{hip::Buffer::share(queries), hip::Buffer::share(query_sums), {}, {}};
    ops::PagedAttention::addChunkProjection(capi::graphOf(graph), plan->plan, b, w, pagesOf(page_table, pool, page_bytes));
  });
}
sp_status spo_attention_add_chunk_attention(spo_graph *graph, const spo_attention_chunk_plan *plan, sp_buffer *queries,
                                            sp_buffer *query_sums, sp_buffer *partials, sp_buffer *partial_sums, sp_buffer *tree_rows,
                                            sp_buffer *page_table, sp_buffer *pool, uint64_t page_bytes, sp_buffer *output,
                                            sp_buffer *output_table, sp_buffer *packed_qkv) {
  return capi::guard([&] {
    capi::require(graph && plan, "graph or plan");
    ops::AttentionWorkspace w{hip::Buffer::share(queries), hip::Buffer::share(query_sums), hip::Buffer::share(partials),
                              hip::Buffer::share(partial_sums)};
    ops::PagedAttention::addChunkAttention(capi::graphOf(graph), plan->plan, w, hip::Buffer::share(tree_rows),
                                           pagesOf(page_table, pool, page_bytes), hip::Buffer::share(output),
                                           hip::Buffer::share(output_table), hip::Buffer::share(packed_qkv));
  });
}

} // extern "C"
