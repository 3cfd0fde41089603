// C entry points of the glue operators, ops::Sampling and model::DenseVerify (include/splash_ops.h).
#include "splash_ops.h"
#include "capi/Guard.hpp"
#include "capi/Handles.hpp"
#include "capi/Policies.hpp"
#include "model/DenseVerify.hpp"
#include "model/StepResults.hpp"
#include "model/GgufTarget.hpp"
#include "model/LookupProposals.hpp"
#include "splash_gguf.h"
#include "ops/DraftSelector.hpp"
#include "ops/Glue.hpp"
#include "ops/Sampling.hpp"

#include <array>
#include <memory>

using namespace splash;

struct spo_dense_verify {
  std::unique_ptr<hip::Backend> backend;  // a borrowed wrapper of the caller's backend
  std::unique_ptr<model::DenseVerify> verify;
};

namespace {
hip::Buffer B(sp_buffer *b) { return hip::Buffer::share(b); }
std::vector<model::VerifyLane> lanesOf(const spo_verify_lane *lanes, uint32_t count) {
  capi::require(lanes && count, "lanes");
  std::vector<model::VerifyLane> out;
  for (uint32_t i = 0; i < count; ++i)
    out.push_back({lanes[i].rows, lanes[i].committed, lanes[i].table_first,
                   ops::SamplingPolicy{lanes[i].temperature, lanes[i].min_p, lanes[i].top_k, lanes[i].top_p > 0.0f ? lanes[i].top_p : 1.0f},
                   lanes[i].remaining});
  return out;
}
ops::AttentionPlan planOf(const model::DenseVerify &v, const std::vector<model::VerifyLane> &lanes) {
  const model::DenseDimensions &d = v.dimensions();
  std::vector<ops::AttentionRows> sequences;
  uint32_t rows = 0;
  for (const model::VerifyLane &l : lanes) { sequences.push_back({rows, l.rows, l.committed, l.tableFirst}); rows += l.rows; }
  return ops::PagedAttention::plan({d.qHeads, d.kvHeads, d.headDimension, d.rotaryPairs, d.normalizeHeads}, sequences);
}
} // namespace

extern "C" {

sp_status spo_norm_add_rms(spo_graph *graph, sp_buffer *input, sp_buffer *weight, sp_buffer *output, uint32_t width, uint32_t rows) {
  return capi::guard([&] { capi::require(graph, "graph"); ops::Normalization::addRms(capi::graphOf(graph), B(input), B(weight), B(output), width, rows); });
}
sp_status spo_norm_add_rms_table(spo_graph *graph, sp_buffer *input, sp_buffer *weight, sp_buffer *output, sp_buffer *table,
                                 uint32_t width, uint32_t rows) {
  return capi::guard([&] {
    capi::require(graph, "graph");
    ops::LinearScratch scratch{B(table), {}, {}};
    ops::Normalization::addRmsTable(capi::graphOf(graph), B(input), B(weight), B(output), scratch, width, rows);
  });
}
sp_status spo_embedding_add(spo_graph *graph, uint32_t format, sp_buffer *native_rows, uint32_t vocabulary, uint32_t hidden,
                            sp_buffer *tokens, sp_buffer *output, uint32_t rows) {
  return capi::guard([&] {
    capi::require(graph, "graph");
    ops::Embedding::add(capi::graphOf(graph), {B(native_rows), format, vocabulary, hidden}, B(tokens), B(output), rows);
  });
}
sp_status spo_row_copy_add(spo_graph *graph, sp_buffer *source, uint32_t from_row, uint32_t from_stride, uint32_t from_column,
                           sp_buffer *destination, uint32_t to_row, uint32_t to_stride, uint32_t to_column, uint32_t rows, uint32_t width) {
  return capi::guard([&] {
    capi::require(graph, "graph");
    ops::RowCopy::add(capi::graphOf(graph), B(source), {from_row, from_stride, from_column}, B(destination), {to_row, to_stride, to_column},
                      rows, width);
  });
}
sp_status spo_rope_add_tree_tables(spo_graph *graph, sp_buffer *inverse_frequency, sp_buffer *depth, sp_buffer *cosines,
                                   sp_buffer *sines, uint32_t pairs, const spo_rope_sequence *sequences, uint32_t count) {
  return capi::guard([&] {
    capi::require(graph && sequences, "graph or sequences");
    std::vector<ops::RopeSequence> list;
    for (uint32_t i = 0; i < count; ++i) list.push_back({sequences[i].first_row, sequences[i].rows, sequences[i].anchor});
    ops::RoPE::addTreeTables(capi::graphOf(graph), B(inverse_frequency), B(depth), B(cosines), B(sines), pairs, list);
  });
}

sp_status spo_float_projection_add(spo_graph *graph, sp_buffer *input, sp_buffer *weight_rows, uint32_t output_size, uint32_t input_size,
                                   uint32_t bf16_weights, sp_buffer *output, uint32_t rows, uint32_t out_stride, uint32_t out_offset,
                                   uint32_t float32_output) {
  return capi::guard([&] {
    capi::require(graph, "graph");
    ops::FloatProjection::add(capi::graphOf(graph), B(input), ops::FloatRows{B(weight_rows), output_size, input_size, bf16_weights != 0},
                              B(output), rows, out_stride, out_offset, float32_output ? ops::FloatOutput::Float32 : ops::FloatOutput::BFloat16);
  });
}

sp_status spo_sampling_workspace(uint32_t rows, uint64_t sizes[5]) {
  return capi::guard([&] {
    capi::require(sizes, "result");
    const ops::SamplingWorkspaceSize s = ops::Sampling::workspace(rows);
    sizes[0] = s.partialValues; sizes[1] = s.partialIndices; sizes[2] = s.masses; sizes[3] = s.ranges; sizes[4] = s.decisions;
  });
}
sp_status spo_sampling_add_verify(spo_graph *graph, const spo_sampling_buffers *b, uint32_t vocabulary, uint32_t logits_stride,
                                  const spo_lane_rows *lanes, const spo_sampling_policy *policy, uint32_t count,
                                  const uint32_t *stop_tokens) {
  return capi::guard([&] {
    capi::require(graph && b && lanes && policy, "graph, buffers, lanes or policies");
    ops::SamplingBuffers buffers{B(b->logits), B(b->tokens), B(b->partial_values), B(b->partial_indices), B(b->draft_probabilities),
                                 B(b->uniforms), B(b->masses), B(b->ranges), B(b->decisions), B(b->input_tokens), B(b->tree_rows),
                                 B(b->token_mask), b->mask_words, B(b->candidate_ids), B(b->candidate_probabilities), B(b->candidate_draws),
                                 B(b->child_uniforms)};
    std::vector<ops::LaneRows> rows;
    std::vector<ops::SamplingPolicy> policies;
    for (uint32_t i = 0; i < count; ++i) { rows.push_back({lanes[i].first, lanes[i].rows}); policies.push_back({policy[i].temperature, policy[i].min_p, policy[i].top_k, policy[i].top_p, policy[i].constrained != 0, policy[i].excludes_stop_tokens != 0}); }
    std::array<uint32_t, SAMPLING_STOP_TOKENS> stops{SAMPLING_NO_TOKEN, SAMPLING_NO_TOKEN, SAMPLING_NO_TOKEN, SAMPLING_NO_TOKEN};
    if (stop_tokens) for (size_t s = 0; s < stops.size(); ++s) stops[s] = stop_tokens[s];
    ops::Sampling::addVerify(capi::graphOf(graph), buffers, vocabulary, logits_stride, rows, policies, stops);
  });
}
sp_status spo_sampling_rebuild_penalty_words(uint32_t *words, uint32_t vocabulary, const uint32_t *history, uint64_t history_tokens,
                                             uint64_t generated_tokens, uint32_t pending_token, uint32_t mark_prompt) {
  return capi::guard([&] {
    capi::require(words && history, "words or history");
    ops::Sampling::rebuildPenaltyWords({words, vocabulary}, {history, size_t(history_tokens)}, generated_tokens,
                                       pending_token == SAMPLING_NO_TOKEN ? std::nullopt : std::optional<uint32_t>(pending_token),
                                       mark_prompt != 0);
  });
}
sp_status spo_sampling_add_penalties(spo_graph *graph, sp_buffer *logits, sp_buffer *words, sp_buffer *input_tokens, sp_buffer *tree_rows,
                                     uint32_t vocabulary, uint32_t logits_stride, const spo_lane_rows *lanes,
                                     const spo_sampling_penalties *penalties, uint32_t count) {
  return capi::guard([&] {
    capi::require(graph && lanes && penalties, "graph, lanes or penalties");
    const capi::PenalizedLanes p = capi::penalizedLanes(lanes, penalties, count);
    ops::SamplingBuffers buffers{};
    buffers.logits = B(logits);
    buffers.inputTokens = B(input_tokens);
    buffers.treeRows = B(tree_rows);
    ops::Sampling::addPenalties(capi::graphOf(graph), buffers, vocabulary, logits_stride, p.rows, p.policies, {B(words), p.tableRows});
  });
}
sp_status spo_sampling_add_penalty_count(spo_graph *graph, sp_buffer *words, sp_buffer *tokens, sp_buffer *retained, uint32_t vocabulary,
                                         const spo_lane_rows *lanes, const spo_sampling_penalties *penalties, uint32_t count) {
  return capi::guard([&] {
    capi::require(graph && lanes && penalties, "graph, lanes or penalties");
    const capi::PenalizedLanes p = capi::penalizedLanes(lanes, penalties, count);
    ops::AcceptanceBuffers buffers{};
    buffers.tokens = B(tokens);
    buffers.retained = B(retained);
    ops::Sampling::addPenaltyCount(capi::graphOf(graph), buffers, vocabulary, p.rows, p.active, {B(words), p.tableRows});
  });
}
sp_status spo_sampling_add_thinking_cutoff(spo_graph *graph, sp_buffer *input_tokens, sp_buffer *tree_rows, sp_buffer *tokens,
                                           sp_buffer *token_mask, uint32_t mask_words, uint32_t vocabulary,
                                           const spo_lane_rows *lanes, const spo_thinking_cutoff *cutoffs, uint32_t count) {
  return capi::guard([&] {
    capi::require(graph && lanes && cutoffs, "graph, lanes or cutoffs");
    std::vector<ops::LaneRows> rows;
    std::vector<ops::SamplingPolicy> policies(count);
    for (uint32_t i = 0; i < count; ++i) {
      rows.push_back({lanes[i].first, lanes[i].rows});
      policies[i].thinkingCutoff = capi::cutoffOf(&cutoffs[i]);
      policies[i].constrained = cutoffs[i].active && cutoffs[i].waits_for_mask;
    }
    ops::SamplingBuffers buffers{};
    buffers.inputTokens = B(input_tokens);
    buffers.treeRows = B(tree_rows);
    buffers.tokens = B(tokens);
    buffers.tokenMask = B(token_mask);
    buffers.maskWords = mask_words;
    ops::Sampling::addThinkingCutoff(capi::graphOf(graph), buffers, vocabulary, rows, policies);
  });
}
sp_status spo_sampling_add_acceptance(spo_graph *graph, sp_buffer *input_tokens, sp_buffer *tree_rows, sp_buffer *tokens,
                                      sp_buffer *retained, sp_buffer *accepted_count, sp_buffer *retained_rows,
                                      const spo_lane_rows *lanes, const uint32_t *remaining, uint32_t count,
                                      const uint32_t stop_tokens[4]) {
  return capi::guard([&] {
    capi::require(graph && lanes && remaining && stop_tokens, "graph, lanes, remaining or stop tokens");
    std::vector<ops::LaneRows> rows;
    std::vector<uint32_t> left;
    for (uint32_t i = 0; i < count; ++i) { rows.push_back({lanes[i].first, lanes[i].rows}); left.push_back(remaining[i]); }
    ops::Sampling::addAcceptance(capi::graphOf(graph), {B(input_tokens), B(tree_rows), B(tokens), B(retained), B(accepted_count), B(retained_rows)},
                                 rows, left, {stop_tokens[0], stop_tokens[1], stop_tokens[2], stop_tokens[3]});
  });
}

sp_status spo_draft_candidate_scratch_bytes(uint32_t lanes, uint32_t columns, uint64_t *bytes) {
  return capi::guard([&] {
    capi::require(bytes, "result");
    *bytes = ops::DraftSelector::candidateScratchBytes(lanes, columns);
  });
}

sp_status spo_draft_add_candidates(spo_graph *graph, sp_buffer *logits, sp_buffer *selector_hidden, sp_buffer *scratch,
                                   sp_buffer *candidates, sp_buffer *unary, sp_buffer *edges, sp_buffer *predecessor_codebook,
                                   sp_buffer *successor_codebook, uint32_t leading, uint32_t trailing, uint32_t vocabulary,
                                   const uint32_t *anchors, uint32_t lanes) {
  return capi::guard([&] {
    capi::require(graph && (anchors || !lanes), "graph or anchors");
    ops::DraftSelector::addCandidates(capi::graphOf(graph), {B(logits), B(selector_hidden), B(scratch), B(candidates), B(unary), B(edges)},
                                      {B(predecessor_codebook), B(successor_codebook)}, {leading, trailing}, vocabulary,
                                      std::span<const uint32_t>(anchors, lanes));
  });
}

sp_status spo_draft_add_tree(spo_graph *graph, sp_buffer *candidates, sp_buffer *unary, sp_buffer *edges, sp_buffer *chain_tokens,
                             sp_buffer *chain_rates, sp_buffer *tree_tokens, sp_buffer *trees, sp_buffer *tree_scores,
                             sp_buffer *tree_sizes, sp_buffer *tree_draws, sp_buffer *tree_next, sp_buffer *tree_caps,
                             const spo_draft_tree_lane *lanes, uint32_t count) {
  return capi::guard([&] {
    capi::require(graph && lanes, "graph or lanes");
    std::vector<ops::DraftTreeLane> list;
    for (uint32_t l = 0; l < count; ++l) {
      ops::DraftTreeLane lane;
      lane.anchor = lanes[l].anchor;
      lane.depth = lanes[l].depth;
      lane.children = lanes[l].children;
      lane.chain = lanes[l].chain;
      lane.slope = lanes[l].slope;
      for (size_t p = 0; p < lane.intercept.size(); ++p) lane.intercept[p] = lanes[l].intercept[p];
      lane.temperature = lanes[l].temperature;
      lane.noise = uint64_t{lanes[l].noise[1]} << 32 | lanes[l].noise[0];
      list.push_back(lane);
    }
    ops::DraftSelector::addTree(capi::graphOf(graph),
                                {B(candidates), B(unary), B(edges), B(chain_tokens), B(chain_rates), B(tree_tokens), B(trees), B(tree_scores),
                                 B(tree_sizes), B(tree_draws), B(tree_next), B(tree_caps)},
                                list);
  });
}

sp_status spo_draft_add_verify_children(spo_graph *graph, sp_buffer *verify_sources, sp_buffer *lane_rows, sp_buffer *tree_rows,
                                        sp_buffer *candidates, sp_buffer *tree_next, sp_buffer *tree_draws, sp_buffer *candidate_ids,
                                        sp_buffer *candidate_probabilities, sp_buffer *candidate_draws, sp_buffer *depths,
                                        uint32_t lanes, uint32_t rows) {
  return capi::guard([&] {
    capi::require(graph, "graph");
    ops::DraftSelector::addVerifyChildren(capi::graphOf(graph),
                                          {B(verify_sources), B(lane_rows), B(tree_rows), B(candidates), B(tree_next), B(tree_draws),
                                           B(candidate_ids), B(candidate_probabilities), B(candidate_draws), B(depths)},
                                          {lanes, rows, SAMPLING_MAXIMUM_ROWS});
  });
}

sp_status spo_draft_add_verify_rows(spo_graph *graph, sp_buffer *tree_tokens, sp_buffer *trees, sp_buffer *tree_scores,
                                    sp_buffer *tree_sizes, sp_buffer *input_tokens, sp_buffer *tree_rows, sp_buffer *lane_rows,
                                    sp_buffer *verify_sources, uint32_t lanes, uint32_t rows, uint32_t lane_cap, float floor) {
  return capi::guard([&] {
    capi::require(graph, "graph");
    ops::DraftSelector::addVerifyRows(capi::graphOf(graph),
                                      {B(tree_tokens), B(trees), B(tree_scores), B(tree_sizes), B(input_tokens), B(tree_rows), B(lane_rows),
                                       B(verify_sources)},
                                      {lanes, rows, lane_cap}, floor);
  });
}

sp_status spo_draft_add_verify_row_slots(spo_graph *graph, sp_buffer *tree_tokens, sp_buffer *trees, sp_buffer *tree_scores,
                                         sp_buffer *tree_sizes, sp_buffer *input_tokens, sp_buffer *tree_rows, sp_buffer *lane_rows,
                                         sp_buffer *verify_sources, uint32_t lanes, uint32_t lane_cap, float floor) {
  return capi::guard([&] {
    capi::require(graph, "graph");
    ops::DraftSelector::addVerifyRows(capi::graphOf(graph),
                                      {B(tree_tokens), B(trees), B(tree_scores), B(tree_sizes), B(input_tokens), B(tree_rows), B(lane_rows),
                                       B(verify_sources)},
                                      {lanes, lanes * lane_cap, lane_cap, true}, floor);
  });
}

sp_status spo_dense_verify_set_staged_prefill(spo_dense_verify *verify, int on) {
  return capi::guard([&] {
    capi::require(verify, "verify");
    verify->verify->setStagedPrefill(on != 0);
  });
}

sp_status spo_dense_verify_set_capture(spo_dense_verify *verify, const uint32_t *layers, uint32_t count, sp_buffer *destination) {
  return capi::guard([&] {
    capi::require(verify && (layers || !count), "verify or layers");
    verify->verify->setCapture(std::vector<uint32_t>(layers, layers + count), B(destination));
  });
}

sp_status spo_dense_verify_create(sp_backend *backend, const spo_dense_dimensions *d, uint32_t max_lanes, uint32_t physical_pages,
                                  uint32_t page_table_entries, spo_dense_verify **out) {
  return spo_dense_verify_create_chunked(backend, d, max_lanes, physical_pages, page_table_entries, 0, out);
}
sp_status spo_dense_verify_create_chunked(sp_backend *backend, const spo_dense_dimensions *d, uint32_t max_lanes, uint32_t physical_pages,
                                          uint32_t page_table_entries, uint32_t prefill_rows, spo_dense_verify **out) {
  return capi::guard([&] {
    capi::require(backend && d && out, "backend, dimensions or result");
    auto holder = std::make_unique<spo_dense_verify>();
    holder->backend = std::make_unique<hip::Backend>(backend);
    model::DenseDimensions dims{d->hidden, d->q_heads, d->kv_heads, d->head_dim, d->ffn, d->vocabulary, d->layers,
                                d->rotary_pairs, d->normalize_heads != 0, d->rope_theta};
    holder->verify = std::make_unique<model::DenseVerify>(*holder->backend, dims, max_lanes, physical_pages, page_table_entries, prefill_rows);
    *out = holder.release();
  });
}
void spo_dense_verify_destroy(spo_dense_verify *verify) { delete verify; }

sp_status spg_dense_dimensions(const spg_file *file, spo_dense_dimensions *out) {
  return capi::guard([&] {
    capi::require(out, "result");
    const model::DenseDimensions d = model::ggufDenseDimensions(capi::ggufOf(file));
    *out = {d.hidden, d.qHeads, d.kvHeads, d.headDimension, d.ffn, d.vocabulary, d.layers, d.rotaryPairs, d.normalizeHeads ? 1u : 0u, d.ropeTheta};
  });
}
sp_status spo_dense_verify_load_gguf(spo_dense_verify *verify, const spg_file *file) {
  return capi::guard([&] {
    capi::require(verify, "verify");
    model::loadGgufDenseWeights(*verify->backend, capi::ggufOf(file), *verify->verify);
  });
}

sp_status spo_dense_verify_set_layer(spo_dense_verify *verify, uint32_t layer, const spo_projection *qkv, const spo_projection *output,
                                     const spo_projection *gate, const spo_projection *up, const spo_projection *down,
                                     sp_buffer *input_norm, sp_buffer *post_norm, sp_buffer *query_norm, sp_buffer *key_norm) {
  return capi::guard([&] {
    capi::require(verify && qkv && output && gate && up && down, "verify or projections");
    model::DenseWeights &w = verify->verify->weights();
    if (layer >= w.layers.size()) throw std::invalid_argument("no such layer");
    w.layers[layer] = {capi::projectionOf(qkv), capi::projectionOf(output), capi::projectionOf(gate), capi::projectionOf(up),
                       capi::projectionOf(down), B(input_norm), B(post_norm), B(query_norm), B(key_norm)};
  });
}
sp_status spo_dense_verify_set_head(spo_dense_verify *verify, uint32_t embedding_format, sp_buffer *embedding_rows,
                                    sp_buffer *final_norm, const spo_projection *head) {
  return capi::guard([&] {
    capi::require(verify && head, "verify or head");
    model::DenseWeights &w = verify->verify->weights();
    const model::DenseDimensions &d = verify->verify->dimensions();
    w.embedding = {B(embedding_rows), embedding_format, d.vocabulary, d.hidden};
    w.finalNorm = B(final_norm);
    w.head = capi::projectionOf(head);
    w.head.destination = ops::FloatOutput::Float32;
  });
}
sp_status spo_dense_verify_buffer(spo_dense_verify *verify, spo_verify_buffer which, uint32_t index, sp_buffer **out) {
  return capi::guard([&] {
    capi::require(verify && out, "verify or result");
    model::DenseVerify &v = *verify->verify;
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
    case SPO_VERIFY_QKV_ROWS: b = v.qkvRows(); break;
    case SPO_VERIFY_ATTENTION_ROWS: b = v.attentionRows(); break;
    case SPO_VERIFY_FFN_ROWS: b = v.ffnRows(); break;
    case SPO_VERIFY_CANDIDATE_CHILDREN: b = v.candidateChildren(index); break;
    case SPO_VERIFY_PENALTY_WORDS: b = v.penaltyWords(); break;
    case SPO_VERIFY_TOKEN_MASK: b = v.tokenMask(); break;
    default: throw std::invalid_argument("no such verify buffer");
    }
    sp_buffer_retain(b.handle());
    *out = b.handle();
  });
}
sp_status spo_verify_check_results(const spo_lane_rows *lanes, const uint32_t *remaining, uint32_t count, uint32_t step_rows,
                                   uint32_t vocabulary, const uint32_t *tokens, const uint32_t *retained, const uint32_t *accepted,
                                   const uint32_t *retained_rows) {
  return capi::guard([&] {
    capi::require(lanes && count && tokens && retained && accepted && retained_rows, "lanes or results");
    std::vector<model::StepLane> list;
    std::vector<model::StepLaneResult> results;
    for (uint32_t i = 0; i < count; ++i) {
      list.push_back({lanes[i].first, lanes[i].rows, remaining ? remaining[i] : 0xFFFFFFFFu});
      if (uint64_t{lanes[i].first} + lanes[i].rows > step_rows) throw hip::BackendError("lane " + std::to_string(i) + ": its rows are not rows of the step");
      results.push_back({retained[i], accepted[i], retained_rows[i], tokens + lanes[i].first});
    }
    model::validateStepResults(list, results, step_rows, vocabulary);
  });
}
sp_status spo_dense_verify_results(spo_dense_verify *verify, const spo_verify_lane *lanes, uint32_t count, uint32_t *tokens,
                                   uint32_t *retained, uint32_t *accepted, uint32_t *retained_rows) {
  return capi::guard([&] {
    capi::require(verify && tokens && retained && accepted && retained_rows, "verify or results");
    model::DenseVerify &v = *verify->verify;
    std::vector<model::StepLane> list;
    uint32_t first = 0;
    for (const model::VerifyLane &l : lanesOf(lanes, count)) { list.push_back({first, l.rows, l.remaining}); first += l.rows; }
    if (v.takeChainStatus()) throw hip::BackendError("a chained projection's wait for the one before it gave up: the step's results are void");
    model::readStepResults(list, v.tokens(), v.retained(), v.acceptedCount(), v.retainedRows(), v.dimensions().vocabulary, tokens, retained,
                           accepted, retained_rows);
  });
}
sp_status spo_dense_verify_encode_prefill(spo_dense_verify *verify, spo_graph *graph, uint32_t table_first, uint32_t committed,
                                          uint32_t tokens) {
  return capi::guard([&] {
    capi::require(verify && graph, "verify or graph");
    verify->verify->encodePrefill(capi::graphOf(graph), table_first, committed, tokens);
  });
}
sp_status spo_dense_verify_set_penalties(spo_dense_verify *verify, uint32_t lane, float repetition, float presence, float frequency) {
  return capi::guard([&] {
    capi::require(verify, "verify");
    verify->verify->setPenalties(lane, {repetition, presence, frequency});
  });
}
sp_status spo_dense_verify_set_admission(spo_dense_verify *verify, uint32_t lane, uint32_t constrained, uint32_t excludes_stop_tokens) {
  return capi::guard([&] {
    capi::require(verify, "verify");
    verify->verify->setAdmission(lane, constrained != 0, excludes_stop_tokens != 0);
  });
}
sp_status spo_dense_verify_set_stop_tokens(spo_dense_verify *verify, const uint32_t *stop_tokens) {
  return capi::guard([&] {
    capi::require(verify, "verify");
    std::array<uint32_t, SAMPLING_STOP_TOKENS> stops{SAMPLING_NO_TOKEN, SAMPLING_NO_TOKEN, SAMPLING_NO_TOKEN, SAMPLING_NO_TOKEN};
    if (stop_tokens) for (size_t i = 0; i < stops.size(); ++i) stops[i] = stop_tokens[i];
    verify->verify->setStopTokens(stops);
  });
}
sp_status spo_dense_verify_set_thinking_cutoff(spo_dense_verify *verify, uint32_t lane, const spo_thinking_cutoff *cutoff) {
  return capi::guard([&] {
    capi::require(verify, "verify");
    verify->verify->setThinkingCutoff(lane, capi::cutoffOf(cutoff));
  });
}
sp_status spo_dense_verify_set_test_children(spo_dense_verify *verify, int on) {
  return capi::guard([&] {
    capi::require(verify, "verify");
    verify->verify->setTestChildren(on != 0);
  });
}
sp_status spo_dense_verify_chain_status(spo_dense_verify *verify, uint32_t *status) {
  return capi::guard([&] {
    capi::require(verify && status, "verify or status");
    *status = verify->verify->takeChainStatus();
  });
}
sp_status spo_dense_verify_set_chained(spo_dense_verify *verify, int chained) {
  return capi::guard([&] {
    capi::require(verify, "verify");
    verify->verify->setChained(chained != 0);
  });
}
sp_status spo_dense_verify_set_fused_prepare(spo_dense_verify *verify, int fused) {
  return capi::guard([&] {
    capi::require(verify, "verify");
    verify->verify->setFusedPrepare(fused != 0);
  });
}
uint64_t spo_dense_verify_page_bytes(const spo_dense_verify *verify) { return verify ? verify->verify->pageBytes() : 0; }
uint64_t spo_dense_verify_step_bytes(const spo_dense_verify *verify, const spo_verify_lane *lanes, uint32_t count) {
  uint64_t bytes = 0;
  capi::guard([&] { capi::require(verify, "verify"); bytes = verify->verify->stepBytes(lanesOf(lanes, count)); });
  return bytes;
}
sp_status spo_dense_verify_encode(spo_dense_verify *verify, spo_graph *graph, const spo_verify_lane *lanes, uint32_t count, int commit) {
  return capi::guard([&] {
    capi::require(verify && graph, "verify or graph");
    verify->verify->encode(capi::graphOf(graph), lanesOf(lanes, count), commit != 0);
  });
}
sp_status spo_dense_verify_encode_part(spo_dense_verify *verify, spo_graph *graph, uint32_t part, uint32_t index,
                                       const spo_verify_lane *lanes, uint32_t count) {
  return capi::guard([&] {
    capi::require(verify && graph, "verify or graph");
    const std::vector<model::VerifyLane> list = lanesOf(lanes, count);
    uint32_t rows = 0;
    for (const model::VerifyLane &l : list) rows += l.rows;
    if (part == 0) verify->verify->encodeEmbedding(capi::graphOf(graph), rows);
    else if (part == 1) verify->verify->encodeLayer(capi::graphOf(graph), index, planOf(*verify->verify, list), rows);
    else if (part == 2) verify->verify->encodeHead(capi::graphOf(graph), rows);
    else throw std::invalid_argument("no such part of the step");
  });
}

} // extern "C"

struct spo_lookup_index {
  splash::model::LookupIndex index;
};
sp_status spo_lookup_index_create(spo_lookup_index **out) {
  return capi::guard([&] {
    capi::require(out, "result");
    *out = new spo_lookup_index{};
  });
}
void spo_lookup_index_destroy(spo_lookup_index *index) { delete index; }
sp_status spo_lookup_index_append(spo_lookup_index *index, const uint32_t *tokens, uint64_t count) {
  return capi::guard([&] {
    capi::require(index && (tokens || !count), "index or tokens");
    if (index->index.tokens().size() + count > UINT32_MAX / 2) throw std::invalid_argument("a lookup index holds fewer than 2^31 tokens");
    index->index.append({tokens, size_t(count)});
  });
}
sp_status spo_lookup_index_match(const spo_lookup_index *index, uint32_t *length, uint32_t *end) {
  return capi::guard([&] {
    capi::require(index && length && end, "index or results");
    *length = index->index.match().length;
    *end = index->index.match().end;
  });
}
uint32_t spo_lookup_index_proposals(const spo_lookup_index *index, uint32_t count, uint32_t *out) {
  if (!index || !out) return 0;
  const std::span<const uint32_t> proposals = index->index.proposals(count);
  std::copy(proposals.begin(), proposals.end(), out);
  return uint32_t(proposals.size());
}
uint32_t spo_lookup_agreement(uint32_t token, uint32_t depth, const uint32_t *candidates, uint32_t positions, uint32_t per_position) {
  if (!candidates) return uint32_t(splash::model::LookupAgreement::Unknown);
  return uint32_t(splash::model::lookupAgreement(token, depth, {candidates, size_t{positions} * per_position}, per_position));
}
