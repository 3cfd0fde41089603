/* splash_ops.h -- flat C entry points of the verify step's C++ operators (splash::ops::*), for
 * hosts that bind through an FFI (the Python tests and bench of this repository, a cgo/JNI stub).
 * Each function wraps one method of an operator that keeps the reference's name and argument
 * meaning; the reference method is cited beside it. A std::invalid_argument of an operator comes
 * back as SP_INVALID_ARGUMENT with its message in sp_last_error(), thrown -- as in the reference --
 * before any dispatch is added to the graph.
 */
#ifndef SPLASH_OPS_H
#define SPLASH_OPS_H

#include "splash_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct spo_graph spo_graph;           /* metal::CommandGraph (runtime/metal/CommandGraph.hpp:26) */
typedef struct spo_projection spo_projection; /* ops::Projection (runtime/ops/Weights.hpp:170) */
typedef struct spo_linear spo_linear;         /* ops::Linear (runtime/ops/Linear.hpp:289) */

/* ---- CommandGraph ---- */
sp_status spo_graph_create(spo_graph **out);
void spo_graph_destroy(spo_graph *graph);
uint32_t spo_graph_size(const spo_graph *graph);
/* The kernel name of dispatch `index`; returns the bytes needed. */
size_t spo_graph_kernel(const spo_graph *graph, uint32_t index, char *out, size_t capacity);
/* CommandGraph::add (CommandGraph.hpp:44-54): a raw dispatch with a parameter struct. */
sp_status spo_graph_add(spo_graph *graph, const char *kernel, sp_buffer *const *buffers, uint32_t buffer_count,
                        const void *params, uint32_t params_bytes, const uint32_t grid[3], const uint32_t block[3]);
/* MetalBackend::submitCommandAsync(graph.dispatches()) (MetalBackend.hpp:490-491). */
sp_status spo_graph_submit(sp_backend *backend, const spo_graph *graph, sp_ticket **out);
/* The graph recorded for replay (sp_command_create). */
sp_status spo_graph_record(sp_backend *backend, const spo_graph *graph, sp_command **out);

/* ---- prompt lookup (model::LookupIndex, runtime/model/LookupProposals.hpp:17-105): host code ----
 * A request's tokens (its prompt, then every token its decode selects) and, after the latest, the match: the longest
 * suffix, counted up to 64 tokens and none shorter than 3, that also ends at an earlier token, at its most recent such
 * end. The tokens that followed it there are the lane's host chain (spo_draft_tree_lane.chain_tokens). */
typedef struct spo_lookup_index spo_lookup_index;
sp_status spo_lookup_index_create(spo_lookup_index **out);
void spo_lookup_index_destroy(spo_lookup_index *index);
sp_status spo_lookup_index_append(spo_lookup_index *index, const uint32_t *tokens, uint64_t count);
/* length 0: no match; end: the index of the earlier occurrence's last token. */
sp_status spo_lookup_index_match(const spo_lookup_index *index, uint32_t *length, uint32_t *end);
/* Up to `count` tokens that followed the match, at most as far as the latest token, into `out`; returns how many. */
uint32_t spo_lookup_index_proposals(const spo_lookup_index *index, uint32_t count, uint32_t *out);
/* LookupAgreement of a lookup token `depth` positions past the anchor with the draft's candidates (per_position a
 * position, most likely first, `positions` positions): 0 the most likely, 1 another candidate, 2 none, 3 not known. */
uint32_t spo_lookup_agreement(uint32_t token, uint32_t depth, const uint32_t *candidates, uint32_t positions, uint32_t per_position);

/* ---- weight image (load-time repack: runtime/model/GgufPreparation.cpp, gguf_repack.metal) ---- */
uint64_t spo_gguf_image_bytes(uint32_t format, uint32_t rows, uint32_t input_size);
uint64_t spo_gguf_table_bytes(uint32_t input_size, uint32_t rows);
sp_status spo_gguf_pack_image(uint32_t format, const uint8_t *native, uint32_t rows, uint32_t input_size, uint8_t *image);
sp_status spo_gguf_unpack_image(uint32_t format, const uint8_t *image, uint32_t rows, uint32_t input_size, uint8_t *native);
/* ggml types read through another format's blocks of the same values, bit for bit: Q3_K (ggml type 11) as Q6_K, Q4_0
 * (2) and Q5_0 (6) as Q8_0. spo_gguf_rewrite_format gives that format (0xFFFFFFFF for a type with no rewrite) and
 * spo_gguf_rewrite writes `super_blocks` times 256 values of `source` as that format's native blocks, which
 * spo_gguf_pack_image then takes; the GGUF loader does both by itself. (The reference runs these through kernels of their
 * own formats: runtime/metal/abi/QuantFormat.h GGUF_FMT_Q3K, _Q40, _Q50; the values are GGML's dequantize_row_* either way.) */
uint32_t spo_gguf_rewrite_format(uint32_t ggml_type);
sp_status spo_gguf_rewrite(uint32_t ggml_type, const uint8_t *source, uint64_t super_blocks, uint8_t *out);
/* The image's fp32 values [rows][input_size] (the reference's gguf_dequant_test.metal kernel). */
sp_status spo_gguf_add_dequant(spo_graph *graph, uint32_t format, sp_buffer *image, sp_buffer *out, uint32_t rows,
                               uint32_t input_size);

/* ---- Projection (Weights.hpp:170-186): segments tile the leading output columns in order. Segments may differ
 *      in format, as the reference's fused q|k|v takes a format per segment (gguf_linear.metal:237-261,
 *      LinearGguf.cpp:78-96): such a projection runs as one dispatch of a kernel that holds every format, under a
 *      plain bf16 plan (no epilogue, whole_groups 0), each segment a multiple of 64 columns. ---- */
sp_status spo_projection_create(uint32_t segments, const uint32_t *formats, const uint32_t *output_sizes,
                                uint32_t input_size, sp_buffer *const *images, int float32_destination,
                                spo_projection **out);
/* Projection::rows (Weights.hpp:193-204): a view of a projection of one tensor over one or two ranges of its rows, whole
 * 16-row tiles, which become its output columns in order; slices of the same image, no copy. The draft's vocabulary head
 * over a subset of the tokens (DraftVocabulary::rows, DraftSelector.hpp:108-112: rows [0, leading) and [trailing, V)). */
sp_status spo_projection_rows(const spo_projection *projection, const uint32_t *firsts, const uint32_t *counts, uint32_t ranges,
                              spo_projection **out);
void spo_projection_destroy(spo_projection *projection);
uint64_t spo_projection_weight_bytes(const spo_projection *projection);

/* ---- Linear ---- */
/* ops::Linear::Linear(device, ...) (Linear.hpp:291): plans follow the device the backend opened. */
sp_status spo_linear_create(sp_backend *backend, spo_linear **out);
/* A Linear of a given calibration (KernelCalibration), for CPU tests and sweeps. */
sp_status spo_linear_create_calibrated(uint32_t compute_units, uint32_t groups_per_unit, uint32_t minimum_blocks_per_wave,
                                       spo_linear **out);
void spo_linear_destroy(spo_linear *linear);
/* LinearEpilogue (Linear.hpp:77): 0 None, 1 Residual, 2 GateUp. */
typedef struct spo_linear_plan {
  uint32_t rows, epilogue;
  uint32_t splits, whole_groups; /* LinearConfig: K partitions, and the leading workgroups that take K whole */
  uint32_t storage_rows;    /* LinearPlan::storageRows */
  uint32_t float32;         /* LinearPlan::destination */
  /* LinearTile: 0 the register rule (exact 128 + code operands, one fp32 multiply-add a group;
   * linear_gguf_sgmatrix.metal:140-288), 1 the staged rule (weights decoded with fp32 group coefficients and rounded
   * once to half, products accumulated in fp32; kernels/common/gguf_staged.h:12-66, gguf_linear.metal:120-140): plain
   * and residual plans of one format, set with spo_linear_plan_with; 2 the column rule (LinearTile::GgufColumn,
   * kernels/common/gguf_column_tile.h:25-68, kernels/decode/linear_gguf_column.metal:33-66; LinearGguf.cpp:141-147): one
   * or two rows, unsplit, half weights and every addition in the reference's order, so the results are the reference's bit
   * for bit; plain, residual and one-pass gate/up plans, a dispatch a tensor over the rows as they are. */
  uint32_t tile, reserved;
  uint64_t scratch_input, scratch_partials, scratch_counters; /* LinearPlan::scratchSize */
} spo_linear_plan;
/* Linear::plan(projection, rows, epilogue) (Linear.hpp:307-309): the device's plan. */
sp_status spo_linear_plan_for(const spo_linear *linear, const spo_projection *projection, uint32_t rows, uint32_t epilogue,
                              spo_linear_plan *out);
/* Linear::plan(workload, config, destination) (Linear.hpp:327-328): the plan of a given configuration;
 * fills storage_rows and scratch sizes from rows, epilogue, splits, whole_groups, float32. */
sp_status spo_linear_plan_with(const spo_projection *projection, spo_linear_plan *plan);
/* Linear::add (Linear.hpp:330-332). table/partials/counters are the LinearScratch; `prepared`
 * nonzero says the table already holds `input` (PreparedInput): 1 the table of the rows themselves, 2 the
 * table a residual + norm plan wrote, whose rows still lack their inverse RMS (this projection applies it
 * to its sums). gate only for a GateUp plan. */
sp_status spo_linear_add(const spo_linear *linear, spo_graph *graph, const spo_projection *projection,
                         const spo_projection *gate, const spo_linear_plan *plan, sp_buffer *input, sp_buffer *output,
                         sp_buffer *residual, sp_buffer *table, sp_buffer *partials, sp_buffer *counters, int prepared);
/* Linear::add of a plan whose epilogue is 3 (residual + norm): output = bf16(residual + W input), and those rows
 * as the activation table of the projection that follows their RMS norm under norm_weight (bf16 [output size]),
 * in next_table (spo_gguf_table_bytes(output size, rows) bytes, not `table`): no norm dispatch runs between the
 * two projections. The table holds bf16(output * norm_weight) and the sums of squares of the output rows; the
 * projection that reads it (`prepared` 2) multiplies its sums by each row's inverse RMS, so its results differ from
 * those of a norm pass, which rounds bf16(output * inverse RMS * norm_weight), by the rounding of that one bf16
 * operand. One tensor, whole super-blocks of output columns. */
sp_status spo_linear_add_residual_norm(const spo_linear *linear, spo_graph *graph, const spo_projection *projection,
                                       const spo_linear_plan *plan, sp_buffer *input, sp_buffer *output, sp_buffer *residual,
                                       sp_buffer *norm_weight, sp_buffer *next_table, sp_buffer *table, sp_buffer *partials,
                                       sp_buffer *counters, int prepared);
/* Linear::addSwiGlu (Linear.hpp:352-354): output = residual + down(silu(gate x) * up x).
 * next_table (optional, spo_gguf_table_bytes(ffn, rows) bytes, not `table`): the gate/up pass
 * then writes the down projection's activation table from its epilogue and no separate table
 * pass is recorded; results are bit-identical either way. */
sp_status spo_linear_add_swiglu(const spo_linear *linear, spo_graph *graph, const spo_projection *gate,
                                const spo_projection *up, const spo_projection *down, sp_buffer *normalized,
                                sp_buffer *intermediate, sp_buffer *residual, sp_buffer *output, uint32_t rows,
                                sp_buffer *table, sp_buffer *partials, sp_buffer *counters, sp_buffer *next_table);
/* Linear::addChain: up to four projections of up to 64 rows as ONE dispatch, each reading what the one before it wrote
 * (the table its epilogue leaves in next_table, the residual rows), in place of the reference's one dispatch a
 * projection with a kernel boundary between them (QwenTarget.cpp:457-496 encodes a layer's projections one after the
 * other): the next link's workgroups fetch their first weights while the link before drains and wait for its count of
 * finished workgroups. A link is what spo_linear_add / spo_linear_add_residual_norm take: a plain plan (epilogue 0), a
 * gate/up plan with next_table (2), or a residual + norm plan (3); `prepared` is 1 or 2 for every link (its table
 * exists or the link before writes it); every link's table, partials and counters are its own, and no table is written
 * that an earlier link of the chain read. `progress`: SPO_CHAIN_PROGRESS_BYTES bytes the chain owns, zero before its
 * first dispatch; the word at SPO_CHAIN_STATUS_OFFSET reads nonzero after a dispatch in which a workgroup's bounded
 * wait gave up (then the results are not to be used, and the caller zeroes the buffer). Results equal those of the
 * links dispatched one by one, bit for bit. */
#define SPO_CHAIN_LINKS 4u
#define SPO_CHAIN_PROGRESS_BYTES 65792u
#define SPO_CHAIN_STATUS_OFFSET 16u
typedef struct spo_chain_link {
  const spo_projection *projection, *gate;
  spo_linear_plan plan;
  sp_buffer *input, *output, *residual, *norm_weight, *next_table, *table, *partials, *counters;
  int32_t prepared;
  uint32_t reserved;
} spo_chain_link;
sp_status spo_linear_add_chain(const spo_linear *linear, spo_graph *graph, const spo_chain_link *links, uint32_t count,
                               sp_buffer *progress);
/* Linear::add (Linear.hpp:330-332) of one link's buffers, as a dispatch of its own: every field of LinearBuffers, so
 * also a gate/up plan that writes the next projection's table (next_table) outside Linear::addSwiGlu. */
sp_status spo_linear_add_link(const spo_linear *linear, spo_graph *graph, const spo_chain_link *link);
/* KernelCalibration::chainSpinLimit: the polls (about a microsecond each) a chained projection's workgroup waits for the
 * link before it, of chains added from now on. 0 makes every wait that finds the count short give up at once, which is
 * how a host tests the failure path without a kernel that does not end. */
sp_status spo_linear_set_chain_spin_limit(spo_linear *linear, uint32_t polls);
/* Linear::addPrefill: a chunk of 1 to 16384 rows (a prompt's) through the projection under the staged rule, a workgroup
 * 128 rows x 128 columns with K whole: the counterpart of the reference's prefill tile (LinearTile::GgufPrefill,
 * gguf_linear.metal:79-118, Linear.hpp:330-332 with a prefill plan). output = bf16 (fp32 for a projection created so)
 * of input x W^T, plus the bf16 residual rows when `residual` is not NULL. Every tensor of the projection holds a
 * multiple of 128 columns. `table`: spo_linear_prefill_table_bytes(input size, rows) bytes of the rows' activation
 * tables, which the dispatches write first. */
uint64_t spo_linear_prefill_table_bytes(uint32_t input_size, uint32_t rows);
sp_status spo_linear_add_prefill(spo_graph *graph, const spo_projection *projection, sp_buffer *input, sp_buffer *output,
                                 sp_buffer *residual, sp_buffer *table, uint32_t rows);
/* Linear::scratchSize (Linear.hpp:319): of every plan of up to `rows` rows of the matrix. */
sp_status spo_linear_scratch_size(const spo_linear *linear, uint32_t output_size, uint32_t input_size, uint32_t rows,
                                  uint64_t *table, uint64_t *partials, uint64_t *counters);

/* ---- PagedAttention (runtime/ops/PagedAttention.hpp:259-366) ---- */
typedef struct spo_attention_plan spo_attention_plan; /* ops::AttentionPlan (PagedAttention.hpp:179-234) */
typedef struct spo_attention_geometry {
  uint32_t q_heads, kv_heads, head_dim;
  uint32_t rotary_pairs; /* RoPE pairs (i, i + pairs) */
  uint32_t normalize;    /* RMS-norm q and k heads */
  uint32_t gated;        /* the projection row holds each query head's queries, then its gate; the output rows
                            are multiplied by the gates' sigmoids (kernels/common/attention_gate.h:19-44) */
  uint32_t int8_queries; /* the block's queries score as INT8 codes with a scale per head and row, exactly in int32
                            (the "q8q" kernels, PagedAttention.cpp:380-383); 0: as the bf16 rows */
} spo_attention_geometry;
typedef struct spo_attention_rows { /* one sequence: ops::AttentionRows / AttentionHistory */
  uint32_t first_row, rows, committed, table_first;
} spo_attention_rows;
/* kv::Layout::bytesPerLayerPage (runtime/ops/PagedKv.hpp:155-260) at 256-token pages, fp16 scales. */
uint64_t spo_kv_page_bytes(uint32_t kv_heads, uint32_t head_dim);
/* Element offsets of the page layout, for hosts that fill or read pages (abi/KvExtent.h:23-111). */
uint64_t spo_kv_key_index(uint32_t head, uint32_t token, uint32_t dim, uint32_t head_dim);
uint64_t spo_kv_value_index(uint32_t head, uint32_t token, uint32_t dim, uint32_t head_dim);
/* PagedAttention::plan (PagedAttention.cpp:351-389). */
sp_status spo_attention_plan_create(const spo_attention_geometry *geometry, const spo_attention_rows *sequences,
                                    uint32_t count, spo_attention_plan **out);
void spo_attention_plan_destroy(spo_attention_plan *plan);
uint32_t spo_attention_plan_splits(const spo_attention_plan *plan);
/* PagedAttention::workspace: bytes of the staged queries, their sums, the split partials, their sums. */
sp_status spo_attention_workspace(const spo_attention_plan *plan, uint64_t sizes[4]);
/* PagedAttention::addProjection (PagedAttention.cpp:441-464). */
sp_status spo_attention_add_projection(spo_graph *graph, const spo_attention_plan *plan, sp_buffer *qkv,
                                       sp_buffer *query_norm, sp_buffer *key_norm, sp_buffer *rope_cos,
                                       sp_buffer *rope_sin, sp_buffer *queries, sp_buffer *query_sums,
                                       sp_buffer *page_table, sp_buffer *pool, uint64_t page_bytes);
/* The block's q|k|v projection and spo_attention_add_projection's work as ONE dispatch, where the reference runs the
 * projection and its prepare kernel one after the other (QwenTarget.cpp:457-470, PagedAttention.cpp:441-464): the
 * workgroup that completes a head's columns norms, rotates, stages or stores it. `qkv` is what spo_linear_add_link
 * takes (a plain bf16 plan; its output is the block's packed rows); its partials hold plan.splits x
 * (output size / 64) x storage_rows x 256 bytes and its counters 4 bytes a 64 columns, whatever the plan's parts. The
 * packed rows, staged queries, their sums and the cache bytes equal those of the two dispatches bit for bit.
 * spo_attention_fuses_projection: 1 when the kernels take the pair (up to 64 rows, every workgroup one part of K,
 * heads of 64 or 128 dimensions whole in the projection's tensors, fp16 queries, no gates), else 0. */
int spo_attention_fuses_projection(const spo_attention_plan *plan, const spo_projection *projection, const spo_linear_plan *linear_plan);
sp_status spo_attention_add_fused_projection(const spo_linear *linear, spo_graph *graph, const spo_chain_link *qkv,
                                             const spo_attention_plan *plan, sp_buffer *query_norm, sp_buffer *key_norm,
                                             sp_buffer *rope_cos, sp_buffer *rope_sin, sp_buffer *queries,
                                             sp_buffer *query_sums, sp_buffer *page_table, sp_buffer *pool, uint64_t page_bytes);
/* PagedAttention::addAttention (PagedAttention.cpp:466-607): split, then ordered reduce.
 * output_table (optional, spo_gguf_table_bytes(q_heads * head_dim, rows) bytes): the reduce also
 * writes the rows as the activation table of the projection that follows. packed_qkv: the rows'
 * projection, which holds the gates of a gated geometry (NULL otherwise). */
sp_status spo_attention_add_attention(spo_graph *graph, const spo_attention_plan *plan, sp_buffer *queries,
                                      sp_buffer *query_sums, sp_buffer *partials, sp_buffer *partial_sums,
                                      sp_buffer *tree_rows, sp_buffer *page_table, sp_buffer *pool, uint64_t page_bytes,
                                      sp_buffer *output, sp_buffer *output_table, sp_buffer *packed_qkv);
/* Prompt chunks: the plan over kv::ChunkedPrefillParams (PagedAttention.hpp:28-39, :270-275; PagedAttention.cpp:351-389).
 * A chunk is `tokens` rows (1 to 2048, SPLASH_PREFILL_TOKEN_BUDGET) of one sequence at positions from `committed`,
 * attending causally; it runs as tiles of 16 rows, eight tiles a dispatch, each tile's history split by its own length
 * alone, so a row's result is bit for bit the one its tile gives as a verify block. The workspace holds the staged
 * queries of every tile and the partials of the largest dispatch. add_chunk_projection stores every row's K and V
 * before add_chunk_attention lets any row attend; buffers as the single-dispatch calls', over all the chunks' rows
 * (tree_rows: a chain a tile; output_table: the one table of all the rows). */
typedef struct spo_attention_chunk_plan spo_attention_chunk_plan;
typedef struct spo_attention_chunk { uint32_t first_row, tokens, committed, table_first; } spo_attention_chunk;
sp_status spo_attention_chunk_plan_create(const spo_attention_geometry *geometry, const spo_attention_chunk *chunks, uint32_t count,
                                          spo_attention_chunk_plan **out);
void spo_attention_chunk_plan_destroy(spo_attention_chunk_plan *plan);
uint32_t spo_attention_chunk_plan_dispatches(const spo_attention_chunk_plan *plan);
sp_status spo_attention_chunk_workspace(const spo_attention_chunk_plan *plan, uint64_t sizes[4]);
sp_status spo_attention_add_chunk_projection(spo_graph *graph, const spo_attention_chunk_plan *plan, sp_buffer *qkv,
                                             sp_buffer *query_norm, sp_buffer *key_norm, sp_buffer *rope_cos, sp_buffer *rope_sin,
                                             sp_buffer *queries, sp_buffer *query_sums, sp_buffer *page_table, sp_buffer *pool,
                                             uint64_t page_bytes);
sp_status spo_attention_add_chunk_attention(spo_graph *graph, const spo_attention_chunk_plan *plan, sp_buffer *queries,
                                            sp_buffer *query_sums, sp_buffer *partials, sp_buffer *partial_sums,
                                            sp_buffer *tree_rows, sp_buffer *page_table, sp_buffer *pool, uint64_t page_bytes,
                                            sp_buffer *output, sp_buffer *output_table, sp_buffer *packed_qkv);
/* PagedAttention::addPathCommit (PagedAttention.cpp:647-667). */
sp_status spo_attention_add_path_commit(spo_graph *graph, const spo_attention_plan *plan, sp_buffer *retained,
                                        sp_buffer *page_table, sp_buffer *pool, uint64_t page_bytes);

/* ---- Normalization, Embedding, RoPE (runtime/ops/Normalization.cpp:16-40, Embedding.cpp:20-47, RoPE.hpp:33-37) ---- */
sp_status spo_norm_add_rms(spo_graph *graph, sp_buffer *input, sp_buffer *weight, sp_buffer *output, uint32_t width,
                           uint32_t rows);
/* The norm that also writes the projection activation table of its rows (norm_rms_table16_decode). */
sp_status spo_norm_add_rms_table(spo_graph *graph, sp_buffer *input, sp_buffer *weight, sp_buffer *output,
                                 sp_buffer *table, uint32_t width, uint32_t rows);
sp_status spo_embedding_add(spo_graph *graph, uint32_t format, sp_buffer *native_rows, uint32_t vocabulary,
                            uint32_t hidden, sp_buffer *tokens, sp_buffer *output, uint32_t rows);
/* RowCopy::add (runtime/ops/RowCopy.hpp:9-28): `rows` rows of `width` bf16 values from row from_row of `source`
 * (rows from_stride values apart, from value from_column on) to the like region of `destination`. */
sp_status spo_row_copy_add(spo_graph *graph, sp_buffer *source, uint32_t from_row, uint32_t from_stride, uint32_t from_column,
                           sp_buffer *destination, uint32_t to_row, uint32_t to_stride, uint32_t to_column, uint32_t rows,
                           uint32_t width);
/* The fp32 projection of weights kept as rows (addGgufFloat, LinearGguf.cpp:545-612; kernels/shared/gguf_float.metal): a
 * MoE router, or the GDN alpha/beta gates of a GGUF that keeps them F32. weight_rows: [output_size][input_size] F32, or
 * BF16 with bf16_weights; input: bf16 [rows][input_size], input_size a multiple of 8; output row r's columns
 * [out_offset, out_offset + output_size) of out_stride values, fp32 with float32_output, else rounded to bf16. Every
 * operand is exact in fp32; a sum's order is fixed (four chains by k mod 4, then (c0 + c1) + (c2 + c3)), so a row's
 * result depends on no other row. */
sp_status spo_float_projection_add(spo_graph *graph, sp_buffer *input, sp_buffer *weight_rows, uint32_t output_size,
                                   uint32_t input_size, uint32_t bf16_weights, sp_buffer *output, uint32_t rows,
                                   uint32_t out_stride, uint32_t out_offset, uint32_t float32_output);
typedef struct spo_rope_sequence { uint32_t first_row, rows, anchor; } spo_rope_sequence;
sp_status spo_rope_add_tree_tables(spo_graph *graph, sp_buffer *inverse_frequency, sp_buffer *depth, sp_buffer *cosines,
                                   sp_buffer *sines, uint32_t pairs, const spo_rope_sequence *sequences, uint32_t count);

/* ---- GDN (runtime/ops/GDN.hpp:16-203, GDN.cpp:225-330): the verify step of Gated DeltaNet layers ---- */
typedef struct spo_gdn_shape { /* ops::GdnShape (GDN.hpp:16-36); head dimension 128 */
  uint32_t key_heads, value_heads;
  uint32_t convolution_dimension; /* (2 key_heads + value_heads) * 128 */
  uint32_t packed_width;          /* [q | k | v | z | b | a] */
  uint32_t sigmoid_gate;
} spo_gdn_shape;
typedef struct spo_gdn_state_strides { /* ops::GdnStateStrides (GDN.hpp:63-73), fp32 recurrent states */
  uint64_t convolution_layer_bytes, recurrent_layer_bytes, convolution_state_bytes;
} spo_gdn_state_strides;
/* The strides and size of a state cell of `layers` layers, and one layer's tape bytes of one lane's
 * step (gdnTapeLayerBytes, GDN.hpp:120). Any of the results may be NULL. */
sp_status spo_gdn_layout(const spo_gdn_shape *shape, uint32_t layers, spo_gdn_state_strides *strides, uint64_t *cell_bytes,
                         uint64_t *tape_layer_bytes);
typedef struct spo_gdn_lane { /* ops::GdnTapeLane + SplashLaneRows + the lane's cells */
  uint32_t first_row, rows;
  uint32_t pending_path; /* rows of the lane's previous step it accepted and its state does not hold yet */
  uint32_t reserved;
  uint64_t pending_tape, step_tape;   /* byte offsets of this layer's tapes in the tape buffer */
  uint64_t current_cell, next_cell;   /* byte offsets of the lane's cells in the states buffer */
} spo_gdn_lane;
typedef struct spo_gdn_decode_buffers { /* ops::GdnDecodeBuffers (GDN.hpp:122-152) */
  sp_buffer *packed, *convolution_weights, *states, *tape, *decay_weights, *time_bias, *mixer_norm, *hidden;
  uint32_t float_norm; /* the output norm's weights are fp32 */
  sp_buffer *tree_rows; /* the step's rows' places in their blocks (SplashTreeRow, 8 bytes a row) */
  sp_buffer *hidden_table; /* optional (NULL: none): the hidden rows also as the activation table of the projection that
                              reads them, spo_gguf_table_bytes(value_heads * 128, rows) bytes; that projection is added
                              with `prepared` 1 and no table pass runs before it */
} spo_gdn_decode_buffers;
/* GDN::addDecode (GDN.hpp:184): the step of 1 to 8 lanes of one layer. The state a step writes is
 * the one BEFORE its rows (the lane's pending path folded in); its rows go to the lane's tape.
 * Every row, of a chain as of any other tree, reads the state before the block along its own path
 * (GDN.hpp:143-147), and every row's convolution reads its path's tokens. */
sp_status spo_gdn_add_decode(spo_graph *graph, const spo_gdn_decode_buffers *buffers, const spo_gdn_shape *shape, uint32_t layer,
                             const spo_gdn_state_strides *state, uint32_t tiled_heads, const spo_gdn_lane *lanes, uint32_t count);
/* GDN::addFold (GDN.hpp:198): the state after the first `rows` rows of the path a lane retained of a
 * step (retained_rows[0]), every layer, written to fold_cell exactly as the lane's next step would
 * hold it; nothing when the path holds fewer rows. */
sp_status spo_gdn_add_fold(spo_graph *graph, sp_buffer *states, sp_buffer *tape, sp_buffer *retained_rows, uint64_t step_tape,
                           uint64_t state_cell, uint64_t fold_cell, const spo_gdn_shape *shape, uint32_t layers, uint32_t rows,
                           const spo_gdn_state_strides *state);
typedef struct spo_gdn_prefill_buffers { /* ops::GdnPrefillBuffers (GDN.hpp:75-93) */
  sp_buffer *packed, *convolution_weights, *states, *decay_weights, *time_bias, *mixer_norm;
  uint32_t float_norm; /* the output norm's weights are fp32 */
  uint32_t reserved;
  sp_buffer *queries, *keys;    /* bf16 [tokens][key_heads * 128], written by the prepare pass */
  sp_buffer *values;            /* bf16 [tokens][value_heads * 128] */
  sp_buffer *decay, *beta;      /* fp32 and bf16 [tokens][value_heads] */
  sp_buffer *recurrent_rows;    /* bf16 [tokens][value_heads * 128]: the scan's rows before the gated norm */
  sp_buffer *hidden;            /* bf16 [tokens][value_heads * 128] */
  uint64_t current_cell, next_cell; /* byte offsets in the states buffer: the cell the chunk starts from, the one it leaves */
} spo_gdn_prefill_buffers;
typedef struct spo_gdn_prefill_capture { /* ops::GdnPrefillCapture (GDN.hpp:95-104): the cell after the chunk's first `tokens` rows */
  uint32_t tokens, reserved;
  uint64_t cell;
} spo_gdn_prefill_capture;
/* GDN::addPrefill (GDN.hpp:166-181, GDN.cpp:132-222): a prompt chunk of `tokens` rows of one lane and layer, every row
 * entering the state: a prepare and a scan dispatch for each run between captures (ascending, inside the rows; a run
 * continues from the cell the run before wrote, and no run writes the cell it reads), then one gate dispatch over all
 * rows. The cells hold, bit for bit, what the same rows leave when they enter as accepted verify blocks. */
sp_status spo_gdn_add_prefill(spo_graph *graph, const spo_gdn_prefill_buffers *buffers, const spo_gdn_shape *shape, uint32_t layer,
                              uint32_t tokens, const spo_gdn_state_strides *state, uint32_t tiled_heads,
                              const spo_gdn_prefill_capture *captures, uint32_t count);

/* ---- StateCodec (runtime/ops/StateCodec.hpp:11-49; runtime/metal/abi/StateCodec.h): the cached form of the
 *      recurrent layers, int8 codes row by row and then a bf16 scale per block of 32 values ---- */
typedef struct spo_state_codec_shape { /* ops::StateCodecShape (StateCodec.hpp:17-34) */
  uint32_t layers, rows, columns; /* a layer's value rows (every value head's) of `columns` values, a multiple of 32 */
  uint32_t bf16_state;            /* the running state holds bf16 values (GdnStateFormat::BFloat16), else fp32 */
  uint64_t state_layer_bytes, codes_layer_bytes; /* between consecutive layers of the running and of the cached state */
} spo_state_codec_shape;
/* state_codec_layer_bytes (abi/StateCodec.h:31-33): a cached layer's bytes. */
uint64_t spo_state_codec_layer_bytes(uint32_t rows, uint32_t columns);
/* StateCodec::addQuantize / addDequantize / addCopy (StateCodec.hpp:41-48); the buffers start at the first layer. */
sp_status spo_state_codec_add_quantize(spo_graph *graph, sp_buffer *state, sp_buffer *codes, const spo_state_codec_shape *shape);
sp_status spo_state_codec_add_dequantize(spo_graph *graph, sp_buffer *codes, sp_buffer *state, const spo_state_codec_shape *shape);
sp_status spo_state_codec_add_copy(spo_graph *graph, sp_buffer *from, sp_buffer *to, const spo_state_codec_shape *shape);

/* ---- MoE (runtime/ops/MoE.hpp:403-410, MoE.cpp:143-287; runtime/metal/abi/MoE.h:23-245) ---- */
typedef struct spo_moe_shape {
  uint32_t hidden, ffn, experts, top_k;
  /* The shared expert (MoE.hpp:50-63): shared_slices experts of the routed experts' width that every row visits after
   * its routed ones, ids experts .. experts + shared_slices - 1, their images after the routed experts' in the same
   * buffers; shared_gate: each weighs sigmoid(row . scalar gate), else 1. */
  uint32_t shared_slices, shared_gate;
  uint32_t sigmoid_router; /* MoeRouter::SigmoidNormalized (moe.metal:21, :104-110) instead of the softmax of the selected scores */
  uint32_t reserved;
} spo_moe_shape;
typedef struct spo_moe_workspace { /* in the order of spo_moe_workspace_sizes */
  sp_buffer *selected, *weights, *route_slot, *slot_row, *tile_expert, *tile_rows, *tile_total, *tables, *next_tables,
      *intermediate, *expert_output;
} spo_moe_workspace;
/* Bytes of each workspace buffer for a step of `rows` rows (1..256). */
sp_status spo_moe_workspace_sizes(const spo_moe_shape *shape, uint32_t rows, uint64_t sizes[11]);
/* MoE::addRouting (MoE.cpp:143-206): from fp32 router scores [rows][score_stride], each row's top_k
 * experts by (score descending, id ascending) in selected, their weights exp2((s_r - s_0) log2 e) / sum
 * in rank order, and the routes grouped by expert into tiles of up to 16 rows. */
sp_status spo_moe_add_routing(spo_graph *graph, sp_buffer *scores, uint32_t score_stride, const spo_moe_workspace *workspace,
                              const spo_moe_shape *shape, uint32_t rows, sp_buffer *input, sp_buffer *shared_scalar_gate);
/* MoE::addRouted (MoE.cpp:242-287): output = bf16(residual + sum over a row's routes, in rank order, of
 * weight * down_e(silu(gate_e x) * up_e x)). *_images hold every expert's re-tiled image of the tensor,
 * expert e at e * spo_gguf_image_bytes(format, rows of the tensor, its inputs). */
sp_status spo_moe_add_routed(spo_graph *graph, sp_buffer *normalized, sp_buffer *residual, sp_buffer *output, sp_buffer *gate_images,
                             sp_buffer *up_images, sp_buffer *down_images, uint32_t format, uint32_t down_format,
                             const spo_moe_workspace *workspace, const spo_moe_shape *shape, uint32_t rows);
/* The same, and the output rows also leave as the activation table (spo_gguf_table_bytes(hidden, rows) bytes) of the
 * projection after their RMS norm under norm_weight (bf16 [hidden]), as spo_linear_add_residual_norm writes it: that
 * projection is added with `prepared` = 2 and no norm dispatch runs before it. hidden a multiple of 256. */
sp_status spo_moe_add_routed_norm(spo_graph *graph, sp_buffer *normalized, sp_buffer *residual, sp_buffer *output,
                                  sp_buffer *gate_images, sp_buffer *up_images, sp_buffer *down_images, uint32_t format,
                                  uint32_t down_format, const spo_moe_workspace *workspace, const spo_moe_shape *shape,
                                  uint32_t rows, sp_buffer *norm_weight, sp_buffer *next_table);

/* ---- Sampling (runtime/ops/Sampling.hpp:64-254, Sampling.cpp:283-357) ---- */
typedef struct spo_lane_rows { uint32_t first, rows; } spo_lane_rows; /* SplashLaneRows */
/* Sampling::workspace: bytes of the argmax partial values and indices, the masses, ranges, decisions. */
sp_status spo_sampling_workspace(uint32_t rows, uint64_t sizes[5]);
typedef struct spo_sampling_buffers {
  sp_buffer *logits, *tokens, *partial_values, *partial_indices;
  sp_buffer *draft_probabilities, *uniforms, *masses, *ranges, *decisions, *input_tokens, *tree_rows; /* sampled lanes */
  sp_buffer *token_mask; /* constrained lanes: uint32 [rows][mask_words], bit t % 32 of word t / 32 of a row admits token t */
  uint32_t mask_words;
  /* A tree block's sampled rows (the reference's DrawChildren, sampling.metal:680-690; NULL for blocks whose rows have
   * one child tested against a full-vocabulary draft distribution): each row's sixteen candidates -- uint32 ids and fp32
   * draft probabilities [rows][16] --, the candidate indices of the children its draft drew in the order drawn (bytes
   * [rows][4], 0xFF past them) and a uniform for each child's test (fp32 [rows][4]). With these the sampled lanes' rows
   * run recursive rejection sampling over their children (sampling.metal:697-880); draft_probabilities is not read. */
  sp_buffer *candidate_ids, *candidate_probabilities, *candidate_draws, *child_uniforms;
} spo_sampling_buffers;
/* ops::SamplingPolicy (Sampling.hpp:56-83): temperature 0 is greedy; a sampling lane keeps the tokens that
 * weigh at least min_p of its heaviest (0: all), then the top_k most likely of those (0: all), then their
 * top_p nucleus (1: all). */
typedef struct spo_sampling_policy {
  float temperature, min_p;
  uint32_t top_k;
  float top_p;
  uint32_t constrained;          /* the lane's rows admit only the tokens of their token_mask rows */
  uint32_t excludes_stop_tokens; /* the lane never selects a stop token */
} spo_sampling_policy;
/* Sampling::addVerify (Sampling.cpp:283-328). The logits rows of a constrained or stop-excluding lane are rewritten
 * first, -infinity at the tokens the lane does not admit (TargetRow::admits, sampling.metal:42-46).
 * stop_tokens: four ids, 0xFFFFFFFF for none; NULL for none at all. */
sp_status spo_sampling_add_verify(spo_graph *graph, const spo_sampling_buffers *buffers, uint32_t vocabulary,
                                  uint32_t logits_stride, const spo_lane_rows *lanes, const spo_sampling_policy *policies,
                                  uint32_t count, const uint32_t *stop_tokens);
/* The sampling penalties (ops::SamplingPenalties and PenaltyTable, Sampling.hpp:17-30, :85-91): repetition scales the
 * logit of every token the prompt or the output holds (a positive logit is divided, another multiplied), presence and
 * frequency lower that of every token the output holds by presence + frequency x count; 1, 0, 0 change nothing.
 * table_row: the lane's row of the penalty table, `vocabulary` words a row in device memory: bit 31 marks a prompt
 * token, the other bits count how often the target selected the token (abi/Sampling.h:120-125). */
typedef struct spo_sampling_penalties {
  float repetition, presence, frequency;
  uint32_t table_row;
} spo_sampling_penalties;
/* Sampling::rebuildPenaltyWords (Sampling.cpp:91-114): a request's row of the table, in host memory (upload it to the
 * row), from its history: the prompt, then the generated_tokens outputs it emitted; pending_token (0xFFFFFFFF: none) is
 * counted too; mark_prompt sets the prompt bit of the prompt's tokens (only repetition reads it). SP_INVALID_ARGUMENT
 * for a token past the vocabulary or a history with no prompt. */
sp_status spo_sampling_rebuild_penalty_words(uint32_t *words, uint32_t vocabulary, const uint32_t *history, uint64_t history_tokens,
                                             uint64_t generated_tokens, uint32_t pending_token, uint32_t mark_prompt);
/* Sampling::addPenalties (Sampling.cpp:163-180; its addVerify runs it first): the logits rows of every lane whose
 * penalties are active are rewritten in place, before spo_sampling_add_verify reads them. A row's context adds, to
 * the table's counts, the block's draft tokens (input_tokens) on the row's path (tree_rows), the anchor's excepted.
 * Dispatches nothing when no lane's penalties are active. */
sp_status spo_sampling_add_penalties(spo_graph *graph, sp_buffer *logits, sp_buffer *words, sp_buffer *input_tokens, sp_buffer *tree_rows,
                                     uint32_t vocabulary, uint32_t logits_stride, const spo_lane_rows *lanes,
                                     const spo_sampling_penalties *penalties, uint32_t count);
/* Sampling::countPenaltyTokens (Sampling.cpp:116-121), on the device: the tokens each penalized lane retained of the
 * step (spo_sampling_add_acceptance's tokens and retained counts) are counted into its row of the table, so the
 * next step's penalties see them without a host round trip. */
sp_status spo_sampling_add_penalty_count(spo_graph *graph, sp_buffer *words, sp_buffer *tokens, sp_buffer *retained, uint32_t vocabulary,
                                         const spo_lane_rows *lanes, const spo_sampling_penalties *penalties, uint32_t count);
/* ops::ThinkingCutoff of a lane's policy (Sampling.hpp:30-55): the lane's selected rows of depth `row` on take the
 * `count` tokens of `end` in order (as many as the block holds) unless a draft token on a row's path up to that depth is
 * the last of `end` or `also_ends` (0xFFFFFFFF: none), which ended thinking first; with waits_for_mask the end starts,
 * along each path, at the first row from depth `row` on whose constraint-mask row admits end[0]. active 0: no cutoff. */
typedef struct spo_thinking_cutoff {
  uint32_t active, row, count;
  uint32_t end[16];
  uint32_t also_ends, waits_for_mask;
} spo_thinking_cutoff;
/* The end of Sampling::addSelection (Sampling.cpp:314-327): rewrites the selections spo_sampling_add_verify left in
 * `tokens`, before spo_sampling_add_acceptance walks them. token_mask (uint32 [rows][mask_words]) is read only for lanes
 * whose end waits for their mask; NULL otherwise. Dispatches nothing when no lane's cutoff lies inside its block. */
sp_status spo_sampling_add_thinking_cutoff(spo_graph *graph, sp_buffer *input_tokens, sp_buffer *tree_rows, sp_buffer *tokens,
                                           sp_buffer *token_mask, uint32_t mask_words, uint32_t vocabulary,
                                           const spo_lane_rows *lanes, const spo_thinking_cutoff *cutoffs, uint32_t count);
/* Sampling::addAcceptance (Sampling.cpp:330-357). */
sp_status spo_sampling_add_acceptance(spo_graph *graph, sp_buffer *input_tokens, sp_buffer *tree_rows, sp_buffer *tokens,
                                      sp_buffer *retained, sp_buffer *accepted_count, sp_buffer *retained_rows,
                                      const spo_lane_rows *lanes, const uint32_t *remaining, uint32_t count,
                                      const uint32_t stop_tokens[4]);
/* No counterpart in the reference. For callers that cannot allocate device memory or a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the greedy selection of spo_sampling_add_verify --
 * every row's largest logit, the lower id among equals, NaN and -infinity never, 0xFFFFFFFF for a row with no
 * selectable logit -- launched directly on `stream` (a hipStream_t; NULL is the null stream) over device pointers:
 * logits fp32 [rows][logits_stride], tokens uint32 [rows]. The shards' partial results live in a device array of the
 * library (64 KiB a GPU, held until the process ends) instead of a workspace argument: the call allocates nothing,
 * frees nothing and returns once its two kernels are launched. At most SPO_SAMPLING_STATIC_MAXIMUM_ROWS rows a call
 * (more is SP_INVALID_ARGUMENT). Every call on one GPU shares that GPU's array: calls that overlap on one GPU
 * (different streams, or threads) race; calls in stream order on one stream do not. A GPU's FIRST call looks the
 * array's address up (hipGetSymbolAddress, under a mutex; it may load the code object), which is not a call to make
 * under stream capture: make one call per GPU outside any capture first (any row count, e.g. at start-up); every
 * later call on that GPU is two kernel launches and nothing else. */
#define SPO_SAMPLING_STATIC_MAXIMUM_ROWS 256u
sp_status spo_sampling_greedy_rows_static(const float *logits, uint32_t rows, uint32_t vocabulary, uint32_t logits_stride,
                                          uint32_t *tokens, void *stream);

/* ---- DraftSelector::addVerifyRows (runtime/ops/DraftSelector.hpp:139-147; StepRows, LaneRows.hpp:49-67): a decode
 *      step's rows from the trees a draft selector grew. Each lane's tree holds tree_sizes[lane] rows of 16 (tokens,
 *      SplashTreeRow rows, fp32 pairs of draft probability and estimate), best first; the step takes every lane's
 *      anchor and the best other rows by estimate that `rows` and `lane_cap` hold, none estimated below `floor`,
 *      numbers each lane's in preorder and writes their tokens, tree rows, lane rows {first, rows} and sources (the
 *      tree row each is; 0xFFFFFFFF for the rows past the lanes', which belong to no lane). ---- */
/* The first two kernels of DraftSelector::add (runtime/ops/DraftSelector.cpp:37-140; draft_select_top16_sharded and
 * draft_select_edges, runtime/metal/kernels/decode/sampling.metal:1099-1356): of each of a lane's 7 proposal positions
 * (rows 1-7 of its 8 query rows of `logits`, fp32 [lanes * 8][columns], columns = leading + vocabulary - trailing) the 16
 * tokens of the largest logits, the larger first and among equal ones the smaller column (`candidates` uint32
 * [lanes * 7][16], `unary` their logits; 0xFFFFFFFF and -inf where the columns run out), and `edges` fp32
 * [lanes * 7][16][16]: [predecessor][candidate] the sum over the selector's rank of 256 of predecessor_codebook[token
 * of the position before, anchors[lane] at position 0 (row 0 alone)] x selector_hidden[row] x successor_codebook[token],
 * bf16 factors, fp32 sums. Codebooks bf16 [vocabulary][256]; selector_hidden bf16 [lanes * 8][256]; `scratch` of
 * spo_draft_candidate_scratch_bytes. Up to 524288 columns. */
sp_status spo_draft_candidate_scratch_bytes(uint32_t lanes, uint32_t columns, uint64_t *bytes);
sp_status spo_draft_add_candidates(spo_graph *graph, sp_buffer *logits, sp_buffer *selector_hidden, sp_buffer *scratch,
                                   sp_buffer *candidates, sp_buffer *unary, sp_buffer *edges, sp_buffer *predecessor_codebook,
                                   sp_buffer *successor_codebook, uint32_t leading, uint32_t trailing, uint32_t vocabulary,
                                   const uint32_t *anchors, uint32_t lanes);
/* The third kernel of DraftSelector::add (DraftSelector.cpp:96-118; draft_select_tree, sampling.metal:1357-1766, its
 * rule in abi/Sampling.h:209-255): each lane's tree over those candidates and edges, best first by the estimate that the
 * target accepts the path to a row, up to 16 rows a lane, as spo_draft_add_verify_rows and the sampled rows of a verify
 * step (spo_sampling_buffers' candidate fields: a row's next-position probabilities and drawn children) read them.
 * chain_tokens uint32 [lanes][15] and chain_rates fp32 [lanes][15][4] hold each lane's host chain (its rate by its
 * agreement with the draft at its depth: the draft's likeliest, another candidate, none, past the draft's positions);
 * tree_draws bytes [lanes][16][4], tree_next fp32 [lanes][16][16], tree_caps fp32 [lanes][16]. */
typedef struct spo_draft_tree_lane {
  uint32_t anchor, depth, children, chain; /* depth < 16, children 1..4, chain <= 15 */
  float slope, intercept[7], temperature;  /* estimate = sigmoid(slope * logit(q) + intercept[position]); temperature 0: greedy */
  uint32_t noise[2];                        /* the 64-bit seed of a sampled lane's draws, low word first */
} spo_draft_tree_lane;
sp_status spo_draft_add_tree(spo_graph *graph, sp_buffer *candidates, sp_buffer *unary, sp_buffer *edges, sp_buffer *chain_tokens,
                             sp_buffer *chain_rates, sp_buffer *tree_tokens, sp_buffer *trees, sp_buffer *tree_scores,
                             sp_buffer *tree_sizes, sp_buffer *tree_draws, sp_buffer *tree_next, sp_buffer *tree_caps,
                             const spo_draft_tree_lane *lanes, uint32_t count);
/* The step's side of the trees, row by row of the step (no counterpart kernel in the reference, whose sampled selection
 * reads the trees through verify_sources itself, sampling.metal:697-780): for every row the candidates of its next
 * position (candidate_ids uint32 [rows][16], candidate_probabilities fp32 [rows][16]) and the children its draft drew
 * (candidate_draws bytes [rows][4], 0xFF past them) -- spo_sampling_buffers' candidate fields -- and its depth (depths
 * uint32 [rows], what the RoPE tables take), from verify_sources, lane_rows and tree_rows as spo_draft_add_verify_rows
 * wrote them and candidates, tree_next and tree_draws of the trees. */
sp_status spo_draft_add_verify_children(spo_graph *graph, sp_buffer *verify_sources, sp_buffer *lane_rows, sp_buffer *tree_rows,
                                        sp_buffer *candidates, sp_buffer *tree_next, sp_buffer *tree_draws, sp_buffer *candidate_ids,
                                        sp_buffer *candidate_probabilities, sp_buffer *candidate_draws, sp_buffer *depths,
                                        uint32_t lanes, uint32_t rows);
sp_status spo_draft_add_verify_rows(spo_graph *graph, sp_buffer *tree_tokens, sp_buffer *trees, sp_buffer *tree_scores,
                                    sp_buffer *tree_sizes, sp_buffer *input_tokens, sp_buffer *tree_rows, sp_buffer *lane_rows,
                                    sp_buffer *verify_sources, uint32_t lanes, uint32_t rows, uint32_t lane_cap, float floor);
/* The same layout in slots (no counterpart in the reference, whose kernels read each lane's rows from the device,
 * SplashLaneRows, where a step's lanes here are fixed when its graph is recorded): lane l's rows are rows l * lane_cap on,
 * its anchor and the best rows of its tree at or above the floor, up to lane_cap; the rest of its slot are inert rows
 * (token 0xFFFFFFFF, whose embedding is zero and which no row selects; on no path but their own; a child of the anchor
 * that never follows it; no source). A step recorded once for lane_cap rows a lane then takes trees of any size the
 * device grows: lane_rows[l] is {l * lane_cap, the rows the lane took}. */
sp_status spo_draft_add_verify_row_slots(spo_graph *graph, sp_buffer *tree_tokens, sp_buffer *trees, sp_buffer *tree_scores,
                                         sp_buffer *tree_sizes, sp_buffer *input_tokens, sp_buffer *tree_rows, sp_buffer *lane_rows,
                                         sp_buffer *verify_sources, uint32_t lanes, uint32_t lane_cap, float floor);

/* ---- ops::DraftAttention (runtime/ops/DraftAttention.hpp:12-152, DraftAttention.cpp:85-309; kernels/decode/draft.metal,
 *      kernels/prefill/draft_context.metal): the attention block of the draft model that proposes a step's rows. The
 *      compiled shape: 32 query heads over 8 KV heads of 128 dimensions (a q|k|v row 6144 values, an attention row 4096),
 *      8 query rows a lane, up to 8 lanes, over a hidden state of `hidden` values (a whole number of 16-channel
 *      convolution groups). A lane's ring of a layer: keys bf16 [8 KV heads][2048 slots][128], values bf16 [8][128][2048],
 *      position p in slot p % 2048, each 4 MiB, `keys[l]` / `values[l]` bytes into the bound rings buffer (where the
 *      reference binds a buffer a lane, DraftAttention.hpp:80-89). ---- */
/* DraftAttentionPlan::workspace(): sizes[0..4] = convolution rows, q|k|v rows, grouped queries with the splits'
 * partials behind them, query keys, query values. */
sp_status spo_draft_attention_workspace(uint32_t hidden, uint32_t lanes, uint64_t sizes[5]);
/* DraftAttention::addConvolution: a stage of a dynamic convolution over each lane's eight rows (finish: the stage
 * after the attention or MLP, which adds the residual). dynamic bf16 [lanes * 8][4 * hidden / 16]: [stage][tap][group];
 * weights bf16 [stage][tap][hidden]. out = in * (w[tap 0] + dyn[tap 0]) + in[row - 1] * (w[tap 1] + dyn[tap 1]) (+ residual). */
sp_status spo_draft_attention_add_convolution(spo_graph *graph, sp_buffer *input, sp_buffer *dynamic, sp_buffer *weights, sp_buffer *residual,
                                              sp_buffer *output, uint32_t hidden, uint32_t lanes, uint32_t finish);
/* DraftAttention::addPrepare: head norms and RoPE of the rows' queries (grouped [lane][query head][8][128]) and keys
 * (query_keys [lane][KV head][8][128]), values transposed (query_values [lane][KV head][128][8]). rope_cos / rope_sin
 * fp32 [lane][16][64]: a lane's rows take the first eight of its sixteen RoPE rows. */
sp_status spo_draft_attention_add_prepare(spo_graph *graph, sp_buffer *qkv, sp_buffer *grouped_queries, sp_buffer *query_norm,
                                          sp_buffer *key_norm, sp_buffer *rope_cos, sp_buffer *rope_sin, sp_buffer *query_keys,
                                          sp_buffer *query_values, uint32_t hidden, uint32_t lanes);
/* DraftAttention::addDecode: each row r of a lane at position cache_lengths[l] + r attends to the ring's positions of
 * its window of 2048 and to all eight current rows; the rows leave in the grouped queries' place as
 * [lane][row][query head][128], the output projection's input. */
sp_status spo_draft_attention_add_decode(spo_graph *graph, sp_buffer *grouped_queries, sp_buffer *rings, const uint64_t *keys,
                                         const uint64_t *values, sp_buffer *query_keys, sp_buffer *query_values,
                                         const uint32_t *cache_lengths, uint32_t hidden, uint32_t lanes);
/* DraftAttention::addContextPrefill: `tokens` context rows (bf16 [tokens][1024 keys | 1024 values]) of one lane into
 * the slots of positions start_position on: keys head-normalized, weighed by key_norm and turned by RoPE row r,
 * values copied. */
sp_status spo_draft_attention_add_context_prefill(spo_graph *graph, sp_buffer *context_kv, sp_buffer *key_norm, sp_buffer *rope_cos,
                                                  sp_buffer *rope_sin, sp_buffer *rings, uint64_t keys, uint64_t values, uint32_t tokens,
                                                  uint32_t start_position, uint32_t hidden);
/* DraftAttention::addContextCommit: each lane's retained rows of a step (retained_rows uint32 [lanes], the masks
 * acceptance wrote; lane_rows {first, rows} [lanes], which the step's proposer wrote) into its rings: the path's i-th
 * row at position start_positions[l] + i, turned by the lane's RoPE row i. A step of `rows` rows, `lane_cap` a lane at most. */
sp_status spo_draft_attention_add_context_commit(spo_graph *graph, sp_buffer *context_kv, sp_buffer *key_norm, sp_buffer *rope_cos,
                                                 sp_buffer *rope_sin, sp_buffer *rings, const uint64_t *keys, const uint64_t *values,
                                                 sp_buffer *retained_rows, sp_buffer *lane_rows, const uint32_t *start_positions,
                                                 uint32_t lanes, uint32_t rows, uint32_t lane_cap, uint32_t hidden);
/* The context window (DraftAttention.hpp:117-151): per ring slot the context row of `width` values in 4-bit codes over
 * groups of 64 with an fp16 scale and minimum each: all slots' codes, then the (scale, minimum) pairs. Store, commit
 * (the rows one lane retained, as the context commit picks them) and load. */
sp_status spo_draft_context_window_bytes(uint32_t width, uint64_t *bytes);
sp_status spo_draft_attention_add_window_store(spo_graph *graph, sp_buffer *context, sp_buffer *window, uint32_t rows, uint32_t start_position,
                                               uint32_t width);
sp_status spo_draft_attention_add_window_commit(spo_graph *graph, sp_buffer *context, sp_buffer *window, sp_buffer *retained,
                                                sp_buffer *lane_rows, uint32_t context_rows, uint32_t rows, uint32_t start_position,
                                                uint32_t width);
sp_status spo_draft_attention_add_window_load(spo_graph *graph, sp_buffer *window, sp_buffer *context, uint32_t rows, uint32_t start_position,
                                              uint32_t width);
/* Embedding::addDraftMaskRows (runtime/ops/Embedding.cpp:49-58): rows 1..7 of each lane's eight input rows take the mask row. */
sp_status spo_draft_attention_add_mask_rows(spo_graph *graph, sp_buffer *mask, sp_buffer *rows, uint32_t width, uint32_t lanes);

/* ---- model::DFlashDraft (runtime/model/DFlashDraft.hpp:66-356, DFlashDraft.cpp:184-430): the draft model that proposes a
 *      step's rows. Per lane eight query rows (the anchor token's embedding in row 0, the mask embedding in rows 1..7)
 *      through `layers` layers of norm -> dynamic convolution -> q|k|v -> attention over the lane's rings -> output ->
 *      convolution with the residual -> norm -> dynamic convolution -> SwiGLU -> down -> convolution with the residual;
 *      then the final norm, the target's vocabulary head (fp32 logits; of the whole vocabulary, or of a subset of the
 *      tokens when `head` is a view of the head's rows, spo_projection_rows: the reference's subsetRows, DFlashDraft.cpp:44-52,
 *      the logits rows then holding the view's columns) and the selector's
 *      projection, as spo_draft_add_candidates reads them. The context side turns the target's captured hidden rows
 *      (target_layers layers' rows concatenated) into each layer's ring keys and values and the 4-bit window. The handle
 *      owns the step's buffers and the state of max_lanes lanes (lane l of a call uses state l); projections may be of any
 *      image format (the reference's draft quantizes in groups of 64 columns, a loader's concern). ---- */
typedef struct spo_dflash_draft spo_dflash_draft;
typedef struct spo_dflash_layout {
  uint32_t layers, hidden, vocabulary, intermediate, target_layers;
} spo_dflash_layout;
typedef struct spo_dflash_layer {   /* DFlashDraftLayerWeights (DFlashDraft.hpp:195-209) */
  const spo_projection *attention_dynamic, *qkv, *output, *mlp_dynamic, *gate, *up, *down;
  sp_buffer *input_norm, *attention_convolution, *query_norm, *key_norm, *post_attention_norm, *mlp_convolution;
} spo_dflash_layer;
/* context_rows: the most rows a context call takes (at least a step's 16 a lane, at most 256). */
sp_status spo_dflash_draft_create(sp_backend *backend, const spo_dflash_layout *layout, uint32_t max_lanes, uint32_t context_rows,
                                  spo_dflash_draft **out);
void spo_dflash_draft_destroy(spo_dflash_draft *draft);
sp_status spo_dflash_draft_set_layer(spo_dflash_draft *draft, uint32_t layer, const spo_dflash_layer *weights);
/* DFlashDraftWeights' model section (DFlashDraft.hpp:211-224) and the target's head; mask_embedding may be null. */
sp_status spo_dflash_draft_set_model(spo_dflash_draft *draft, const spo_projection *context_projection, sp_buffer *hidden_norm,
                                     sp_buffer *final_norm, const spo_projection *selector, sp_buffer *mask_embedding,
                                     const spo_projection *head);
/* The draft's buffers; each call returns a new reference (release it). SPO_DFLASH_HIDDEN index 0 holds the step's input
 * rows [lanes * 8][hidden] (the caller writes row 0 of each lane); ROPE_COS / ROPE_SIN fp32 [lane][16][64], a lane's rows at
 * positions cache length + r; RINGS lane l's rings from l * layers * 8 MiB on (layer i's keys, then its values);
 * WINDOWS lane l's window; CAPTURED_TARGET_HIDDEN bf16 [rows][target_layers * hidden] and CONTEXT_ROPE_* fp32 [rows][64]
 * (a prompt's rows one each; a step's [lane][16][64]) are the context calls' inputs. */
typedef enum spo_dflash_buffer {
  SPO_DFLASH_HIDDEN = 0, SPO_DFLASH_LOGITS, SPO_DFLASH_SELECTOR_HIDDEN, SPO_DFLASH_FINAL_HIDDEN, SPO_DFLASH_ROPE_COS, SPO_DFLASH_ROPE_SIN,
  SPO_DFLASH_RINGS, SPO_DFLASH_WINDOWS, SPO_DFLASH_CAPTURED_TARGET_HIDDEN, SPO_DFLASH_CONTEXT_ROPE_COS, SPO_DFLASH_CONTEXT_ROPE_SIN,
  SPO_DFLASH_CONTEXT_HIDDEN
} spo_dflash_buffer;
sp_status spo_dflash_draft_buffer(spo_dflash_draft *draft, spo_dflash_buffer which, uint32_t index, sp_buffer **out);
/* DFlashDraft::addMaskRows and ::addDecode (DFlashDraft.cpp:274-380): the forward pass of `lanes` lanes, lane l's rows at
 * positions cache_lengths[l] on. */
sp_status spo_dflash_draft_encode_decode(spo_dflash_draft *draft, spo_graph *graph, const uint32_t *cache_lengths, uint32_t lanes);
/* DFlashDraft::addContextPrefill (DFlashDraft.cpp:184-213): `rows` prompt rows of lane `lane` at positions start_position on
 * into its window and rings; rebuild: ::addContextRebuild (:215-229), the rings from the window's rows instead. */
sp_status spo_dflash_draft_encode_context_prefill(spo_dflash_draft *draft, spo_graph *graph, uint32_t lane, uint32_t rows,
                                                  uint32_t start_position, int rebuild);
/* DFlashDraft::addContextCommit (DFlashDraft.cpp:382-430): the rows each lane retained of a verify step of `rows` rows
 * (retained_rows uint32 [lanes], lane_rows {first, rows} [lanes], both on the device), the path's i-th at
 * start_positions[l] + i. */
sp_status spo_dflash_draft_encode_context_commit(spo_dflash_draft *draft, spo_graph *graph, sp_buffer *retained_rows, sp_buffer *lane_rows,
                                                 const uint32_t *start_positions, uint32_t lanes, uint32_t rows, uint32_t lane_cap);

/* ---- The dense verify step (the reference's model layer: QwenTarget.cpp:206-395, :457-496;
 *      Runtime.cpp:2677-2717, :2883-2892) ---- */
typedef struct spo_dense_verify spo_dense_verify;
typedef struct spo_dense_dimensions {
  uint32_t hidden, q_heads, kv_heads, head_dim, ffn, vocabulary, layers, rotary_pairs, normalize_heads;
  float rope_theta;
} spo_dense_dimensions;
typedef struct spo_verify_lane {
  uint32_t rows, committed, table_first;
  float temperature;  /* 0: greedy */
  uint32_t remaining; /* tokens the lane may still keep */
  float min_p;        /* as spo_sampling_policy; all zero keeps every token */
  uint32_t top_k;
  float top_p;        /* 0 is read as 1 */
} spo_verify_lane;
sp_status spo_dense_verify_create(sp_backend *backend, const spo_dense_dimensions *dimensions, uint32_t max_lanes,
                                  uint32_t physical_pages, uint32_t page_table_entries, spo_dense_verify **out);
/* The same with room for prompt chunks of up to prefill_rows rows (spo_dense_verify_encode_prefill; 0: a step's most,
 * 16 x max_lanes; at most 2048, SPLASH_PREFILL_TOKEN_BUDGET): the rows' buffers (input tokens, tree rows, depths, hidden
 * rows, q|k|v and attention rows) are sized for it. */
sp_status spo_dense_verify_create_chunked(sp_backend *backend, const spo_dense_dimensions *dimensions, uint32_t max_lanes,
                                          uint32_t physical_pages, uint32_t page_table_entries, uint32_t prefill_rows,
                                          spo_dense_verify **out);
void spo_dense_verify_destroy(spo_dense_verify *verify);
sp_status spo_dense_verify_set_layer(spo_dense_verify *verify, uint32_t layer, const spo_projection *qkv,
                                     const spo_projection *output, const spo_projection *gate, const spo_projection *up,
                                     const spo_projection *down, sp_buffer *input_norm, sp_buffer *post_norm,
                                     sp_buffer *query_norm, sp_buffer *key_norm);
sp_status spo_dense_verify_set_head(spo_dense_verify *verify, uint32_t embedding_format, sp_buffer *embedding_rows,
                                    sp_buffer *final_norm, const spo_projection *head);
/* DenseVerify::setStagedPrefill: a prompt chunk of more rows than a step's runs its projections through the prefill tile
 * (spo_linear_add_prefill: the staged rule, as the reference's prompt chunks do, LinearTile::GgufPrefill), its norms and
 * SwiGLU as passes of their own; off by default (the chunk then equals its blocks run as steps bit for bit). Needs a
 * driver created with prefill_rows and tensors of whole 128-column workgroups. */
sp_status spo_dense_verify_set_staged_prefill(spo_dense_verify *verify, int on);
/* The hidden rows a draft's context is computed from (QwenTarget's addCapture over RowCopy, runtime/ops/RowCopy.hpp:17-28):
 * after layer layers[i] (ascending) every row's output goes to columns [i * hidden, (i + 1) * hidden) of its row of
 * destination, bf16 [rows][count * hidden], in a step and in a prompt chunk alike; what spo_dflash_draft's context calls
 * read (SPO_DFLASH_CAPTURED_TARGET_HIDDEN may be bound here directly). count 0 captures nothing. */
sp_status spo_dense_verify_set_capture(spo_dense_verify *verify, const uint32_t *layers, uint32_t count, sp_buffer *destination);
/* The step's buffers; each call returns a new reference (release it). `index` is the layer for KV pools and the
   stream (0 or 1) for the hidden rows. The last three hold what the layer that ran last left in them: its fused
   q|k|v rows before the head norms, its attention rows before the output projection, its SwiGLU rows before the
   down projection (what a layer-by-layer check of the step reads). */
typedef enum spo_verify_buffer {
  SPO_VERIFY_INPUT_TOKENS = 0, SPO_VERIFY_TREE_ROWS, SPO_VERIFY_DEPTHS, SPO_VERIFY_UNIFORMS, SPO_VERIFY_TOKENS,
  SPO_VERIFY_RETAINED, SPO_VERIFY_ACCEPTED, SPO_VERIFY_RETAINED_ROWS, SPO_VERIFY_PAGE_TABLE, SPO_VERIFY_KV_POOL,
  SPO_VERIFY_LOGITS, SPO_VERIFY_DRAFT_PROBABILITIES, SPO_VERIFY_HIDDEN,
  SPO_VERIFY_QKV_ROWS = 15, SPO_VERIFY_ATTENTION_ROWS = 16, SPO_VERIFY_FFN_ROWS = 17,
  /* the sampled rows' candidate children (spo_sampling_buffers): index 0 ids, 1 probabilities, 2 drawn children, 3 child
     uniforms; host-visible, allocated by the first call. Fetching them changes no step: spo_dense_verify_set_test_children
     chooses which test the sampled lanes of later steps run */
  SPO_VERIFY_CANDIDATE_CHILDREN = 18,
  /* the penalty table: uint32 [max lanes][vocabulary] in device memory, lane l's row at words l x vocabulary on
     (spo_sampling_rebuild_penalty_words makes a row); allocated, zeroed, by the first call or by set_penalties */
  SPO_VERIFY_PENALTY_WORDS = 19,
  /* the constraint masks of constrained lanes: uint32 [max rows][ceil(vocabulary / 32)] in device memory, bit t % 32 of
     word t / 32 of a packed row admits token t; allocated by the first call */
  SPO_VERIFY_TOKEN_MASK = 20
} spo_verify_buffer;
sp_status spo_dense_verify_buffer(spo_dense_verify *verify, spo_verify_buffer which, uint32_t index, sp_buffer **out);
/* The sampling penalties of dispatch lane `lane` (SamplingPolicy::penalties, Sampling.hpp:71 in the reference) for the
 * steps encoded after: its rows of the head's logits are rewritten from its row of SPO_VERIFY_PENALTY_WORDS before the
 * step selects (spo_sampling_add_penalties), and a step that commits counts the tokens the lane keeps into that row
 * (spo_sampling_add_penalty_count). 1, 0, 0 turns them off. */
sp_status spo_dense_verify_set_penalties(spo_dense_verify *verify, uint32_t lane, float repetition, float presence, float frequency);
/* SamplingPolicy::constrained and ::excludesStopTokens of dispatch lane `lane` (Sampling.hpp:66-70) for the steps
 * encoded after: a constrained lane's rows admit only the tokens of their rows of SPO_VERIFY_TOKEN_MASK; a lane that
 * excludes stop tokens never selects one. */
sp_status spo_dense_verify_set_admission(spo_dense_verify *verify, uint32_t lane, uint32_t constrained, uint32_t excludes_stop_tokens);
/* The stop tokens of the steps encoded after (StopTokens of Sampling::addVerify / addAcceptance): four ids, 0xFFFFFFFF
 * for none; NULL for none at all. Acceptance ends a lane's path at one. */
sp_status spo_dense_verify_set_stop_tokens(spo_dense_verify *verify, const uint32_t *stop_tokens);
/* The thinking cutoff of dispatch lane `lane` (SamplingPolicy::thinkingCutoff, Sampling.hpp:76) for the steps encoded
 * after; NULL, or active 0, clears it. An end that waits for its mask needs a constrained lane (set_admission). */
sp_status spo_dense_verify_set_thinking_cutoff(spo_dense_verify *verify, uint32_t lane, const spo_thinking_cutoff *cutoff);
uint64_t spo_dense_verify_page_bytes(const spo_dense_verify *verify);
/* Algorithmic HBM bytes of one step: weights once, each lane's KV, logits written and read. */
uint64_t spo_dense_verify_step_bytes(const spo_dense_verify *verify, const spo_verify_lane *lanes, uint32_t count);
/* Appends the whole target part of a cycle (Runtime.cpp:3985-3993) to the graph. */
sp_status spo_dense_verify_encode(spo_dense_verify *verify, spo_graph *graph, const spo_verify_lane *lanes, uint32_t count,
                                  int commit);
/* One part of it, for per-part timing: 0 embedding, 1 one layer (index), 2 final norm + head. */
sp_status spo_dense_verify_encode_part(spo_dense_verify *verify, spo_graph *graph, uint32_t part, uint32_t index,
                                       const spo_verify_lane *lanes, uint32_t count);

/* A completed step's results, checked as Runtime::finalizeDecode checks them before a lane commits (Runtime.cpp:2943-2972,
 * invalidSelection :1559-1582): per lane 1 <= retained <= min(rows, remaining), popcount(retained_rows) == retained with
 * bit 0 set and no bit at or past the lane's rows, accepted < rows and <= retained, every retained token below
 * `vocabulary`. SP_BACKEND_ERROR with the lane and the rule in sp_last_error() otherwise. Host arrays only: lanes[i]
 * gives lane i's first packed row and its rows, tokens holds the step's packed rows. */
sp_status spo_verify_check_results(const spo_lane_rows *lanes, const uint32_t *remaining, uint32_t count, uint32_t step_rows,
                                   uint32_t vocabulary, const uint32_t *tokens, const uint32_t *retained, const uint32_t *accepted,
                                   const uint32_t *retained_rows);
/* Reads a completed step's results out of the driver's buffers (call after the command's ticket has been waited for),
 * checks them as spo_verify_check_results does, and copies them: tokens uint32 [the lanes' rows, packed], the others
 * uint32 [count]. */
sp_status spo_dense_verify_results(spo_dense_verify *verify, const spo_verify_lane *lanes, uint32_t count, uint32_t *tokens,
                                   uint32_t *retained, uint32_t *accepted, uint32_t *retained_rows);
/* Whether steps encoded from now on chain a layer's projections after its attention into one dispatch
 * (spo_linear_add_chain: output, gate/up, down and the next layer's q|k|v, the LM head after the last layer) where
 * their shapes allow: off by default; the results are the same bit for bit. spo_dense_verify_results fails with
 * SP_BACKEND_ERROR after a step in which a chained projection's bounded wait gave up. A chained dispatch rests on
 * two things HIP does not promise: that the device starts a grid's workgroups in index order (a link's workgroups are
 * started before any of the next link's), and that a link's results, stored with agent scope and counted in only after
 * the stores completed, are seen by a later link that never read those addresses before. The bounded wait turns a
 * break of either into a status, never a hang. */
/* Whether the sampled lanes of steps encoded from now on test the children their draft drew among sixteen candidates
 * (SPO_VERIFY_CANDIDATE_CHILDREN; sampling.metal:697-880) or, the default, one child against the full-vocabulary draft
 * distribution (SPO_VERIFY_DRAFT_PROBABILITIES). A step reads only the buffers of the test it runs. */
sp_status spo_dense_verify_set_test_children(spo_dense_verify *verify, int on);
/* The chained projections' status of the last completed step, for a caller that reads logits or hidden rows through
 * spo_dense_verify_buffer without spo_dense_verify_results: *status 0 when every wait was met (always, of a step that
 * chains nothing), nonzero when one gave up and what the step left is void. Reading it clears it. No counterpart in the
 * reference, whose projections are a dispatch each. */
sp_status spo_dense_verify_chain_status(spo_dense_verify *verify, uint32_t *status);
/* DenseVerify::encodePrefill: a chunk of 1 to 16 x max_lanes (or the prefill_rows it was created with) prompt tokens of ONE sequence (its pages from table_first,
 * `committed` tokens cached before the chunk) in one pass over the weights, where the reference prefills a prompt in
 * chunks (Runtime.cpp's chunked prefill over QwenTarget.cpp:457-496): the tokens go in SPO_VERIFY_INPUT_TOKENS, a chain
 * of tree rows a block of sixteen in SPO_VERIFY_TREE_ROWS, each row's depth in its block in SPO_VERIFY_DEPTHS, as a
 * step's. Every layer runs, the head and the acceptance do not: the tokens' keys and values are in the pages and the
 * hidden rows where a step leaves them, bit for bit those of the blocks run one step after the other; the caller
 * advances the sequence's committed tokens. */
sp_status spo_dense_verify_encode_prefill(spo_dense_verify *verify, spo_graph *graph, uint32_t table_first, uint32_t committed,
                                          uint32_t tokens);
sp_status spo_dense_verify_set_chained(spo_dense_verify *verify, int chained);
/* DenseVerify::setFusedPrepare: a layer's q|k|v projection also prepares its attention block
 * (spo_attention_add_fused_projection) where the kernels take the pair: off by default (on MI355X the two dispatches
 * are the faster at the 27B shape); the results are the same bit for bit. */
sp_status spo_dense_verify_set_fused_prepare(spo_dense_verify *verify, int fused);

/* ---- The hybrid mixture-of-experts verify step (the reference's Qwen3.5 target with Gated
 *      DeltaNet mixers: QwenTarget.cpp:206-255 the GDN mixer, :263-347 the attention mixer, :372-395
 *      the MoE routing, :457-496 the layer recipe; Runtime.cpp:2701-2707 tape parity and pending
 *      path). Layer l attends when (l + 1) % attention_interval == 0; the others run GDN. ---- */
typedef struct spo_hybrid_verify spo_hybrid_verify;
typedef struct spo_hybrid_dimensions {
  uint32_t hidden, vocabulary, layers, attention_interval;
  uint32_t q_heads, kv_heads, head_dim, rotary_pairs, normalize_heads;
  uint32_t gated_attention; /* the attention layers' rows carry output gates (the reference's Qwen3.5 attention) */
  float rope_theta;
  uint32_t gdn_key_heads, gdn_value_heads, gdn_packed_width; /* packed row [q|k|v|z|b|a], whole column tiles */
  uint32_t experts, top_k, expert_ffn;
  uint32_t shared_slices, shared_gate; /* the shared expert, as in spo_moe_shape */
  uint32_t dense_ffn; /* with experts 0: every layer's FFN is a dense SwiGLU of this width (QwenTarget.cpp:351-370) */
} spo_hybrid_dimensions;
typedef struct spo_hybrid_lane {
  spo_verify_lane block;
  uint32_t pending_path; /* rows of the lane's previous step it accepted: that step's retained-rows mask */
  uint32_t parity;       /* the step reads the lane's cell `parity` and writes the other; the next step flips it */
} spo_hybrid_lane;
typedef struct spo_hybrid_layer {
  const spo_projection *mixer_input, *mixer_output; /* q|k|v and o, or the packed GDN row and its output projection */
  sp_buffer *input_norm, *post_norm;
  sp_buffer *query_norm, *key_norm;                                   /* attention layers */
  sp_buffer *convolution_weights, *decay_weights, *time_bias, *mixer_norm; /* GDN layers; mixer_norm bf16 [128] */
  const spo_projection *router;                                       /* hidden -> experts, fp32 scores */
  sp_buffer *gate_images, *up_images, *down_images;                   /* every expert's image of each tensor */
  uint32_t expert_format, expert_down_format;
  sp_buffer *shared_scalar_gate; /* fp32 [hidden], of a gated shared expert (NULL otherwise) */
  const spo_projection *ffn_gate, *ffn_up, *ffn_down; /* a dense model's SwiGLU (router and images NULL) */
} spo_hybrid_layer;
sp_status spo_hybrid_verify_create(sp_backend *backend, const spo_hybrid_dimensions *dimensions, uint32_t max_lanes,
                                   uint32_t physical_pages, uint32_t page_table_entries, spo_hybrid_verify **out);
/* The same with room for prompt chunks of up to prefill_rows rows (spo_hybrid_verify_encode_prefill; 0: a step's most; at
 * most 2048, SPLASH_PREFILL_TOKEN_BUDGET). */
sp_status spo_hybrid_verify_create_chunked(sp_backend *backend, const spo_hybrid_dimensions *dimensions, uint32_t max_lanes,
                                           uint32_t physical_pages, uint32_t page_table_entries, uint32_t prefill_rows,
                                           spo_hybrid_verify **out);
void spo_hybrid_verify_destroy(spo_hybrid_verify *verify);
sp_status spo_hybrid_verify_set_layer(spo_hybrid_verify *verify, uint32_t layer, const spo_hybrid_layer *weights);
sp_status spo_hybrid_verify_set_head(spo_hybrid_verify *verify, uint32_t embedding_format, sp_buffer *embedding_rows,
                                     sp_buffer *final_norm, const spo_projection *head);
/* As spo_dense_verify_set_capture: the hidden rows after the named layers, for a draft's context. */
sp_status spo_hybrid_verify_set_capture(spo_hybrid_verify *verify, const uint32_t *layers, uint32_t count, sp_buffer *destination);
/* The step's buffers, as spo_dense_verify_buffer; `index` is the attention layer for KV pools. */
#define SPO_VERIFY_GDN_STATES 13
#define SPO_VERIFY_GDN_TAPE 14
sp_status spo_hybrid_verify_buffer(spo_hybrid_verify *verify, uint32_t which, uint32_t index, sp_buffer **out);
/* As spo_dense_verify_set_penalties. */
sp_status spo_hybrid_verify_set_penalties(spo_hybrid_verify *verify, uint32_t lane, float repetition, float presence, float frequency);
/* As spo_dense_verify_set_admission, _set_stop_tokens and _set_thinking_cutoff. */
sp_status spo_hybrid_verify_set_admission(spo_hybrid_verify *verify, uint32_t lane, uint32_t constrained, uint32_t excludes_stop_tokens);
sp_status spo_hybrid_verify_set_stop_tokens(spo_hybrid_verify *verify, const uint32_t *stop_tokens);
sp_status spo_hybrid_verify_set_thinking_cutoff(spo_hybrid_verify *verify, uint32_t lane, const spo_thinking_cutoff *cutoff);
/* HybridVerify::encodePrefill: a chunk of `tokens` prompt tokens of the sequence of lane `lane` (its pages from table_first,
 * `committed` tokens cached; inputs as spo_dense_verify_encode_prefill's) through layers [first_layer, first_layer +
 * layer_count) (layer_count 0: to the last; the embedding with first_layer 0), no head: the reference's chunked prefill over
 * its hybrid target (QwenTarget.cpp:206-347 with GDN::addPrefill, GDN.cpp:132-222; PagedAttention.cpp:351-389). Attention
 * layers store the chunk's keys and values and attend causally; Gated DeltaNet layers take every row into the state, from
 * the lane's cell of `parity` to its other cell: the lane's next step has the other parity and no pending path. */
sp_status spo_hybrid_verify_encode_prefill(spo_hybrid_verify *verify, spo_graph *graph, uint32_t lane, uint32_t table_first,
                                           uint32_t committed, uint32_t tokens, uint32_t parity, uint32_t first_layer,
                                           uint32_t layer_count);
/* As spo_dense_verify_results. */
sp_status spo_hybrid_verify_results(spo_hybrid_verify *verify, const spo_hybrid_lane *lanes, uint32_t count, uint32_t *tokens,
                                    uint32_t *retained, uint32_t *accepted, uint32_t *retained_rows);
/* Where the recurrent state lives: a lane's cell of a parity at (lane * 2 + parity) * cell_bytes in the
 * states buffer (strides as spo_gdn_layout gives them for the model's GDN layers), GDN layer g's tape of
 * a lane's step of a parity at ((lane * 2 + parity) * gdn_layers + g) * tape_layer_bytes in the tape buffer. */
sp_status spo_hybrid_verify_layout(const spo_hybrid_verify *verify, uint64_t *page_bytes, uint64_t *cell_bytes,
                                   uint64_t *tape_layer_bytes, spo_gdn_state_strides *strides);
uint64_t spo_hybrid_verify_step_bytes(const spo_hybrid_verify *verify, const spo_hybrid_lane *lanes, uint32_t count);
sp_status spo_hybrid_verify_encode(spo_hybrid_verify *verify, spo_graph *graph, const spo_hybrid_lane *lanes, uint32_t count,
                                   int commit);
/* One part of it: 0 embedding, 1 one layer (index), 2 final norm + head. */
sp_status spo_hybrid_verify_encode_part(spo_hybrid_verify *verify, spo_graph *graph, uint32_t part, uint32_t index,
                                        const spo_hybrid_lane *lanes, uint32_t count);

#ifdef __cplusplus
}
#endif
#endif /* SPLASH_OPS_H */
