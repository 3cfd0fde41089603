// CPU oracle of the speculative-decoding verify step: TEST INFRASTRUCTURE ONLY.
//
// A plain C++ restatement of the arithmetic rules of the reference (incoai/splash): its test
// references (dev/tests/engine/*Reference.hpp, the fp64 references inside the kernel tests) and
// the operation order of its kernels. Only tests/, __graft_entry__.smoke() and bench.py's
// cpu_baseline leg may load this library, and only as the checker or the reported CPU baseline.
// Nothing under splash_amd/ links, loads or calls it.
//
// Pin status of each group of functions (what fixes it besides its own formula):
//   orc_dequant_rows (Q4_K, Q5_K,   pinned: SHA-256 goldens of upstream GGML over the 256x1024
//     Q6_K, Q8_0, IQ4_XS, IQ4_NL)   fixture (dev/tests/fixtures/weight-goldens/goldens.json:3-7,9)
//                                   and the compiled reference header (oracle/_ref).
//   orc_fixture                     pinned by the same goldens (a wrong byte order changes the hash).
//   orc_quantize_q4k / q6k          PARITY UNPINNED: the K-quantizer lives in llama.cpp/ggml
//                                   (goldens cite commit 7ab4ee7), absent from the reference tree.
//                                   Oracle and GPU consume the same bytes, so verify parity does not
//                                   depend on it; tests bound its round-trip error only.
//   orc_gemm_*                      pinned by fp64 dot + projectionBound interval, and invariants.
//   orc_kv_quantize                 pinned: closed form, compiled reference header (oracle/_ref).
//   orc_attention_*                 pinned by dense-softmax special cases and invariants.
//   orc_gdn_*                       pinned by the fp64 textbook recurrence (orc_gdn_reference, the check
//                                   the reference's own test makes) and fold/rollback invariants; tree
//                                   blocks by the same recurrence along each row's path.
//   orc_argmax / orc_accept_tree    pinned by brute force on tiny vocabularies.
//   orc_draft_verify_rows           pinned by an independent statement (a stable sort of the estimates, a recursive
//                                   preorder) in the tests.
//   orc_draft_tree                  pinned by an independent statement in the tests (every path's entry enumerated in fp64,
//                                   a stable sort by estimate, cases whose order hangs on less than 1e-4 set aside), by the
//                                   caps' and estimates' invariants, and by the frequencies of a sampled row's draws.
//   orc_draft_candidates            pinned by a lexicographic sort of (logit descending, column ascending) in the tests,
//                                   ties, signed zeros and short rows among the cases.
//   orc_draft_edges                 pinned by the fp64 trilinear sum over the decoded bf16 factors (numpy einsum), to the
//                                   rounding of its fp32 products.
//   orc_rejection_*                 pinned by enumeration: selection law equals target to 1e-12.
//   orc_distribution_end            pinned by an independent fp64 sort (min_p, top_k with ties, nucleus).
//   orc_moe_*                       pinned by a stable sort and softmax closed form; the layer by the dense FFN it
//                                   reduces to when every expert is the same.
//   orc_state_codes / _values       pinned: the compiled reference header (oracle/_ref, StateCodecReference.hpp) bit for
//                                   bit, and the closed form (a value restores within half its block's step).
//   orc_draft_conv / _prepare /     pinned by fp64 statements in numpy (the convolution exactly on dyadic inputs, as the
//     _context_write                reference's test draws them; the head norm and rotation to a bf16 step; slots and
//                                   untouched bytes by position).
//   orc_draft_attention             pinned by a dense fp64 softmax in numpy over the rows' windows (short, wrapping and
//                                   full rings) and by shift invariance: a ring rotated with its positions gives the same rows.
//   orc_draft_window_*              pinned by the closed form (a value restores within half its group's step, extremes
//                                   within an fp16 step of themselves) and numpy's codes.
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

// Format ids follow the reference's GGUF_FMT_* numbering (runtime/metal/abi/QuantFormat.h:138-154).
enum { ORC_FMT_Q4K = 0, ORC_FMT_IQ4XS = 1, ORC_FMT_IQ4NL = 2, ORC_FMT_Q5K = 3, ORC_FMT_Q6K = 4, ORC_FMT_Q3K = 5, ORC_FMT_Q80 = 6, ORC_FMT_Q40 = 15,
       ORC_FMT_Q50 = 39 };

// ---- half / bfloat16 scalar conversions (round to nearest even) ----
uint16_t orc_f2h(float f);
float orc_h2f(uint16_t h);
uint16_t orc_f2bf(float f);
float orc_bf2f(uint16_t b);

// ---- GGUF K-quants ----
// Bytes of one native row of K values (K a multiple of 256). 0 for an unknown format.
uint64_t orc_row_bytes(uint32_t fmt, uint32_t K);
// dev/tests/engine/GgufFixtures.hpp:148-165 fixture(f, rows, K, seed): random bytes, finite half scales.
int orc_fixture(uint32_t fmt, uint32_t rows, uint32_t K, uint32_t seed, uint8_t *native);
// dev/tests/engine/GgufFormatReference.hpp:195-219,295-323 makeNative with realistic scales.
int orc_make_native(uint32_t fmt, uint32_t rows, uint32_t K, uint32_t seed, uint8_t *native);
// llama.cpp dequantize_row_q4_K / q5_K / q6_K / q8_0 semantics (GgufFormatReference.hpp:370-381, :405-432, :453-458).
int orc_dequant_rows(uint32_t fmt, const uint8_t *native, uint32_t rows, uint32_t K, float *out);
// llama.cpp-style quantize_row_q4_K_ref / q6_K_ref (parity unpinned, see header).
int orc_quantize_rows(uint32_t fmt, const float *values, uint32_t rows, uint32_t K, uint8_t *native);

// Projection out[m][n] = sum_k x[m][k] W[n][k], x bf16 [M][K], W native rows [N].
// exact:  fp64 dot product.  bound: projectionBound(register tile) (GgufFormatReference.hpp:739-742).
// chain:  the register rule in fp32 (linear_gguf_sgmatrix.metal:140-151, :199-288).
// Any of the three outputs may be NULL. threads <= 0 uses every core.
int orc_gemm(uint32_t fmt, const uint8_t *native, const uint16_t *x, uint32_t M, uint32_t K, uint32_t N,
             double *exact, double *bound, float *chain, int threads);
// The staged tile's projection (kernels/common/gguf_staged.h:12-66: every weight decoded with fp32 group coefficients
// and rounded once to half; gguf_linear.metal:1-12: fp32 accumulation of its products with the bf16 inputs).
// exact:  fp64 dot product with the weights' fp32 values (what the reference's test measures from).
// bound:  projectionBound(staged) (GgufFormatReference.hpp:739-742): 2^-16 sum|x| max|w| + 2^-11 sum|x w| + 2^-25 sum|x|.
// staged: the fp64 dot product with the weights rounded to half, rounded to fp32: what the tile computes but for the
//         order and roundings of its fp32 accumulation, which 2^-16 sum|x| max|w| (accumulation) bounds.
// Pinned by the reference's own dot and projectionBound (oracle/_ref) and numpy's float16 rounding of orc_dequant_rows.
int orc_gemm_staged(uint32_t fmt, const uint8_t *native, const uint16_t *x, uint32_t M, uint32_t K, uint32_t N,
                    double *exact, double *bound, float *staged, double *accumulation, int threads);
// The column tile's fp32 totals out[M][N] (kernels/common/gguf_column_tile.h:25-68, linear_gguf_column.metal:33-66):
// half weights, a group's 32 products added in element order, groups added to their part of K (eight parts of
// G / 8 groups, by integer division of s G), the parts added in order. Pinned by closed forms that only this order
// satisfies (tests/test_oracle_gguf.py) and by the staged interval of orc_gemm_staged.
int orc_gemv_column(uint32_t fmt, const uint8_t *native, const uint16_t *x, uint32_t M, uint32_t K, uint32_t N, float *out,
                    int threads);
// Epilogues on fp32 sums (kernels/common/gguf_tile.h:10-16, gguf_linear.metal:34-71).
uint16_t orc_epilogue_plain(float v);
uint16_t orc_epilogue_residual(float v, uint16_t residual);
uint16_t orc_epilogue_swiglu(float gate, float up);
float orc_silu(float x);

// ---- glue ----
// bf16((x * rsqrt(sum x^2 / W + 1e-6)) * w) per row (normalization.metal:59-99).
void orc_rms_norm(const uint16_t *x, const uint16_t *w, uint32_t rows, uint32_t width, uint16_t *out);
// The fp32 projection of weights kept as rows (gguf_float.metal:1-8): x bf16 [rows][k], w F32 (or BF16) [n][k], out fp32
// [rows][n]; four chains of fused multiply-adds by k mod 4, added (c0 + c1) + (c2 + c3). Pinned by the fp64 product
// (it differs by fp32 accumulation only), by BF16 weights giving the bits of their F32 values, and by sums that only
// this order gives exactly (tests/test_oracle_glue.py).
void orc_float_projection(const uint16_t *x, const void *w, uint32_t bf16_weights, uint32_t rows, uint32_t n, uint32_t k, float *out);
// Token gather from native rows: bf16(decode(table[token][dim])), token >= vocab -> 0 (embedding.metal:10-18).
int orc_embed(uint32_t fmt, const uint8_t *table, uint32_t vocab, uint32_t hidden, const uint32_t *tokens,
              uint32_t rows, uint16_t *out);
// cos/sin of (anchor + depth[row]) * invfreq[pair], fp32 (rope.metal:51-80).
void orc_rope_tables(uint32_t anchor, const uint32_t *depth, uint32_t rows, const float *invfreq, uint32_t pairs,
                     float *cosv, float *sinv);

// ---- INT8 KV ----
// Per (token, head) over D values: scale = max|v| / 127, code = clamp(rint(v * 127 / max), -127, 127)
// (Q8PageFormatReference.hpp:107-122, attention_store.h:52-85). The stored scale is fp16 when
// half_scale is nonzero (rounded after the codes are computed), else fp32; *scale_out holds its value.
void orc_kv_quantize(const float *v, uint32_t D, int half_scale, int8_t *codes, float *scale_out);

struct OrcAttention {
  uint32_t q_heads, kv_heads, head_dim;
  uint32_t rows;        // query rows of the block
  uint32_t committed;   // tokens in the cache before the block; row r sits at slot committed + r
  uint32_t page_tokens; // tokens per page
  uint32_t splits;      // history splits merged in split order (1 = none)
  uint32_t pages_per_split;
  uint32_t half_scale;  // scales are fp16 values (already rounded) -- informational
  uint32_t int8_queries; // the page loop scores INT8 codes of each (row, head)'s queries (paged_attention_tile.h:294-322)
};
// q/k per-head RMS norm + partial RoPE + staging (attention_qkv_prepare.h:28-91).
// qkv bf16 [rows][(q_heads + 2 kv_heads) * D]; qw/kw bf16 [D] norm weights (NULL = no norm);
// cos/sin fp32 [rows][pairs]; pairs*2 <= D rotated as (i, i + pairs).
// q_out bf16 [rows][q_heads][D]; k_out/v_out fp32 [rows][kv_heads][D] are the values to quantize.
void orc_attention_prepare(const struct OrcAttention *a, const uint16_t *qkv, const uint16_t *qw, const uint16_t *kw,
                           const float *cosv, const float *sinv, uint32_t pairs, uint16_t *q_out, float *k_out,
                           float *v_out);
// common/int8_activations.h:22-28: a block of activations as INT8 codes and one scale: with m the block's largest
// magnitude, code = clamp(rint(x * (127 / m)), -127, 127) (ties to even, the quotient rounded first) and scale = m / 127;
// a block whose m is 2^-100 or less codes as zeros with scale 0; one that holds an infinity or a NaN takes a NaN scale.
void orc_int8_activation_block(const float *x, uint32_t n, int8_t *codes, float *scale);
// Block-causal attention over paged INT8 KV, page by page with the online softmax of
// paged_attention_tile.h:179-285 and the ordered split merge of :499-535.
// pages: page_table[p] names the physical page of logical page p. A physical page holds
// keys int8 [kv_heads][page_tokens][D], values int8 [kv_heads][page_tokens][D] and scales
// float [kv_heads][page_tokens] each (already the stored, possibly fp16-rounded, values).
// ancestors[r]: bit j set when block row j is visible to row r (chain: (2 << r) - 1).
// out bf16 [rows][q_heads * D]. out64 (optional) is the fp64 dense-softmax reference
// (q8_flash_attention_metal_test.mm:485-536), unrounded.
void orc_attention(const struct OrcAttention *a, const uint16_t *q, const int8_t *kcodes, const float *kscales,
                   const int8_t *vcodes, const float *vscales, const uint32_t *page_table,
                   const uint32_t *ancestors, uint16_t *out, double *out64, int threads);

// ---- acceptance ----
#define ORC_NO_TOKEN 0xFFFFFFFFu
// Largest finite logit, ties to the lowest id; NaN and -inf skipped (sampling.metal:1896-1997).
uint32_t orc_argmax(const float *logits, uint32_t vocab);
struct OrcTreeRow { uint32_t ancestors; uint16_t parent; uint16_t depth; };
// sampling.metal:2044-2083 decode_accept_tree for one lane.
// tokens[r]: input token of row r; selected[r]: the target's selection at row r.
// Returns kept count; out_tokens[0..kept), *accepted, *retained_rows (ancestor mask of the last kept row).
uint32_t orc_accept_tree(const struct OrcTreeRow *tree, const uint32_t *tokens, const uint32_t *selected,
                         uint32_t rows, uint32_t remaining, const uint32_t *stop_tokens, uint32_t stops,
                         uint32_t *out_tokens, uint32_t *accepted, uint32_t *retained_rows);
// sampling.metal:1799-1895 draft_verify_rows: a decode step's rows from each lane's tree (16 rows a lane: tokens, tree
// rows, {draft probability, estimate} pairs; sizes[lane] rows held). Outputs as the kernel writes them: tokens, tree rows
// and sources [rows], lane_rows {first, rows} [lanes].
void orc_draft_verify_rows(const uint32_t *tree_tokens, const struct OrcTreeRow *trees, const float *scores, const uint32_t *sizes,
                           uint32_t lanes, uint32_t rows, uint32_t lane_cap, float floor, uint32_t *tokens, struct OrcTreeRow *tree,
                           uint32_t *lane_rows, uint32_t *sources);
// The same rows in slots (a layout of this build; see abi/Sampling.h): lane l's rows from row l * lane_cap on, the rest of its
// slot inert. Pinned by its relation to the packed layout above and by what makes a row inert to the step
// (tests/test_oracle_sampling.py).
void orc_draft_verify_row_slots(const uint32_t *tree_tokens, const struct OrcTreeRow *trees, const float *scores, const uint32_t *sizes,
                                uint32_t lanes, uint32_t lane_cap, float floor, uint32_t *tokens, struct OrcTreeRow *tree,
                                uint32_t *lane_rows, uint32_t *sources);
// sampling.metal:1357-1766 draft_select_tree for one lane: candidates uint32 [7][16], unary fp32 [7][16], edges fp32
// [7][16][16] ([position][predecessor][candidate]; position 0 reads predecessor 0 alone), the lane's host chain (15 tokens, a
// rate for each of 4 agreements a token) and parameters (Sampling.h:242-252, one lane's). Outputs, 16 rows: tokens, tree
// rows, {draft probability, estimate} pairs, the rows held, each row's drawn children (candidate indices, 0xFF past them),
// its next position's probabilities, and its cap.
struct OrcDraftTreeLane {
  uint32_t anchor, depth, chain, children;
  float slope, intercept[7], temperature;
  uint32_t noise[2];
};
void orc_draft_tree(const uint32_t *candidates, const float *unary, const float *edges, const uint32_t *chain_tokens,
                    const float *chain_rates, const struct OrcDraftTreeLane *lane, uint32_t *tokens, struct OrcTreeRow *tree,
                    float *scores, uint32_t *size, uint8_t *draws, float *next, float *caps);
// sampling.metal:1099-1264: of each proposal position's logits row (rows 1-7 of a lane's eight, fp32 [lanes * 8][columns])
// the sixteen columns of the largest logits, the larger first, the smaller column first among equal ones; candidates their
// tokens (a column at or past `leading` is token column - leading + trailing), unary their logits, [lanes * 7][16];
// 0xffffffff and -infinity where the columns run out.
void orc_draft_candidates(const float *logits, uint32_t lanes, uint32_t columns, uint32_t leading, uint32_t trailing,
                          uint32_t *candidates, float *unary);
// sampling.metal:1271-1356: edges fp32 [lanes * 7][16][16], [predecessor][candidate]; hidden bf16 [lanes * 8][256], codebooks
// bf16 [vocabulary][256]. Position 0 writes its row 0 alone (predecessor anchors[lane]).
void orc_draft_edges(const uint32_t *candidates, const uint32_t *anchors, uint32_t lanes, uint32_t vocabulary, const uint16_t *hidden,
                     const uint16_t *predecessor_codebook, const uint16_t *successor_codebook, float *edges);
// One sampled verify row under the textbook full-vocabulary rule in the reference's order of
// operations (sampling.metal:713-885): weight_t = exp((logit_t - max) / T); p = weight / total;
// accept the drafted token iff u_child * q[draft] < p[draft]; else draw from max(p - q, 0)
// renormalised by an id-ordered prefix walk at u_row. q NULL: plain draw at u_row * total.
// closeness (optional): the smallest relative distance of a decisive comparison from its threshold;
// tests treat a row below 1e-5 as "close", as target_sampling_metal_test.mm:2645-2709 does.
uint32_t orc_rejection_row(const float *logits, uint32_t vocab, float temperature, const float *q,
                           uint32_t draft_token, float u_child, float u_row, int *accepted_draft, double *closeness);
// A lane's sampling policy (Sampling.hpp:56-83 in the reference): the tokens that weigh at least min_p of
// the heaviest (0: all), then the top_k most likely of those (0: all), then their top_p nucleus (1: all).
struct OrcSamplingPolicy { float temperature, min_p; uint32_t top_k; float top_p; };
// distribution_end (sampling.metal:603-670): the last token the row keeps in the order of the logits
// (larger first, among equals the smaller id first) as (key, last id), the kept mass, and the kept count
// (returned). {0, 0} keeps everything; an end after the last token of its key's run has last id 0xFFFFFFFF. Pinned by brute force against a sort in the tests; masses sum in
// fp64, so a nucleus within rounding of a token's boundary is reported through `closeness`.
uint32_t orc_distribution_end(const float *logits, uint32_t vocab, const struct OrcSamplingPolicy *policy, uint32_t *key,
                              uint32_t *last, float *mass, double *closeness);
// orc_rejection_row and orc_rejection_law over the distribution the policy leaves.
uint32_t orc_rejection_row_policy(const float *logits, uint32_t vocab, const struct OrcSamplingPolicy *policy, const float *q,
                                  uint32_t draft_token, float u_child, float u_row, int *accepted_draft, double *closeness);
void orc_rejection_law_policy(const float *logits, uint32_t vocab, const struct OrcSamplingPolicy *policy, const float *q,
                              double *out);
// The selection law of one sampled row in fp64, for the enumeration check
// (target_sampling_metal_test.mm:2602-2631): out[t] = P(row selects t) when the draft proposes its
// child from q and the row tests and redraws as above. It must equal softmax(logits / T).
// The sampling penalties of one lane's verify rows, in place (PenaltyReference.hpp:27-40 for a logit; sampling.metal:1008-1050
// for the draft tokens a row's context adds): logits fp32 [rows][stride], words uint32 [vocabulary] (bit 31: in the prompt;
// the rest: times selected), the block's input tokens and ancestor masks. Pinned by closed forms on chosen cases
// (tests/test_oracle_sampling.py): untouched tokens bitwise, a prompt token's one product, a count's one difference,
// saturation, unselectable logits, and the rows of a chain and of a forked tree that count a drafted token.
void orc_penalize(float *logits, uint32_t rows, uint32_t vocabulary, uint32_t stride, const uint32_t *words, const uint32_t *input_tokens,
                  const uint32_t *ancestors, float repetition, float presence, float frequency);
// The thinking cutoff of one lane's selections, in place (sampling.metal:1993-2039): tokens uint32 [rows] (the selections),
// the block's input tokens and tree rows, the depth the end starts at, the end's first `count` tokens, the token that
// closes thinking and the other that ends it, and, for an end that waits for its mask, whether each row's mask admits
// end[0] (NULL: the end does not wait). Pinned by hand-worked chains and trees (tests/test_oracle_sampling.py): the rows
// that take which end token, the rows past the end, an end already drafted on the path (and not on a sibling's), the
// sentinel kept, and the waiting end's later start.
void orc_thinking_cutoff(uint32_t *tokens, const uint32_t *input_tokens, const struct OrcTreeRow *tree, uint32_t rows, uint32_t vocabulary,
                         uint32_t cutoff_row, const uint32_t *end, uint32_t count, uint32_t close, uint32_t also_ends,
                         const uint8_t *admits);
// sampling.metal:697-880: a verify row of a tree block: up to four drawn children among sixteen candidates (ids, their
// draft probabilities q, the candidate indices drawn in order, 0xFF for none, one uniform a child), then the last
// residual's draw at u_row. Returns the selected token.
uint32_t orc_children_row(const float *x, uint32_t V, const struct OrcSamplingPolicy *policy, const uint32_t *ids, const float *q,
                          const uint8_t *draws, uint32_t n_draws, const float *u_children, float u_row, double *closeness);
// The law of that selection over the draft's draws without replacement, by enumeration in fp64: out[t] = P(select t).
void orc_children_law(const double *p_target, uint32_t V, const uint32_t *ids, const double *q, uint32_t n_draws, double *out);
void orc_rejection_law(const float *logits, uint32_t vocab, float temperature, const float *q, double *out);

// ---- Gated DeltaNet ----
// Shapes of a layer: packed row = [q (kh 128) | k (kh 128) | v (vh 128) | z (vh 128) | b (vh) | a (vh)],
// conv_dim = (2 kh + vh) 128; flags: 1 tiled output heads, 2 sigmoid gate, 4 fp32 output-norm weights.
struct OrcGdnShape { uint32_t key_heads, value_heads, conv_dim, packed_width, flags; };
// Bytes of one layer's tape of one lane's step (abi/GDN.h:44-67 in the reference): room for 16 rows of
// convolution inputs, k then v rows, decay fp32 and beta bf16.
uint64_t orc_gdn_tape_bytes(const struct OrcGdnShape *s);
// One token on one value head's state S [D v][D k] in the textbook form, sums in fp64 (the
// closed form the restatement below is pinned against): S *= d; mem = S k; delta = beta (v - mem);
// S += delta k^T; o (optional) = S q after the update.
void orc_gdn_step(float *S, uint32_t D, const float *k, const float *v, float decay, float beta, const float *q,
                  float *o);
// One decode step of one lane and one layer over a block of `rows` rows (gdn.metal:139-526): folds
// the pending path of the previous step's tape into the state and writes THAT as state_out (the
// state before this step's rows) with the convolution carry it leaves; writes this step's tape;
// hidden bf16 [rows][vh * 128] are the gated, normed outputs of the block rows.
// conv_in/out bf16 [3][conv_dim]; state fp32 [vh][128][128]; pending_tape may be NULL when the path is 0.
// ancestors[r]: the block rows on row r's path (bit j: row j; NULL: a chain, (2 << r) - 1). A chain's
// rows run the recurrence in order; any other tree's rows read the state before the block along
// their paths (gdn.metal:417-478). Pinned by the fp64 check below on chains, and for trees by the
// same check along each row's path (the tree form is algebraically the chain of the path).
int orc_gdn_decode(const struct OrcGdnShape *s, const uint16_t *packed, uint32_t rows, const uint32_t *ancestors,
                   const uint16_t *conv_weights, const float *a_scale, const uint16_t *dt_bias, const void *norm_weight,
                   const uint16_t *conv_in, const float *state_in, uint8_t *pending_tape, uint32_t pending_path,
                   uint16_t *conv_out, float *state_out, uint8_t *step_tape, uint16_t *hidden);
// The state after the first `rows` rows of `path` of a step's tape, as the lane's next step would
// hold it (gdn.metal:630-698, exact cells). Returns 1 and writes nothing when the path is shorter.
int orc_gdn_fold(const struct OrcGdnShape *s, const uint16_t *conv_in, const float *state_in, uint8_t *step_tape,
                 uint32_t path, uint32_t rows, uint16_t *conv_out, float *state_out);
// A prompt chunk of `tokens` rows of one lane and layer (kernels/prefill/gdn.metal, GDN.cpp:176-222): queries and keys
// bf16 [tokens][kh * 128], values [tokens][vh * 128], decay fp32 and beta bf16 [tokens][vh], the carry and the state
// after the chunk, the scan's rows (recurrent, bf16 [tokens][vh * 128]: o_t = S_t q_t) and their gated norm (hidden).
// Pinned by the fp64 check below under the reference's bounds for the pass (gdn_metal_test.mm:283-409: prepared rows
// within 2 bf16 steps, scan rows within one step + 1e-5, state within 1e-5, gated rows within 2 steps and at most 1 %
// of them off the fp64 rounding), and bit for bit by orc_gdn_decode + orc_gdn_fold over the same rows as accepted
// blocks (tests/test_oracle_gdn.py).
int orc_gdn_prefill(const struct OrcGdnShape *s, const uint16_t *packed, uint32_t tokens, const uint16_t *conv_weights,
                    const float *a_scale, const uint16_t *dt_bias, const void *norm_weight, const uint16_t *conv_in,
                    const float *state_in, uint16_t *queries, uint16_t *keys, uint16_t *values, float *decay, uint16_t *beta,
                    uint16_t *conv_out, float *state_out, uint16_t *recurrent, uint16_t *hidden);
// The fp64 check of a step the reference's test makes (gdn_decode_metal_test.mm:373-522).
int orc_gdn_reference(const struct OrcGdnShape *s, const uint16_t *packed, uint32_t rows, const uint16_t *conv_weights,
                      const float *a_scale, const uint16_t *dt_bias, const uint16_t *conv_in, const float *state_in,
                      double *kv, double *beta, double *decay, double *state_out, double *outputs);

// ---- mixture of experts ----
// kernels/shared/moe.metal:23-113: each row's top_k experts ranked by (score descending, id ascending)
// and their weights exp2((s_r - s_0) log2 e) / sum, the sum in rank order.
void orc_moe_route(const float *scores, uint32_t rows, uint32_t experts, uint32_t stride, uint32_t top_k, uint32_t *selected,
                   float *weights);
// The same selection under the sigmoid router (moe.metal:104-110): weight of rank r = sigmoid(s_r) / (sum over the k
// selected of sigmoid(s) + 1e-20), the sum in rank order.
void orc_moe_route_sigmoid(const float *scores, uint32_t rows, uint32_t experts, uint32_t stride, uint32_t top_k, uint32_t *selected,
                           float *weights);
// kernels/shared/moe.metal:42-65: a gated shared expert's weight of each row, sigmoid(x . gate) with e^-t as
// exp2(-log2(e) t): 64 partial sums, partial l over dimensions l, l + 64, ... in order (a product and a sum, each
// rounded), added pairwise at distances 32, 16, ... 1.
void orc_moe_shared_weights(const uint16_t *x, const float *gate, uint32_t rows, uint32_t hidden, float *weights);
// kernels/shared/moe.metal:367-392: out = bf16(residual + sum over ranks of w y) in fp32, rank order;
// y bf16 [rows][top_k][hidden] the expert outputs of the routes.
void orc_moe_combine(const uint16_t *y, const float *weights, const uint16_t *residual, uint32_t rows, uint32_t top_k,
                     uint32_t hidden, uint16_t *out);

// ---- the cached form of Gated DeltaNet recurrent layers (runtime/ops/StateCodec.hpp, metal/abi/StateCodec.h) ----
// A layer of `rows` value rows of `columns` values: int8 codes row by row, then a bf16 scale per block of 32.
uint64_t orc_state_codec_bytes(uint32_t rows, uint32_t columns);
int orc_state_codes(const float *values, uint32_t rows, uint32_t columns, uint8_t *image);
int orc_state_values(const uint8_t *image, uint32_t rows, uint32_t columns, float *values);

// ---- the draft model's attention block (runtime/ops/DraftAttention.hpp, kernels/decode/draft.metal) ----
// The compiled shape: 32 query heads over 8 KV heads of 128, eight query rows a lane, rings of 2048 slots.
void orc_draft_conv(const uint16_t *input, const uint16_t *dynamic, const uint16_t *base, const uint16_t *residual, uint16_t *output,
                    uint32_t hidden, uint32_t lanes, int finish);
void orc_draft_prepare(const uint16_t *qkv, const uint16_t *query_norm, const uint16_t *key_norm, const float *cosines, const float *sines,
                       uint32_t lanes, uint16_t *queries, uint16_t *keys, uint16_t *values);
void orc_draft_context_write(const uint16_t *context_kv, const uint16_t *key_norm, const float *cosines, const float *sines,
                             const uint32_t *source_rows, const uint32_t *positions, const uint32_t *rope_rows, uint32_t count,
                             uint16_t *ring_keys, uint16_t *ring_values);
void orc_draft_attention(const uint16_t *queries, const uint16_t *ring_keys, const uint16_t *ring_values, const uint16_t *query_keys,
                         const uint16_t *query_values, uint32_t cache_length, double *output);
uint64_t orc_draft_window_bytes(uint32_t width);
void orc_draft_window_store(const uint16_t *context, const uint32_t *source_rows, uint32_t rows, uint32_t start, uint32_t width, uint8_t *window);
void orc_draft_window_load(const uint8_t *window, uint32_t rows, uint32_t start, uint32_t width, uint16_t *context);

#ifdef __cplusplus
}
#endif
