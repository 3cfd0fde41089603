// Parameters of the acceptance kernels (the reference's abi/Sampling.h:50-67, :314-317 and
// abi/VerifyTree.h:40-45).
#pragma once
#include <stdint.h>

#define SAMPLING_SHARDS 32u          // vocabulary shards of one row's scan (one workgroup each)
#define SAMPLING_THREADS 256u
#define SAMPLING_RANGES 256u         // id-ordered ranges a sampled row's draw sums
#define SAMPLING_MAXIMUM_LANES 8u
#define SAMPLING_MAXIMUM_ROWS 16u    // rows of a lane's verify block
#define SAMPLING_STOP_TOKENS 4u
#define SAMPLING_CANDIDATES 16u     // candidates of a row's next position (SPLASH_DRAFT_CANDIDATES)
#define SAMPLING_TREE_CHILDREN 4u   // children a row's draft draws at most (SPLASH_TREE_CHILDREN)
#define SAMPLING_NO_DRAW 0xFFu      // past a row's drawn children
#define SAMPLING_NO_TOKEN 0xFFFFFFFFu  // a row with no selectable logit selects it (SPLASH_NO_TOKEN)
// A sampled row's words of the decisions buffer: the accepted child or SAMPLING_NO_TOKEN, whether
// the row draws from the residual, then the end of its distribution in the order of the logits
// (larger logit first, smaller id first among equals): the last kept token's key and id, and the
// mass and count of the kept tokens.
#define SAMPLING_DECISION_WORDS 8u
#define SAMPLING_END_KEY 2u
#define SAMPLING_END_LAST 3u
#define SAMPLING_END_MASS 4u
#define SAMPLING_END_COUNT 5u

// A lane's rows of the packed rows (SplashLaneRows).
struct SamplingLaneRows {
  uint32_t first;
  uint32_t rows;
};

// decode_sample_argmax_sharded / _reduce, decode_sample_mass_sharded, decode_sample_residual_sharded,
// decode_sample_draw: one dispatch over `rows` packed logits rows of `vocabulary` fp32 logits.
struct TargetSamplingParams {
  uint32_t vocabulary;
  uint32_t rows;          // packed rows
  uint32_t lanes;
  uint32_t logits_stride; // floats between logits rows
  float temperature[SAMPLING_MAXIMUM_LANES];
  uint32_t sampling_mask; // lanes that sample; the others take the argmax
  uint32_t truncating_mask; // lanes whose distribution ends before the last token (min_p, top_k or top_p cut it)
  uint32_t constrained_mask;   // lanes whose rows admit only the tokens of their constraint-mask rows
  uint32_t exclude_stop_mask;  // lanes that ignore end-of-sequence: they never select a stop token
  struct SamplingLaneRows lane[SAMPLING_MAXIMUM_LANES];
  // A sampling lane keeps the tokens that weigh at least min_p of the heaviest, then the top_k most
  // likely of those (0: all), then their top_p nucleus (Sampling.hpp:58-83 in the reference).
  float min_p[SAMPLING_MAXIMUM_LANES];
  uint32_t top_k[SAMPLING_MAXIMUM_LANES];
  float top_p[SAMPLING_MAXIMUM_LANES];
  uint32_t mask_words;      // words of a constraint-mask row (one a packed row): bit t % 32 of word t / 32 admits token t
  uint32_t stop_tokens[SAMPLING_STOP_TOKENS];
  // A tree block's sampled rows test the children their draft drew among SAMPLING_CANDIDATES candidates
  // (decode_sample_draw_children) instead of one child against a full-vocabulary draft distribution.
  uint32_t candidate_children;
  uint32_t reserved[2];
};

// A penalized request's word for each vocabulary token, in its row of the penalty table (the reference's
// SPLASH_PENALTY_PROMPT_BIT / _COUNT_MASK, abi/Sampling.h:120-125): the top bit marks a token of the prompt, the others
// count how often the target selected the token.
#define SAMPLING_PENALTY_PROMPT 0x80000000u
#define SAMPLING_PENALTY_COUNT 0x7FFFFFFFu
// decode_sample_penalize (the reference's SamplingPenaltyParams, abi/Sampling.h:127-142): entry e rewrites the logits
// rows of lane[e] from row table_row[e] of the penalty table. repetition_inverse is 1 / repetition, at most FLT_MAX.
struct SamplingPenaltyParams {
  uint32_t vocabulary;
  uint32_t logits_stride;
  uint32_t entries;
  uint32_t reserved;
  struct SamplingLaneRows lane[SAMPLING_MAXIMUM_LANES];
  uint32_t table_row[SAMPLING_MAXIMUM_LANES];
  float repetition[SAMPLING_MAXIMUM_LANES];
  float repetition_inverse[SAMPLING_MAXIMUM_LANES];
  float presence[SAMPLING_MAXIMUM_LANES];
  float frequency[SAMPLING_MAXIMUM_LANES];
};
// decode_sample_count_tokens: entry e adds the tokens its lane retained of a step (the first retained[lane[e]] of the
// lane's rows of the acceptance's tokens) to row table_row[e] of the penalty table.
struct SamplingCountParams {
  uint32_t vocabulary;
  uint32_t entries;
  uint32_t lane[SAMPLING_MAXIMUM_LANES];        // the entry's lane of the acceptance (its word of `retained`)
  uint32_t first_row[SAMPLING_MAXIMUM_LANES];   // that lane's first packed row
  uint32_t table_row[SAMPLING_MAXIMUM_LANES];
};

// decode_sample_end_thinking (the reference's ThinkingCutoffParams, abi/Sampling.h:147-175): where a lane's thinking
// budget runs out in a selection. Each row's path is cut at its row of depth row[lane] (for a lane of waiting_mask: at
// its first row from that depth on whose constraint-mask row admits tokens[lane][0]); the path's row of depth cut + i
// selects tokens[lane][i], for i below count[lane], unless a draft token on the path up to the cut, the anchor's
// excepted, is close[lane] (the last token of the lane's end) or also_ends[lane]: thinking ended before. A row whose
// selection is the sentinel keeps it. A lane without a cutoff has row SAMPLING_MAXIMUM_ROWS.
struct ThinkingCutoffParams {
  uint32_t vocabulary;
  uint32_t lanes;
  uint32_t waiting_mask;
  uint32_t mask_words;   // words of a constraint-mask row, one a packed row (TargetSamplingParams::mask_words)
  struct SamplingLaneRows lane[SAMPLING_MAXIMUM_LANES];
  uint32_t row[SAMPLING_MAXIMUM_LANES];
  uint32_t count[SAMPLING_MAXIMUM_LANES];
  uint32_t close[SAMPLING_MAXIMUM_LANES];
  uint32_t also_ends[SAMPLING_MAXIMUM_LANES];
  uint32_t tokens[SAMPLING_MAXIMUM_LANES][SAMPLING_MAXIMUM_ROWS];
};

// draft_verify_rows: one workgroup lays out a decode step's rows from the trees a draft selector grew (the reference's
// VerifyRowsParams, abi/Sampling.h:270-298): `rows` rows over `lanes` lanes, each lane its anchor and the best of its
// tree's other rows by estimate that the step's rows and the lanes' cap hold, none estimated below `floor`; the rows
// past the lanes' belong to no lane.
#define SAMPLING_TREE_ROOT 0xFFFFu  // the parent of a row without one (SPLASH_TREE_ROOT)
// With `slots` the rows are not packed: lane l's rows are rows l * lane_cap on (rows == lanes * lane_cap), and the rows of
// its slot past its own are inert -- token SAMPLING_NO_TOKEN (which no row selects, and whose embedding is zero), on no
// path but their own, a child of the anchor that never follows it -- so that a step recorded for lane_cap rows a lane
// takes trees of any size the device grows, with no word from the host. No counterpart in the reference, whose kernels
// read each lane's rows from the device (SplashLaneRows) where these kernels' lanes are fixed when a step is recorded.
struct VerifyRowsParams {
  uint32_t lanes;
  uint32_t rows;
  uint32_t lane_cap;
  float floor;
  uint32_t slots;
  uint32_t reserved[3];
};

// draft_select_top16_sharded, draft_select_edges (the reference's SelectorBatchParams, abi/Sampling.h:184-194, and
// abi/ExecutionGeometry.h:6-7, :60-65): a lane's draft proposes DRAFT_PROPOSAL_TOKENS positions, rows 1-7 of its
// DRAFT_QUERY_ROWS query rows, over the `columns` tokens of the draft's vocabulary: the target's first `leading`
// tokens and those from `trailing` on. A workgroup of the first kernel selects among DRAFT_SHARD_COLUMNS columns.
#define DRAFT_QUERY_ROWS 8u
#define DRAFT_PROPOSAL_TOKENS 7u
#define DRAFT_CANDIDATES 16u
#define DRAFT_SELECTOR_RANK 256u
#define DRAFT_SHARD_COLUMNS 4096u
#define DRAFT_MAXIMUM_SHARDS 128u
struct DraftSelectParams {
  uint32_t anchor[SAMPLING_MAXIMUM_LANES];
  uint32_t lanes;
  uint32_t vocabulary;
  uint32_t columns;
  uint32_t leading;
  uint32_t trailing;
  uint32_t shards;
  uint32_t reserved[2];
};

// draft_select_tree: one wavefront a lane grows the lane's tree over the candidates and edges of draft_select_edges (the
// reference's DraftTreeParams, abi/Sampling.h:209-255). A row's estimate is the probability that the target accepts the
// path to it, the product of its steps' estimates: a step to a draft candidate at proposal position p, of probability q
// among the position's candidates after its parent's, sigmoid(slope * logit(q) + intercept[p]), at most its cap (what the
// parent's host-chain child and the steps the parent drew before it left of 1); a step to host chain token d, its rate
// for its agreement with the draft at depth d (DRAFT_CHAIN_AGREEMENTS: the draft's likeliest there, another of its
// candidates, none, past its positions). The tree grows best first by estimate, a draft row taking children[l]
// candidates (a greedy lane's likeliest; a sampled lane's Gumbel-top-k draws from the probabilities at its temperature,
// with noise[l] as the anchor's key) and a chain row the chain's next token, one row a token path, until it holds
// DRAFT_TREE_ROWS rows, depth[l] + 1 rows, or nothing no deeper than depth[l] is left. Grid (lanes), 64 threads.
#define DRAFT_TREE_ROWS 16u
#define DRAFT_CHAIN_TOKENS (DRAFT_TREE_ROWS - 1u)
#define DRAFT_CHAIN_AGREEMENTS 4u
struct DraftTreeParams {
  uint32_t anchor[SAMPLING_MAXIMUM_LANES];
  uint32_t depth[SAMPLING_MAXIMUM_LANES];     // the deepest row a walk of the tree may retain
  uint32_t chain[SAMPLING_MAXIMUM_LANES];     // tokens of the lane's host chain (0: none)
  uint32_t children[SAMPLING_MAXIMUM_LANES];  // 1..SAMPLING_TREE_CHILDREN
  uint32_t lanes;
  uint32_t reserved[3];
  float slope[SAMPLING_MAXIMUM_LANES];
  float intercept[SAMPLING_MAXIMUM_LANES][DRAFT_PROPOSAL_TOKENS];
  float temperature[SAMPLING_MAXIMUM_LANES];
  uint32_t noise[SAMPLING_MAXIMUM_LANES][2];  // a 64-bit seed, low word first
};

// draft_verify_children: what a verify step's sampled rows read of the trees, row by row of the step (grid (rows), 64
// threads): a row's depth, and of the tree row it is (sources, draft_verify_rows) the candidates of its next position
// (ids, their probabilities at the lane's temperature) and the children its draft drew among them; a row of no lane, or
// one whose children would lie past the draft's positions, gets no candidates and no drawn child (SAMPLING_NO_DRAW),
// so that its selection draws from its whole distribution.
struct VerifyChildrenParams {
  uint32_t lanes;
  uint32_t rows;
  uint32_t reserved[2];
};

// decode_accept_tree: one wavefront per lane, a thread a row (the reference's AcceptBatchParams, abi/Sampling.h:314-317).
struct AcceptBatchParams {
  uint32_t lanes;
  uint32_t reserved[3];
  uint32_t remaining[SAMPLING_MAXIMUM_LANES];
  uint32_t stop_tokens[SAMPLING_STOP_TOKENS];
  struct SamplingLaneRows lane[SAMPLING_MAXIMUM_LANES];
};

#ifdef __cplusplus
static_assert(sizeof(TargetSamplingParams) == 16 + 32 + 16 + 64 + 96 + 32, "target sampling parameters are 256 bytes on both sides");
static_assert(sizeof(DraftSelectParams) == 32 + 32, "draft selector parameters are 64 bytes on both sides");
static_assert(sizeof(DraftTreeParams) == 4 * 32 + 16 + 32 + 224 + 32 + 64, "draft tree parameters are 496 bytes on both sides");
static_assert(sizeof(VerifyChildrenParams) == 16, "verify children parameters are 16 bytes on both sides");
static_assert(sizeof(VerifyRowsParams) == 32, "verify rows parameters are 32 bytes on both sides");
static_assert(sizeof(AcceptBatchParams) == 16 + 32 + 16 + 64, "acceptance parameters are 128 bytes on both sides");
#endif
