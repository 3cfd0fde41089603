// Acceptance of a verify block (the reference's kernels/decode/sampling.metal: argmax_shard
// :1896-1961, argmax_reduce :1963-1997, shard_mass / merge_masses :102-154, vocabulary_draw
// :713-885, decode_accept_tree :2044-2083), on 64-lane wavefronts.
//
// Greedy rows: SAMPLING_SHARDS workgroups scan a row's logits, each thread its tokens in id order
// (shard * 256 + tid + n * shards * 256), keeping the larger value and, among equals, the lower id;
// NaN and -inf are never selected; the shards' partials reduce by the same rule. A row with no
// selectable logit selects SAMPLING_NO_TOKEN.
//
// Sampled rows (temperature > 0): weight_t = exp((logit_t - max) / T). One pass gives each shard's
// online (max, sum), merged in shard order. The row's drafted child d is accepted iff
// u_child * q_d < p_d, p = weight / total. Otherwise the row draws from the residual
// max(p - q, 0): SAMPLING_RANGES id-ordered ranges are summed (a thread sums its chunk of a range in
// id order, the chunks are added in order), the ranges are walked in order to the one that holds
// point = u_row * sum, then its chunks and the hit chunk's tokens, each in id order; rounding
// fall-backs take the last weighted range, chunk and token. A row without a child draws the same
// way from p itself.
//
// A lane's min_p, top_k and top_p cut its rows' distributions (distribution_end, sampling.metal:
// 603-670): in the order of the logits (larger first, among equals the smaller id first) a row keeps
// the tokens at or above the logit that weighs min_p of the heaviest, then the first top_k of those,
// then of those the tokens up to the one at which their mass first exceeds top_p of the kept mass.
// The end is found by radix descent over the order-preserving key of a logit, four bits a pass, each
// pass one scan of the row with a 16-bin histogram of counts and masses (a thread's tokens in id
// order, the threads' sums in a fixed tree), then over the ids of the tokens tied at the last key.
// Everything after it weighs nothing; p is renormalized by the kept mass.
#include "abi/Sampling.h"
#include "abi/PagedAttention.h"
#include "backend/KernelRegistry.hpp"
#include "kernels/device_common.hpp"

#include <cfloat>

namespace splash::kernels {

__device__ __forceinline__ bool unselectable(float v) { return !(v > -INFINITY); }  // NaN or -inf (sampling.metal:986-989)

struct Best {
  float value;
  uint32_t index;
};
__device__ __forceinline__ Best better(Best a, Best b) {
  return (b.value > a.value || (b.value == a.value && b.index < a.index)) ? b : a;
}
__device__ __forceinline__ Best wave_best(Best v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    Best other{__shfl_xor(v.value, o, 64), __shfl_xor(v.index, o, 64)};
    v = better(v, other);
  }
  return v;
}

__device__ __forceinline__ uint32_t lane_of(const TargetSamplingParams &p, uint32_t row) {
  uint32_t lane = 0;
  for (uint32_t l = 0; l < p.lanes; ++l)
    if (row >= p.lane[l].first && row < p.lane[l].first + p.lane[l].rows) lane = l;
  return lane;
}
// decode_sample_admit: grid (rows, ceil(vocabulary / 1024)), 256 threads. A row of a constrained lane
// admits only the tokens of its constraint-mask row, a row of a lane that ignores end-of-sequence no
// stop token (TargetRow::admits, sampling.metal:42-46): the logits of the others become -infinity,
// which every selection kernel leaves out, before any of them reads the row.
__global__ __launch_bounds__(256) void decode_sample_admit(float *__restrict__ logits, const uint32_t *__restrict__ token_mask,
                                                           TargetSamplingParams p) {
  const uint32_t row = blockIdx.x, lane = lane_of(p, row);
  const bool constrained = (p.constrained_mask >> lane) & 1u, excludes = (p.exclude_stop_mask >> lane) & 1u;
  if (!constrained && !excludes) return;
  float *x = logits + size_t(row) * p.logits_stride;
  const uint32_t *mask = token_mask + size_t(row) * p.mask_words;
#pragma unroll
  for (uint32_t i = 0; i < 4; ++i) {
    const uint32_t token = (blockIdx.y * 4u + i) * 256u + threadIdx.x;
    if (token >= p.vocabulary) continue;
    bool admitted = !constrained || ((mask[token / 32u] >> (token % 32u)) & 1u);
    if (excludes)
      for (uint32_t s = 0; s < SAMPLING_STOP_TOKENS; ++s) admitted = admitted && token != p.stop_tokens[s];
    if (!admitted) x[token] = -INFINITY;
  }
}
SP_REGISTER_KERNEL("decode_sample_admit", &decode_sample_admit);

// The sampling penalties of one logit (PenaltyReference.hpp:27-40, sampling.metal:991-1006 in the reference): the
// repetition penalty divides a positive logit and multiplies another when the prompt or the output holds the token;
// presence and frequency lower it by the output's count of the token; the result stays finite. NaN and -infinity, which
// no selection takes, stay as they are. One product, one product and sum, one difference, each rounded once.
__device__ __forceinline__ float penalized_logit(float value, uint32_t count, float repetition, float repetition_inverse, float presence,
                                                 float frequency) {
  const uint32_t bits = __float_as_uint(value);
  if ((bits & 0x7FFFFFFFu) > 0x7F800000u || bits == 0xFF800000u) return value;
  float v = value * (value > 0.0f ? repetition_inverse : repetition);
  if (count) v = v - (frequency * float(count) + presence);
  return fminf(fmaxf(v, -3.402823466e+38f), 3.402823466e+38f);
}
// decode_sample_penalize: grid (ceil(vocabulary / 1024), entries), 256 threads, four tokens a thread 256 apart. A token
// that the entry's table row does not hold and no row of the block drafted is left alone (nearly every token). A row's
// context adds, to the table's count, the block's draft tokens on its path: its ancestors' and its own input token, but
// not the anchor's, which the table counted when the target selected it (sampling.metal:1008-1050).
__global__ __launch_bounds__(256) void decode_sample_penalize(float *__restrict__ logits, const uint32_t *__restrict__ words,
                                                              const uint32_t *__restrict__ input_tokens,
                                                              const AttentionTreeRow *__restrict__ tree, SamplingPenaltyParams p) {
  const uint32_t entry = blockIdx.y;
  const SamplingLaneRows lane = p.lane[entry];
  __shared__ uint32_t drafts[SAMPLING_MAXIMUM_ROWS], paths[SAMPLING_MAXIMUM_ROWS];
  if (threadIdx.x < lane.rows) {
    drafts[threadIdx.x] = input_tokens[lane.first + threadIdx.x];
    paths[threadIdx.x] = tree[lane.first + threadIdx.x].ancestors & ~1u;
  }
  __syncthreads();
  const float repetition = p.repetition[entry], inverse = p.repetition_inverse[entry], presence = p.presence[entry],
              frequency = p.frequency[entry];
  const uint32_t *row_words = words + size_t(p.table_row[entry]) * p.vocabulary;
#pragma unroll
  for (uint32_t i = 0; i < 4; ++i) {
    const uint32_t token = (blockIdx.x * 4u + i) * 256u + threadIdx.x;
    if (token >= p.vocabulary) continue;
    const uint32_t word = row_words[token];
    uint32_t drafted = 0;
    for (uint32_t r = 1; r < lane.rows; ++r) drafted |= uint32_t(drafts[r] == token) << r;
    if (!(word | drafted)) continue;
    const uint32_t selected = word & SAMPLING_PENALTY_COUNT;
    float *column = logits + size_t(lane.first) * p.logits_stride + token;
    for (uint32_t r = 0; r < lane.rows; ++r) {
      const uint32_t count = selected + uint32_t(__popc(drafted & paths[r]));
      if (!count && !(word & SAMPLING_PENALTY_PROMPT)) continue;
      float &x = column[size_t(r) * p.logits_stride];
      x = penalized_logit(x, count, repetition, inverse, presence, frequency);
    }
  }
}
SP_REGISTER_KERNEL("decode_sample_penalize", &decode_sample_penalize);

// decode_sample_count_tokens: grid (entries), 64 threads. The tokens a lane retained of a step (the acceptance's `tokens`
// from the lane's first row, `retained` of them) are counted into its row of the penalty table on the device, where the
// reference's engine counts them on the host into shared memory (Sampling::countPenaltyTokens, Sampling.cpp:116-121).
// A token twice in one step is counted twice (atomic adds).
__global__ __launch_bounds__(64) void decode_sample_count_tokens(uint32_t *__restrict__ words, const uint32_t *__restrict__ tokens,
                                                                 const uint32_t *__restrict__ retained, SamplingCountParams p) {
  const uint32_t entry = blockIdx.x;
  const uint32_t count = min(retained[p.lane[entry]], uint32_t(SAMPLING_MAXIMUM_ROWS));
  if (threadIdx.x >= count) return;
  const uint32_t token = tokens[p.first_row[entry] + threadIdx.x];
  if (token < p.vocabulary) atomicAdd(words + size_t(p.table_row[entry]) * p.vocabulary + token, 1u);
}
SP_REGISTER_KERNEL("decode_sample_count_tokens", &decode_sample_count_tokens);

// decode_sample_end_thinking: grid (lanes), 64 threads, a thread a row of the lane's block (the reference walks a lane's
// rows in one thread, sampling.metal:1993-2039; every row reads and writes its own selection only, so they go side by
// side). The k-th row of a path, ascending, is its row of depth k.
__global__ __launch_bounds__(64) void decode_sample_end_thinking(const uint32_t *__restrict__ input_tokens,
                                                                 const uint32_t *__restrict__ token_mask,
                                                                 const AttentionTreeRow *__restrict__ tree, uint32_t *__restrict__ tokens,
                                                                 ThinkingCutoffParams p) {
  const uint32_t lane = blockIdx.x;
  const SamplingLaneRows block = p.lane[lane];
  if (threadIdx.x >= block.rows || p.row[lane] >= SAMPLING_MAXIMUM_ROWS) return;
  const uint32_t mine = block.first + threadIdx.x;
  const uint32_t path = tree[mine].ancestors, depth = tree[mine].depth;
  const bool waits = (p.waiting_mask >> lane) & 1u;
  const uint32_t start = p.tokens[lane][0];
  // the cut: the first depth from the lane's row on (whose row admits the end's first token, where the end waits)
  uint32_t cut = 0, left = path;
  bool found = false;
  for (; left; left &= left - 1u, ++cut) {
    if (cut < p.row[lane]) continue;
    const uint32_t at = block.first + uint32_t(__ffs(int(left)) - 1);
    if (!waits || ((token_mask[size_t(at) * p.mask_words + start / 32u] >> (start % 32u)) & 1u)) {
      found = true;
      break;
    }
  }
  if (!found || cut > depth || depth - cut >= p.count[lane]) return;
  // thinking that a draft token ended at or before the cut stays ended
  for (uint32_t before = path & ~1u; before; before &= before - 1u) {
    const uint32_t at = block.first + uint32_t(__ffs(int(before)) - 1);
    const uint32_t draft = input_tokens[at];
    if (tree[at].depth <= cut && (draft == p.close[lane] || draft == p.also_ends[lane])) return;
  }
  if (tokens[mine] < p.vocabulary) tokens[mine] = p.tokens[lane][depth - cut];
}
SP_REGISTER_KERNEL("decode_sample_end_thinking", &decode_sample_end_thinking);


// draft_verify_rows (the layout the reference's sampling.metal:1799-1895 produces): lane l's tree holds sizes[l] rows
// from row l * 16 of tree_tokens, trees and scores (a row's draft probability and its estimate, the chance that the
// target accepts it), in the order the selector took them, best first. The step takes every lane's anchor and the
// best other rows by estimate (among equals the lower lane, then the lower row) that its rows and the lanes' cap
// hold, none below the floor; a lane's rows are numbered in preorder, the earlier-taken child first, so that the
// likeliest path of its tree lies on its first rows; the rows of no lane carry lane 0's anchor, no path and no source.
//
// One workgroup of 128 threads, thread (lane, row) = (t / 16, t % 16), no loop over the step's rows:
//   rank      a candidate's place in the order above is the count of candidates that beat it;
//   take      in that order a candidate is eligible if it is at or above the floor and fewer than cap - 1 candidates
//             of its lane precede it; it is taken if fewer than rows - lanes eligible ones precede it (wave ballots
//             over the ranked order);
//   preorder  with ancestor masks, row x precedes row r if x is an ancestor of r or, where their paths part, x's
//             branch was taken earlier (parents are taken before children, so the lowest set bit of a path below
//             the common part is its branch): r's place is the count of the lane's rows that precede it.
__global__ __launch_bounds__(128) void draft_verify_rows(const uint32_t *__restrict__ tree_tokens, const AttentionTreeRow *__restrict__ trees,
                                                         const float2 *__restrict__ scores, const uint32_t *__restrict__ sizes,
                                                         uint32_t *__restrict__ tokens, AttentionTreeRow *__restrict__ tree,
                                                         SamplingLaneRows *__restrict__ lane_rows, uint32_t *__restrict__ sources,
                                                         VerifyRowsParams p) {
  constexpr uint32_t kLanes = SAMPLING_MAXIMUM_LANES, kRows = SAMPLING_MAXIMUM_ROWS, kAll = kLanes * kRows;
  __shared__ float estimateOf[kAll];
  __shared__ uint32_t rankedOwner[kAll];   // the lane of the candidate at each place of the order, kLanes for none
  __shared__ float rankedEstimate[kAll];
  __shared__ uint32_t eligibleBefore[2];   // eligible candidates in the first wave's places
  __shared__ uint32_t takenOf[kLanes];
  __shared__ uint32_t pathOf[kAll];        // a row's ancestors and itself, in its tree's own numbering
  __shared__ uint32_t placeOf[kAll];       // a row's place in its lane's preorder
  if (blockIdx.x) return;
  const uint32_t t = threadIdx.x, lane = t / kRows, row = t % kRows, lanes = min(p.lanes, kLanes);
  const uint32_t size = lane < lanes ? min(sizes[lane], kRows) : 0u;
  const bool candidate = row >= 1 && row < size;
  const float estimate = candidate ? scores[t].y : 0.f;
  estimateOf[t] = candidate ? estimate : -INFINITY;
  rankedOwner[t] = kLanes;
  rankedEstimate[t] = -INFINITY;
  if (t < kLanes) takenOf[t] = 0;
  __syncthreads();
  if (candidate) {
    uint32_t rank = 0;
    for (uint32_t other = 0; other < kAll; ++other) {
      const float e = estimateOf[other];
      rank += (e > estimate || (e == estimate && other < t)) && (other % kRows) >= 1 && e != -INFINITY ? 1u : 0u;
    }
    rankedOwner[rank] = lane;
    rankedEstimate[rank] = estimate;
  }
  __syncthreads();
  // Thread t now stands for place t of the order.
  const uint32_t owner = rankedOwner[t];
  uint32_t before = 0;   // candidates of the same lane at earlier places
  for (uint32_t place = 0; place < t; ++place) before += rankedOwner[place] == owner ? 1u : 0u;
  const bool eligible = owner < kLanes && !(rankedEstimate[t] < p.floor) && before + 1u < p.lane_cap;
  const uint64_t ballot = __builtin_amdgcn_ballot_w64(eligible);
  if ((t & 63u) == 0) eligibleBefore[t >> 6] = uint32_t(__builtin_popcountll(ballot));
  __syncthreads();
  const uint32_t earlier = uint32_t(__builtin_popcountll(ballot & ((uint64_t{1} << (t & 63u)) - 1u))) + (t >= 64 ? eligibleBefore[0] : 0u);
  const uint32_t budget = p.rows > lanes ? p.rows - lanes : 0u;
  if (eligible && earlier < budget) atomicAdd(&takenOf[owner], 1u);
  __syncthreads();
  // Back to thread (lane, row): the lane keeps its anchor and its first taken rows.
  const uint32_t mine = lane < lanes ? takenOf[lane] + 1u : 0u;
  uint32_t first = 0, total = 0;
  for (uint32_t l = 0; l < lanes; ++l) {
    first += l < lane ? takenOf[l] + 1u : 0u;
    total += takenOf[l] + 1u;
  }
  if (p.slots) first = lane * p.lane_cap;
  const bool placed = row < mine;
  const AttentionTreeRow node = placed ? trees[t] : AttentionTreeRow{0u, 0u, 0u};
  pathOf[t] = placed ? node.ancestors : 0u;
  __syncthreads();
  uint32_t place = 0;
  if (placed) {
    const uint32_t path = node.ancestors;
    for (uint32_t x = 0; x < mine; ++x) {
      if (x == row) continue;
      const uint32_t other = pathOf[lane * kRows + x], common = other & path;
      const bool ancestor = (path >> x) & 1u, descendant = (other >> row) & 1u;
      const bool earlierBranch = __builtin_ctz((other & ~common) | 0x10000u) < __builtin_ctz((path & ~common) | 0x10000u);
      place += ancestor || (!descendant && earlierBranch) ? 1u : 0u;
    }
  }
  placeOf[t] = place;
  __syncthreads();
  if (placed) {
    uint32_t ancestors = 0;
    for (uint32_t walk = node.ancestors; walk; walk &= walk - 1u) ancestors |= 1u << placeOf[lane * kRows + uint32_t(__builtin_ctz(walk))];
    const uint32_t depth = uint32_t(__builtin_popcount(node.ancestors)) - 1u;
    const uint32_t up = row ? placeOf[lane * kRows + node.parent] : SAMPLING_TREE_ROOT;
    tokens[first + place] = tree_tokens[t];
    tree[first + place] = AttentionTreeRow{ancestors, uint16_t(up), uint16_t(depth)};
    sources[first + place] = row;
  }
  if (lane < lanes && row == 0) lane_rows[lane] = SamplingLaneRows{first, mine};
  if (p.slots) {
    // the rows of a lane's slot past its own: inert
    if (lane < lanes && row >= mine && row < p.lane_cap) {
      tokens[first + row] = SAMPLING_NO_TOKEN;
      tree[first + row] = AttentionTreeRow{1u << row, uint16_t(0), uint16_t(1)};
      sources[first + row] = SAMPLING_NO_TOKEN;
    }
    return;
  }
  for (uint32_t spare = total + t; spare < p.rows; spare += kAll) {
    tokens[spare] = tree_tokens[0];
    tree[spare] = AttentionTreeRow{0u, uint16_t(SAMPLING_TREE_ROOT), uint16_t(0)};
    sources[spare] = SAMPLING_NO_TOKEN;
  }
}
SP_REGISTER_KERNEL("draft_verify_rows", &draft_verify_rows);

// Grid (rows * SAMPLING_SHARDS), 256 threads. partial_values/indices [row][shard].
__global__ __launch_bounds__(256) void decode_sample_argmax_sharded(const float *__restrict__ logits, float *__restrict__ partial_values,
                                                                    uint32_t *__restrict__ partial_indices, TargetSamplingParams p) {
  __shared__ float values[4];
  __shared__ uint32_t indices[4];
  const uint32_t row = blockIdx.x / SAMPLING_SHARDS, shard = blockIdx.x % SAMPLING_SHARDS, tid = threadIdx.x;
  const float *x = logits + size_t(row) * p.logits_stride;
  Best best{-INFINITY, SAMPLING_NO_TOKEN};
  for (uint32_t token = shard * 256u + tid; token < p.vocabulary; token += SAMPLING_SHARDS * 256u) {
    const float value = __builtin_nontemporal_load(x + token);
    if (unselectable(value)) continue;
    if (value > best.value || (value == best.value && token < best.index)) best = {value, token};
  }
  best = wave_best(best);
  if ((tid & 63u) == 0) {
    values[tid >> 6] = best.value;
    indices[tid >> 6] = best.index;
  }
  __syncthreads();
  if (tid == 0) {
    Best all{values[0], indices[0]};
#pragma unroll
    for (int w = 1; w < 4; ++w) all = better(all, Best{values[w], indices[w]});
    partial_values[blockIdx.x] = all.value;
    partial_indices[blockIdx.x] = all.index;
  }
}
SP_REGISTER_KERNEL("decode_sample_argmax_sharded", &decode_sample_argmax_sharded);

// Grid (rows), 64 threads: the row's token from its shards' partials.
__global__ __launch_bounds__(64) void decode_sample_argmax_reduce(const float *__restrict__ partial_values,
                                                                  const uint32_t *__restrict__ partial_indices,
                                                                  uint32_t *__restrict__ tokens, TargetSamplingParams p) {
  const uint32_t row = blockIdx.x, tid = threadIdx.x;
  Best best{-INFINITY, SAMPLING_NO_TOKEN};
  if (tid < SAMPLING_SHARDS) best = {partial_values[row * SAMPLING_SHARDS + tid], partial_indices[row * SAMPLING_SHARDS + tid]};
  if (unselectable(best.value)) best = {-INFINITY, SAMPLING_NO_TOKEN};
  best = wave_best(best);
  if (tid == 0) tokens[row] = best.index;
}
SP_REGISTER_KERNEL("decode_sample_argmax_reduce", &decode_sample_argmax_reduce);

// decode_accept_tree (what the reference's sampling.metal:2044-2083 decides): grid (lanes), one wavefront a lane, a
// thread a row. tokens: in, each row's selection; out, the lane's retained tokens from its first row.
// A row follows its parent when its input token is the parent's selection and no earlier row of the same parent
// does (one ballot); a row lies on the accepted path when every row of its ancestor mask follows its parent. The
// path's rows, by depth, are the accepted draft tokens' rows; each selects the next token of the output, the last
// the target's own. The output is cut to what the lane may still keep and after its first stop token (a second
// ballot); the retained rows are the ancestor mask of the last kept row.
__global__ __launch_bounds__(64) void decode_accept_tree(const uint32_t *__restrict__ input_tokens, const AttentionTreeRow *__restrict__ tree,
                                                         uint32_t *__restrict__ tokens, uint32_t *__restrict__ retained,
                                                         uint32_t *__restrict__ accepted_count, uint32_t *__restrict__ retained_rows,
                                                         AcceptBatchParams p) {
  const uint32_t lane = blockIdx.x, row = threadIdx.x;
  if (lane >= p.lanes) return;
  const uint32_t first = p.lane[lane].first, rows = min(p.lane[lane].rows, SAMPLING_MAXIMUM_ROWS);
  const bool live = row < rows;
  const AttentionTreeRow node = live ? tree[first + row] : AttentionTreeRow{0u, 0u, 0u};
  const uint32_t input = live ? input_tokens[first + row] : 0u, selection = live ? tokens[first + row] : 0u;
  const uint32_t parent = live && row ? min(uint32_t(node.parent), SAMPLING_MAXIMUM_ROWS - 1u) : 0u;
  const uint32_t parentSelection = __shfl(selection, int(parent), 64);
  const bool matches = live && row && node.parent < row && input == parentSelection;
  // the matching rows of this row's parent before it
  uint32_t siblingsBefore = 0;
  for (uint32_t other = 1; other < rows; ++other) {
    const bool sameParent = __shfl(matches ? int(parent) : -1, int(other), 64) == int(parent);
    siblingsBefore += other < row && sameParent ? 1u : 0u;
  }
  const bool follows = matches && !siblingsBefore;
  const uint32_t following = uint32_t(__builtin_amdgcn_ballot_w64(follows)) | 1u;   // the anchor starts the path
  const bool onPath = live && (node.ancestors & ~following) == 0u && ((node.ancestors >> row) & 1u);
  const uint32_t path = uint32_t(__builtin_amdgcn_ballot_w64(onPath));
  const uint32_t accepted = uint32_t(__builtin_popcount(path)) - 1u;
  const uint32_t depth = live ? uint32_t(__builtin_popcount(path & ((1u << row) - 1u))) : 0u;   // the path's rows rise with depth
  uint32_t kept = min(accepted + 1u, max(p.remaining[lane], 1u));
  bool stop = false;
#pragma unroll
  for (int s = 0; s < int(SAMPLING_STOP_TOKENS); ++s) stop = stop || (p.stop_tokens[s] != SAMPLING_NO_TOKEN && selection == p.stop_tokens[s]);
  // the shallowest path row within the kept ones that selects a stop token ends the output
  const uint32_t stops = uint32_t(__builtin_amdgcn_ballot_w64(onPath && depth < kept && stop));
  if (stops) kept = uint32_t(__builtin_popcount(path & ((2u << __builtin_ctz(stops)) - 1u)));
  if (onPath && depth < kept) tokens[first + depth] = selection;   // every selection was read before any is written
  if (onPath && depth + 1u == kept) {
    retained_rows[lane] = node.ancestors;
    retained[lane] = kept;
    accepted_count[lane] = min(accepted, kept);
  }
}
SP_REGISTER_KERNEL("decode_accept_tree", &decode_accept_tree);

// ---------------------------------------------------------------------------------------------
// Sampled rows.
// ---------------------------------------------------------------------------------------------
struct Mass {
  float maximum, sum;
};
// merge_masses (sampling.metal:122-154): the larger maximum first, then both sums at it.
__device__ __forceinline__ Mass merge(Mass a, Mass b, float inverse_temperature) {
  const float m = fmaxf(a.maximum, b.maximum);
  if (m == -INFINITY) return {m, 0.f};
  const float sa = a.maximum == -INFINITY ? 0.f : a.sum * expf((a.maximum - m) * inverse_temperature);
  const float sb = b.maximum == -INFINITY ? 0.f : b.sum * expf((b.maximum - m) * inverse_temperature);
  return {m, sa + sb};
}
__device__ __forceinline__ uint32_t lane_of_row(const TargetSamplingParams &p, uint32_t row) {
  uint32_t lane = 0;
  for (uint32_t l = 0; l < p.lanes; ++l)
    if (row >= p.lane[l].first && row < p.lane[l].first + p.lane[l].rows) lane = l;
  return lane;
}

// Grid (rows * SAMPLING_SHARDS), 256 threads: the shard's online (max, sum). masses [row][shard][2].
__global__ __launch_bounds__(256) void decode_sample_mass_sharded(const float *__restrict__ logits, float *__restrict__ masses,
                                                                  TargetSamplingParams p) {
  __shared__ float shared[4][2];
  const uint32_t row = blockIdx.x / SAMPLING_SHARDS, shard = blockIdx.x % SAMPLING_SHARDS, tid = threadIdx.x;
  const float inverse = 1.0f / p.temperature[lane_of_row(p, row)];
  const float *x = logits + size_t(row) * p.logits_stride;
  Mass mine{-INFINITY, 0.f};
  for (uint32_t token = shard * 256u + tid; token < p.vocabulary; token += SAMPLING_SHARDS * 256u) {
    const float value = __builtin_nontemporal_load(x + token);
    if (unselectable(value)) continue;
    mine = merge(mine, Mass{value, 1.0f}, inverse);
  }
  // lanes in a fixed butterfly, then the four wavefronts in order
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mine = merge(mine, Mass{__shfl_xor(mine.maximum, o, 64), __shfl_xor(mine.sum, o, 64)}, inverse);
  if ((tid & 63u) == 0) {
    shared[tid >> 6][0] = mine.maximum;
    shared[tid >> 6][1] = mine.sum;
  }
  __syncthreads();
  if (tid == 0) {
    Mass all{shared[0][0], shared[0][1]};
#pragma unroll
    for (int w = 1; w < 4; ++w) all = merge(all, Mass{shared[w][0], shared[w][1]}, inverse);
    masses[2 * blockIdx.x] = all.maximum;
    masses[2 * blockIdx.x + 1] = all.sum;
  }
}
SP_REGISTER_KERNEL("decode_sample_mass_sharded", &decode_sample_mass_sharded);

// The row's (max, total) from its shards, in shard order.
__device__ __forceinline__ Mass row_mass(const float *masses, uint32_t row, float inverse) {
  Mass all{masses[2 * row * SAMPLING_SHARDS], masses[2 * row * SAMPLING_SHARDS + 1]};
  for (uint32_t s = 1; s < SAMPLING_SHARDS; ++s)
    all = merge(all, Mass{masses[2 * (row * SAMPLING_SHARDS + s)], masses[2 * (row * SAMPLING_SHARDS + s) + 1]}, inverse);
  return all;
}
// The child of `row` in its lane's block: the first later row whose parent it is; none: SAMPLING_NO_TOKEN.
__device__ __forceinline__ uint32_t child_token(const TargetSamplingParams &p, const AttentionTreeRow *tree,
                                                const uint32_t *input_tokens, uint32_t row) {
  const uint32_t lane = lane_of_row(p, row), first = p.lane[lane].first, local = row - first;
  for (uint32_t child = local + 1; child < p.lane[lane].rows; ++child)
    if (tree[first + child].parent == local) return input_tokens[first + child];
  return SAMPLING_NO_TOKEN;
}
// The order of the logits as an unsigned key (sampling.metal:197-207): a larger logit has a larger
// key; -0 and +0 share one; every finite logit's key is above that of -infinity.
__device__ __forceinline__ uint32_t logit_key(float value) {
  uint32_t bits = __builtin_bit_cast(uint32_t, value);
  bits = (bits << 1) ? bits : 0u;
  return (bits & 0x80000000u) ? ~bits : bits | 0x80000000u;
}
__device__ __forceinline__ float key_logit(uint32_t key) {
  return __builtin_bit_cast(float, (key & 0x80000000u) ? key & 0x7FFFFFFFu : ~key);
}
constexpr uint32_t kLowestKey = 0x007FFFFFu;  // of -infinity
// A position in the order: the tokens at or before it have a larger key, or its key and an id at
// most `last`. {0, 0} lies after every token.
struct OrderEnd {
  uint32_t key, last;
};
__device__ __forceinline__ bool at_or_before(uint32_t key, uint32_t token, OrderEnd end) {
  return key > end.key || (key == end.key && token <= end.last);
}
// A row's distribution: its maximum, the mass of the tokens it keeps and the last of them.
struct Kept {
  Mass mass;  // maximum, kept mass
  OrderEnd end;
};
__device__ __forceinline__ Kept row_kept(const float *masses, const uint32_t *decisions, uint32_t row, float inverse, bool truncating) {
  Kept kept{row_mass(masses, row, inverse), {0u, 0u}};
  if (truncating) {
    const uint32_t *words = decisions + size_t(row) * SAMPLING_DECISION_WORDS;
    kept.end = {words[SAMPLING_END_KEY], words[SAMPLING_END_LAST]};
    kept.mass.sum = __builtin_bit_cast(float, words[SAMPLING_END_MASS]);
  }
  return kept;
}
__device__ __forceinline__ float token_weight(float logit, Mass mass, float inverse) {
  return unselectable(logit) ? 0.f : expf((logit - mass.maximum) * inverse);
}
// A token's weight in the row's distribution: its softmax weight at or before the end, else 0 (kept_weight, sampling.metal:672-679).
__device__ __forceinline__ float kept_weight(float logit, uint32_t token, const Kept &kept, float inverse) {
  if (unselectable(logit) || !at_or_before(logit_key(logit), token, kept.end)) return 0.f;
  return expf((logit - kept.mass.maximum) * inverse);
}
// The residual weight of token t: max(p_t - q_t, 0) after a rejection, p_t's weight otherwise.
__device__ __forceinline__ float residual_of(float logit, uint32_t token, float q, const Kept &kept, float inverse, bool rejected) {
  const float w = kept_weight(logit, token, kept, inverse);
  return rejected ? fmaxf(w / kept.mass.sum - q, 0.f) : w;
}
// ---------------------------------------------------------------------------------------------
// decode_sample_distribution_end: grid (rows), 256 threads. Writes the row's end words of the
// decisions buffer; rows of lanes that keep every token are left alone.
// ---------------------------------------------------------------------------------------------
struct Measure {
  uint32_t count;
  float mass;
};
struct EndScratch {
  float mass[16][SAMPLING_THREADS];
  uint32_t count[16][SAMPLING_THREADS];
  float binMass[16];
  uint32_t binCount[16];
};
// One scan of the row: the 16-bin histogram of `digit(token, key)` (0..15, or 16 to leave a token
// out) over the selectable tokens at or before `end`, into scratch.binCount / binMass.
template <class Digit>
__device__ __forceinline__ void end_histogram(const float *x, uint32_t vocabulary, Mass mass, float inverse, OrderEnd end, Digit digit,
                                              EndScratch &scratch, uint32_t tid) {
#pragma unroll
  for (uint32_t b = 0; b < 16; ++b) {
    scratch.mass[b][tid] = 0.f;
    scratch.count[b][tid] = 0u;
  }
  for (uint32_t token = tid; token < vocabulary; token += SAMPLING_THREADS) {
    const float value = x[token];
    if (unselectable(value)) continue;
    const uint32_t key = logit_key(value);
    if (!at_or_before(key, token, end)) continue;
    const uint32_t b = digit(token, key);
    if (b >= 16u) continue;
    scratch.mass[b][tid] += expf((value - mass.maximum) * inverse);
    scratch.count[b][tid] += 1u;
  }
  __syncthreads();
  // Wavefront w sums bins 4 w .. 4 w + 3: a lane its four threads in order, the lanes in a fixed butterfly.
  const uint32_t lane = tid & 63u, wave = tid >> 6;
#pragma unroll
  for (uint32_t i = 0; i < 4; ++i) {
    const uint32_t b = 4u * wave + i;
    float m = ((scratch.mass[b][lane] + scratch.mass[b][lane + 64u]) + scratch.mass[b][lane + 128u]) + scratch.mass[b][lane + 192u];
    uint32_t c = scratch.count[b][lane] + scratch.count[b][lane + 64u] + scratch.count[b][lane + 128u] + scratch.count[b][lane + 192u];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      m += __shfl_xor(m, o, 64);
      c += uint32_t(__shfl_xor(int(c), o, 64));
    }
    if (lane == 0) {
      scratch.binMass[b] = m;
      scratch.binCount[b] = c;
    }
  }
  __syncthreads();
}
// The last token kept of the tokens at or before `end` (of which `all` measures everything), in
// order until their count exceeds `countTarget` (ByMass false) or their mass `massTarget` (ByMass
// true); `kept` becomes the measure of the kept tokens. Every thread returns the same.
template <bool ByMass>
__device__ OrderEnd select_last(const float *x, uint32_t vocabulary, Mass mass, float inverse, OrderEnd end, uint32_t countTarget,
                                float massTarget, Measure &kept, EndScratch &scratch, uint32_t tid) {
  auto exceeded = [&](Measure m) { return ByMass ? m.mass > massTarget : m.count > countTarget; };
  Measure above{0u, 0.f};
  uint32_t prefix = 0, tied = 0;
  for (int shift = 28; shift >= 0; shift -= 4) {
    const uint32_t high = shift == 28 ? 0u : prefix >> (shift + 4);
    end_histogram(x, vocabulary, mass, inverse, end,
                  [&](uint32_t, uint32_t key) { return shift != 28 && (key >> (shift + 4)) != high ? 16u : (key >> shift) & 15u; }, scratch, tid);
    int chosen = -1, lowest = -1;
    Measure cumulative = above;
    for (int b = 15; b >= 0 && chosen < 0; --b) {
      if (!scratch.binCount[b]) continue;
      const Measure next{cumulative.count + scratch.binCount[b], cumulative.mass + scratch.binMass[b]};
      lowest = b;
      if (exceeded(next)) chosen = b;
      else cumulative = next;
    }
    if (chosen < 0) {
      // The target is never exceeded: at the first pass every token stays; below it (a bin's mass and
      // its parts' may round apart) the search ends in the last bin that holds a token.
      if (shift == 28 || lowest < 0) {
        kept = cumulative;
        __syncthreads();
        return end;
      }
      chosen = lowest;
      cumulative = {cumulative.count - scratch.binCount[lowest], cumulative.mass - scratch.binMass[lowest]};
    }
    above = cumulative;
    prefix |= uint32_t(chosen) << shift;
    tied = scratch.binCount[chosen];
    __syncthreads();  // every thread has read the bins before the next pass clears them
  }
  // `tied` tokens share the key `prefix` and one weight: as many of them stay as the target takes.
  const float weight = expf((key_logit(prefix) - mass.maximum) * inverse);
  uint32_t keep;
  if (ByMass) {
    keep = weight > 0.f ? uint32_t(fminf(fmaxf((massTarget - above.mass) / weight, 0.f), float(tied))) : tied;
    keep = min(max(keep, 1u), tied);
    while (keep > 1u && above.mass + float(keep - 1u) * weight > massTarget) --keep;
    while (keep < tied && !(above.mass + float(keep) * weight > massTarget)) ++keep;
  } else {
    keep = min(max(countTarget + 1u - above.count, 1u), tied);
  }
  kept = {above.count + keep, above.mass + float(keep) * weight};
  OrderEnd last{prefix, 0xFFFFFFFFu};
  if (keep < tied) {
    // The keep-th smallest id of the tied tokens at or before `end`, by the same descent over ids.
    uint32_t bits = 4;
    while (bits < 32 && (vocabulary - 1u) >> bits) bits += 4;
    uint32_t id = 0, before = 0;
    for (int shift = int(bits) - 4; shift >= 0; shift -= 4) {
      const uint32_t high = shift + 4 >= 32 ? 0u : id >> (shift + 4);
      end_histogram(x, vocabulary, mass, inverse, end,
                    [&](uint32_t token, uint32_t key) {
                      return key != prefix || (shift + 4 < 32 && (token >> (shift + 4)) != high) ? 16u : (token >> shift) & 15u;
                    },
                    scratch, tid);
      uint32_t chosen = 15;
      for (uint32_t b = 0; b < 16; ++b) {
        if (before + scratch.binCount[b] >= keep) {
          chosen = b;
          break;
        }
        before += scratch.binCount[b];
      }
      id |= chosen << shift;
      __syncthreads();
    }
    last.last = id;
  }
  return last;
}

__global__ __launch_bounds__(SAMPLING_THREADS) void decode_sample_distribution_end(const float *__restrict__ logits,
                                                                                  const float *__restrict__ masses,
                                                                                  uint32_t *__restrict__ decisions, TargetSamplingParams p) {
  __shared__ EndScratch scratch;
  const uint32_t row = blockIdx.x, tid = threadIdx.x, laneIndex = lane_of_row(p, row);
  if (!((p.truncating_mask >> laneIndex) & 1u)) return;
  const float temperature = p.temperature[laneIndex], inverse = 1.0f / temperature;
  const Mass mass = row_mass(masses, row, inverse);
  const float *x = logits + size_t(row) * p.logits_stride;
  const float minP = p.min_p[laneIndex], topP = p.top_p[laneIndex];
  const uint32_t topK = p.top_k[laneIndex];
  OrderEnd end{0u, 0u};
  // Everything, and what min_p keeps: the tokens at or above the logit that weighs min_p of the heaviest.
  const uint32_t lowest = minP > 0.f ? logit_key(fminf(mass.maximum + temperature * logf(minP), mass.maximum)) : kLowestKey;
  end_histogram(x, p.vocabulary, mass, inverse, end, [&](uint32_t, uint32_t key) { return key >= lowest ? 1u : 0u; }, scratch, tid);
  Measure kept{scratch.binCount[1], scratch.binMass[1]};
  const uint32_t admitted = scratch.binCount[0] + scratch.binCount[1];
  __syncthreads();
  if (minP > 0.f && kept.count < admitted) end = {lowest, 0xFFFFFFFFu};
  if (topK && topK < kept.count) end = select_last<false>(x, p.vocabulary, mass, inverse, end, topK - 1u, 0.f, kept, scratch, tid);
  if (topP < 1.0f) end = select_last<true>(x, p.vocabulary, mass, inverse, end, 0u, topP * kept.mass, kept, scratch, tid);
  if (tid == 0) {
    uint32_t *words = decisions + size_t(row) * SAMPLING_DECISION_WORDS;
    words[SAMPLING_END_KEY] = end.key;
    words[SAMPLING_END_LAST] = end.last;
    words[SAMPLING_END_MASS] = __builtin_bit_cast(uint32_t, kept.mass);
    words[SAMPLING_END_COUNT] = kept.count;
  }
}
SP_REGISTER_KERNEL("decode_sample_distribution_end", &decode_sample_distribution_end);

constexpr uint32_t kChunks = SAMPLING_THREADS;  // chunks of a range, one per thread
__device__ __forceinline__ uint32_t range_tokens(uint32_t vocabulary) {
  return (vocabulary + SAMPLING_RANGES - 1) / SAMPLING_RANGES;
}
__device__ __forceinline__ uint32_t chunk_tokens(uint32_t vocabulary) { return (range_tokens(vocabulary) + kChunks - 1) / kChunks; }

// Grid (rows * SAMPLING_RANGES / 4), 256 threads: each wavefront sums one range; thread 0 of the
// row's first workgroup also records the rejection test. ranges [row][SAMPLING_RANGES];
// decisions [row][2]: the accepted child token or SAMPLING_NO_TOKEN when the row must draw, and
// whether it draws from the residual (1) or from p (0). uniforms [row][2]: the row's draw, its child's test.
__global__ __launch_bounds__(256) void decode_sample_residual_ranges(const float *__restrict__ logits, const float *__restrict__ draft,
                                                                     const float *__restrict__ masses, const float *__restrict__ uniforms,
                                                                     const AttentionTreeRow *__restrict__ tree,
                                                                     const uint32_t *__restrict__ input_tokens,
                                                                     float *__restrict__ ranges, uint32_t *__restrict__ decisions,
                                                                     TargetSamplingParams p) {
  constexpr uint32_t kPerRow = SAMPLING_RANGES / 4;
  const uint32_t row = blockIdx.x / kPerRow, range = (blockIdx.x % kPerRow) * 4u + (threadIdx.x >> 6), lane = threadIdx.x & 63u;
  const uint32_t laneIndex = lane_of_row(p, row);
  const float inverse = 1.0f / p.temperature[laneIndex];
  const Kept kept = row_kept(masses, decisions, row, inverse, (p.truncating_mask >> laneIndex) & 1u);
  const float *x = logits + size_t(row) * p.logits_stride, *q = draft + size_t(row) * p.logits_stride;
  // a row that tests candidate children sums the ranges of its whole distribution: the draw kernel does the tests
  const uint32_t child = p.candidate_children ? SAMPLING_NO_TOKEN : child_token(p, tree, input_tokens, row);
  bool rejected = false;
  if (child != SAMPLING_NO_TOKEN && child < p.vocabulary) {
    // accept iff u_child * q < p (sampling.metal:790-800)
    const float pc = kept_weight(x[child], child, kept, inverse) / kept.mass.sum;
    rejected = !(uniforms[2 * row + 1] * q[child] < pc);
    if (blockIdx.x % kPerRow == 0 && threadIdx.x == 0) {
      decisions[SAMPLING_DECISION_WORDS * row] = rejected ? SAMPLING_NO_TOKEN : child;
      decisions[SAMPLING_DECISION_WORDS * row + 1] = rejected ? 1u : 0u;
    }
  } else if (blockIdx.x % kPerRow == 0 && threadIdx.x == 0) {
    decisions[SAMPLING_DECISION_WORDS * row] = SAMPLING_NO_TOKEN;
    decisions[SAMPLING_DECISION_WORDS * row + 1] = 0u;
  }
  if (child != SAMPLING_NO_TOKEN && child < p.vocabulary && !rejected) return;  // accepted: nothing to draw
  // the range's residual: a lane sums its tokens in id order, the lanes are added in order
  const uint32_t size = range_tokens(p.vocabulary), begin = range * size, end = min(p.vocabulary, begin + size);
  const uint32_t per = (size + 63u) / 64u;
  float sum = 0.f;
  for (uint32_t i = 0; i < per; ++i) {
    const uint32_t token = begin + lane * per + i;
    if (token < end) sum += residual_of(x[token], token, rejected ? q[token] : 0.f, kept, inverse, rejected);
  }
  float total = 0.f;
  for (int l = 0; l < 64; ++l) total += __shfl(sum, l, 64);
  if (lane == 0) ranges[row * SAMPLING_RANGES + range] = total;
}
SP_REGISTER_KERNEL("decode_sample_residual_ranges", &decode_sample_residual_ranges);

// Grid (rows), 64 threads: the row's selection. A sampled row whose child was accepted selects it;
// otherwise it draws at point = u_row * sum of the ranges, from the residual when its child was
// rejected (decisions[2 row + 1] == 1) and from p itself when it has no child.
__global__ __launch_bounds__(64) void decode_sample_draw(const float *__restrict__ logits, const float *__restrict__ draft,
                                                         const float *__restrict__ masses, const float *__restrict__ uniforms,
                                                         const float *__restrict__ ranges, const uint32_t *__restrict__ decisions,
                                                         uint32_t *__restrict__ tokens, TargetSamplingParams p) {
  const uint32_t row = blockIdx.x, lane = threadIdx.x;
  const uint32_t laneIndex = lane_of_row(p, row);
  if (!((p.sampling_mask >> laneIndex) & 1u)) return;  // a greedy lane keeps its argmax
  const uint32_t decision = decisions[SAMPLING_DECISION_WORDS * row];
  if (decision != SAMPLING_NO_TOKEN) {
    if (lane == 0) tokens[row] = decision;
    return;
  }
  const bool rejected = decisions[SAMPLING_DECISION_WORDS * row + 1] == 1u;
  const float inverse = 1.0f / p.temperature[laneIndex];
  const Kept kept = row_kept(masses, decisions, row, inverse, (p.truncating_mask >> laneIndex) & 1u);
  const float *x = logits + size_t(row) * p.logits_stride, *q = draft + size_t(row) * p.logits_stride;
  const float *r = ranges + row * SAMPLING_RANGES;
  float total = 0.f;
  for (uint32_t j = 0; j < SAMPLING_RANGES; ++j) total += r[j];
  if (!(total > 0.f)) {
    if (lane == 0) tokens[row] = SAMPLING_NO_TOKEN;
    return;
  }
  const float point = uniforms[2 * row] * total;
  // The range that holds the point; the last weighted range on a rounding shortfall.
  uint32_t hit = SAMPLING_RANGES, lastWeighted = 0;
  float before = 0.f, lastBefore = 0.f;
  {
    float cumulative = 0.f;
    for (uint32_t j = 0; j < SAMPLING_RANGES && hit == SAMPLING_RANGES; ++j) {
      if (r[j] > 0.f) { lastWeighted = j; lastBefore = cumulative; }
      if (point < cumulative + r[j]) { hit = j; before = cumulative; }
      cumulative += r[j];
    }
  }
  if (hit == SAMPLING_RANGES) { hit = lastWeighted; before = lastBefore; }
  float target = point - before;
  // Its lanes' chunks, as the ranges kernel summed them, walked in lane order.
  const uint32_t size = range_tokens(p.vocabulary), begin = hit * size, end = min(p.vocabulary, begin + size);
  const uint32_t per = (size + 63u) / 64u;
  float sum = 0.f;
  for (uint32_t i = 0; i < per; ++i) {
    const uint32_t token = begin + lane * per + i;
    if (token < end) sum += residual_of(x[token], token, rejected ? q[token] : 0.f, kept, inverse, rejected);
  }
  uint32_t chunk = 64, lastChunk = 0;
  float chunkBefore = 0.f, lastChunkBefore = 0.f, cumulative = 0.f;
  for (int l = 0; l < 64; ++l) {
    const float c = __shfl(sum, l, 64);
    if (c > 0.f) { lastChunk = uint32_t(l); lastChunkBefore = cumulative; }
    if (chunk == 64 && target < cumulative + c) { chunk = uint32_t(l); chunkBefore = cumulative; }
    cumulative += c;
  }
  if (chunk == 64) { chunk = lastChunk; chunkBefore = lastChunkBefore; }
  target -= chunkBefore;
  if (lane == 0) {
    uint32_t selected = SAMPLING_NO_TOKEN, lastToken = SAMPLING_NO_TOKEN;
    float walked = 0.f;
    for (uint32_t i = 0; i < per; ++i) {
      const uint32_t token = begin + chunk * per + i;
      if (token >= end) break;
      const float w = residual_of(x[token], token, rejected ? q[token] : 0.f, kept, inverse, rejected);
      if (w > 0.f) lastToken = token;
      walked += w;
      if (selected == SAMPLING_NO_TOKEN && w > 0.f && target < walked) selected = token;
    }
    tokens[row] = selected != SAMPLING_NO_TOKEN ? selected : lastToken;
  }
}
SP_REGISTER_KERNEL("decode_sample_draw", &decode_sample_draw);

// decode_sample_draw_children (the rule of the reference's vocabulary_draw with children, sampling.metal:697-880): grid
// (rows), 64 threads. A sampled row of a tree block tests the children its draft drew among its SAMPLING_CANDIDATES
// candidates -- ids [row][16], their draft probabilities q [row][16], the candidate indices drawn in order draws
// [row][4] (bytes, SAMPLING_NO_DRAW past them), a uniform a child child_uniforms [row][4] -- by recursive rejection
// sampling without replacement: child c is selected iff u_c q_c < p_c; a rejection leaves the target its residual
// max(p - q, 0) over the candidates and its mass outside them, renormalized, and the draft its rest, renormalized. A
// row that selects none draws at u_row of the last residual: a candidate in index order, or past them a token
// outside them in id order by the target's own weights. The ranges hold the row's kept weights (the ranges kernel
// ran without a child); the candidates' weights leave them here. Lanes 0..15 weigh a candidate each, lane 0 decides,
// the wavefront walks the drawn range.
__global__ __launch_bounds__(64) void decode_sample_draw_children(const float *__restrict__ logits, const float *__restrict__ masses,
                                                                  const float *__restrict__ uniforms, const float *__restrict__ ranges,
                                                                  const uint32_t *__restrict__ decisions,
                                                                  const uint32_t *__restrict__ candidate_ids,
                                                                  const float *__restrict__ candidate_q,
                                                                  const uint8_t *__restrict__ draws,
                                                                  const float *__restrict__ child_uniforms,
                                                                  uint32_t *__restrict__ tokens, TargetSamplingParams p) {
  constexpr uint32_t K = SAMPLING_CANDIDATES;
  __shared__ float rangeWeight[SAMPLING_RANGES];
  __shared__ float candidateWeight[K];
  __shared__ uint32_t excludedIds[K];
  __shared__ uint32_t decided[4];  // selected (1) or walking (0), token or range, target bits, excluding
  const uint32_t row = blockIdx.x, lane = threadIdx.x;
  const uint32_t laneIndex = lane_of_row(p, row);
  if (!((p.sampling_mask >> laneIndex) & 1u)) return;  // a greedy lane keeps its argmax
  const float inverse = 1.0f / p.temperature[laneIndex];
  const Kept kept = row_kept(masses, decisions, row, inverse, (p.truncating_mask >> laneIndex) & 1u);
  const float *x = logits + size_t(row) * p.logits_stride;
  const uint32_t size = range_tokens(p.vocabulary);
  for (uint32_t j = lane; j < SAMPLING_RANGES; j += 64u) rangeWeight[j] = ranges[row * SAMPLING_RANGES + j];
  if (lane < K) {
    const uint32_t id = candidate_ids[row * K + lane];
    excludedIds[lane] = id;
    candidateWeight[lane] = id < p.vocabulary ? kept_weight(x[id], id, kept, inverse) : 0.f;
  }
  __syncthreads();
  if (lane == 0) {
    float total = 0.f;
    for (uint32_t j = 0; j < SAMPLING_RANGES; ++j) total += rangeWeight[j];
    bool selected = false, excluding = false;
    uint32_t token = SAMPLING_NO_TOKEN;
    float target = uniforms[2 * row] * total;
    const uint8_t *drawn = draws + row * SAMPLING_TREE_CHILDREN;
    if (!(total > 0.f)) {
      selected = true;  // nothing selectable: the sentinel
    } else if (drawn[0] != SAMPLING_NO_DRAW) {
      float pc[K], qc[K];
      for (uint32_t i = 0; i < K; ++i) {
        const uint32_t id = excludedIds[i];
        const float weight = candidateWeight[i];
        if (id < p.vocabulary) rangeWeight[id / size] = fmaxf(rangeWeight[id / size] - weight, 0.f);
        pc[i] = weight / total;
        qc[i] = candidate_q[row * K + i];
      }
      float outsideWeight = 0.f;
      for (uint32_t j = 0; j < SAMPLING_RANGES; ++j) outsideWeight += rangeWeight[j];
      float outside = outsideWeight / total;
      for (uint32_t child = 0; child < SAMPLING_TREE_CHILDREN && !selected; ++child) {
        const uint32_t c = drawn[child];
        if (c >= K) break;
        // a dynamic index into a register array would spill: pick the child's p and q by comparison
        float pChild = 0.f, qChild = 0.f;
        for (uint32_t i = 0; i < K; ++i) { pChild = i == c ? pc[i] : pChild; qChild = i == c ? qc[i] : qChild; }
        if (child_uniforms[row * SAMPLING_TREE_CHILDREN + child] * qChild < pChild) {
          selected = true;
          token = excludedIds[c];
          break;
        }
        float residual = outside;
        for (uint32_t i = 0; i < K; ++i) residual += fmaxf(pc[i] - qc[i], 0.f);
        if (!(residual > 0.f)) break;
        for (uint32_t i = 0; i < K; ++i) pc[i] = fmaxf(pc[i] - qc[i], 0.f) / residual;
        outside /= residual;
        float rest = 0.f;
        for (uint32_t i = 0; i < K; ++i) { qc[i] = i == c ? 0.f : qc[i]; rest += qc[i]; }
        for (uint32_t i = 0; rest > 0.f && i < K; ++i) qc[i] /= rest;
      }
      if (!selected) {
        float inside = 0.f;
        for (uint32_t i = 0; i < K; ++i) inside += pc[i];
        const float point = uniforms[2 * row] * (inside + outside);
        float cumulative = 0.f;
        uint32_t last = K;
        for (uint32_t i = 0; i < K && !(point < cumulative); ++i)
          if (pc[i] > 0.f) {
            last = i;
            cumulative += pc[i];
          }
        if (last < K && (point < cumulative || !(outside > 0.f))) {
          selected = true;
          token = excludedIds[last];
        } else {
          excluding = true;
          target = (point - inside) / outside * outsideWeight;
        }
      }
    }
    uint32_t hit = 0;
    float within = 0.f;
    if (!selected) {
      // the first weighted range whose end lies past the target; the last weighted one on a rounding shortfall
      float cumulative = 0.f;
      for (uint32_t j = 0; j < SAMPLING_RANGES; ++j) {
        const float weight = rangeWeight[j];
        if (!(weight > 0.f)) continue;
        hit = j;
        within = target - cumulative;
        cumulative += weight;
        if (cumulative > target) break;
      }
    }
    decided[0] = selected ? 1u : 0u;
    decided[1] = selected ? token : hit;
    decided[2] = __builtin_bit_cast(uint32_t, within);
    decided[3] = excluding ? 1u : 0u;
  }
  __syncthreads();
  if (decided[0]) {
    if (lane == 0) tokens[row] = decided[1];
    return;
  }
  const uint32_t hit = decided[1];
  const bool excluding = decided[3] != 0u;
  float target = __builtin_bit_cast(float, decided[2]);
  auto weigh = [&](uint32_t token) {
    bool out = false;
    if (excluding)
      for (uint32_t i = 0; i < K; ++i) out = out || excludedIds[i] == token;
    return out ? 0.f : kept_weight(x[token], token, kept, inverse);
  };
  // the range's lanes' chunks, as the ranges kernel summed them (less the candidates), walked in lane order
  const uint32_t begin = hit * size, end = min(p.vocabulary, begin + size), per = (size + 63u) / 64u;
  float sum = 0.f;
  for (uint32_t i = 0; i < per; ++i) {
    const uint32_t token = begin + lane * per + i;
    if (token < end) sum += weigh(token);
  }
  uint32_t chunk = 64, lastChunk = 0;
  float chunkBefore = 0.f, lastChunkBefore = 0.f, cumulative = 0.f;
  for (int l = 0; l < 64; ++l) {
    const float c = __shfl(sum, l, 64);
    if (c > 0.f) { lastChunk = uint32_t(l); lastChunkBefore = cumulative; }
    if (chunk == 64 && c > 0.f && target < cumulative + c) { chunk = uint32_t(l); chunkBefore = cumulative; }
    cumulative += c;
  }
  if (chunk == 64) { chunk = lastChunk; chunkBefore = lastChunkBefore; }
  target -= chunkBefore;
  if (lane == 0) {
    uint32_t selected = SAMPLING_NO_TOKEN, lastToken = SAMPLING_NO_TOKEN;
    float walked = 0.f;
    for (uint32_t i = 0; i < per; ++i) {
      const uint32_t token = begin + chunk * per + i;
      if (token >= end) break;
      const float w = weigh(token);
      if (w > 0.f) lastToken = token;
      walked += w;
      if (selected == SAMPLING_NO_TOKEN && w > 0.f && target < walked) selected = token;
    }
    tokens[row] = selected != SAMPLING_NO_TOKEN ? selected : lastToken;
  }
}
SP_REGISTER_KERNEL("decode_sample_draw_children", &decode_sample_draw_children);

} // namespace splash::kernels

// ---- Greedy selection of packed logits rows without any allocation ------------------------------
// spo_sampling_greedy_rows_static (include/splash_ops.h) is the argmax pair above for callers that
// cannot allocate: the shards' partials live in a file-scope device array instead of a workspace.
// Host code never uses the array's name as an address: each device's copy is looked up once with
// hipGetSymbolAddress and that pointer is what the kernels get.
#include "backend/Internal.hpp"
#include "splash_ops.h"

#include <hip/hip_runtime.h>
#include <mutex>

namespace splash::kernels {
namespace {

struct GreedyPartial {
  float value;
  uint32_t index;
};
constexpr uint32_t kStaticRows = SPO_SAMPLING_STATIC_MAXIMUM_ROWS;
constexpr int kMaximumDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticRows * SAMPLING_SHARDS * sizeof(GreedyPartial)];

std::mutex scratchMutex;
void *scratchOfDevice[kMaximumDevices];  // each device holds its own copy of the array, at its own address

// The current device's copy of the scratch array (looked up on the device's first call).
hipError_t deviceScratch(void **out) {
  int device = -1;
  hipError_t status = hipGetDevice(&device);
  if (status != hipSuccess) return status;
  if (device < 0 || device >= kMaximumDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(scratchMutex);
  if (!scratchOfDevice[device]) {
    void *address = nullptr;
    status = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
    if (status != hipSuccess) return status;
    scratchOfDevice[device] = address;
  }
  *out = scratchOfDevice[device];
  return hipSuccess;
}

} // namespace
} // namespace splash::kernels

extern "C" sp_status spo_sampling_greedy_rows_static(const float *logits, uint32_t rows, uint32_t vocabulary, uint32_t logits_stride,
                                                     uint32_t *tokens, void *stream) {
  using namespace splash::kernels;
  auto fail = [](sp_status code, const std::string &message) {
    splash::hipbackend::setLastError(message);
    return code;
  };
  if (!logits || !tokens) return fail(SP_INVALID_ARGUMENT, "null logits or tokens");
  if (!rows || rows > kStaticRows)
    return fail(SP_INVALID_ARGUMENT, "the static greedy selection takes 1 to " + std::to_string(kStaticRows) + " rows");
  if (!vocabulary || logits_stride < vocabulary) return fail(SP_INVALID_ARGUMENT, "a logits row holds its vocabulary");
  void *memory = nullptr;
  hipError_t status = deviceScratch(&memory);
  if (status != hipSuccess) return fail(SP_BACKEND_ERROR, std::string("hipGetSymbolAddress: ") + hipGetErrorString(status));
  // Every (row, shard) partial of this call is written by the first kernel before the second reads
  // it, so nothing of an earlier call's contents is read and nothing needs clearing.
  float *values = static_cast<float *>(memory);
  uint32_t *indices = reinterpret_cast<uint32_t *>(values + size_t(kStaticRows) * SAMPLING_SHARDS);
  TargetSamplingParams p{};
  p.vocabulary = vocabulary;
  p.rows = rows;
  p.lanes = 1;
  p.logits_stride = logits_stride;
  p.lane[0] = SamplingLaneRows{0, rows};
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(decode_sample_argmax_sharded, dim3(rows * SAMPLING_SHARDS), dim3(256), 0, s, logits, values, indices, p);
  hipLaunchKernelGGL(decode_sample_argmax_reduce, dim3(rows), dim3(64), 0, s, values, indices, tokens, p);
  status = hipGetLastError();
  if (status != hipSuccess) return fail(SP_BACKEND_ERROR, std::string("launch: ") + hipGetErrorString(status));
  return SP_OK;
}
