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
#include "abi/Sampling.h"
#include "abi/PagedAttention.h"
#include "backend/KernelRegistry.hpp"
#include "kernels/device_common.hpp"

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

// Grid (lanes), 1 thread (sampling.metal:2044-2083). tokens: in, each row's selection; out, the
// lane's retained tokens from its first row.
__global__ void decode_accept_tree(const uint32_t *__restrict__ input_tokens, const AttentionTreeRow *__restrict__ tree,
                                   uint32_t *__restrict__ tokens, uint32_t *__restrict__ retained,
                                   uint32_t *__restrict__ accepted_count, uint32_t *__restrict__ retained_rows,
                                   AcceptBatchParams p) {
  const uint32_t lane = blockIdx.x;
  if (lane >= p.lanes || threadIdx.x) return;
  const uint32_t first = p.lane[lane].first, rows = p.lane[lane].rows;
  const uint32_t *inputs = input_tokens + first;
  const AttentionTreeRow *nodes = tree + first;
  uint32_t *selected = tokens + first;
  uint32_t path[SAMPLING_MAXIMUM_ROWS];
  path[0] = 0;
  uint32_t accepted = 0;
  for (uint32_t row = 0;;) {
    const uint32_t token = selected[row];
    uint32_t next = 0;
    for (uint32_t child = row + 1; child < rows && !next; ++child)
      next = nodes[child].parent == row && inputs[child] == token ? child : 0;
    if (!next) break;
    path[++accepted] = next;
    row = next;
  }
  uint32_t kept = min(accepted + 1, max(p.remaining[lane], 1u));
  for (uint32_t i = 0; i < kept; ++i) {
    const uint32_t token = selected[path[i]];
    selected[i] = token;
    bool stop = false;
#pragma unroll
    for (int s = 0; s < int(SAMPLING_STOP_TOKENS); ++s) stop = stop || (p.stop_tokens[s] != SAMPLING_NO_TOKEN && token == p.stop_tokens[s]);
    if (stop) kept = i + 1;
  }
  accepted_count[lane] = min(accepted, kept);
  retained[lane] = kept;
  retained_rows[lane] = nodes[path[kept - 1]].ancestors;
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
__device__ __forceinline__ float token_weight(float logit, Mass mass, float inverse) {
  return unselectable(logit) ? 0.f : expf((logit - mass.maximum) * inverse);
}
// The residual weight of token t: max(p_t - q_t, 0) after a rejection, p_t's weight otherwise.
__device__ __forceinline__ float residual_of(float logit, float q, Mass mass, float inverse, bool rejected) {
  const float w = token_weight(logit, mass, inverse);
  return rejected ? fmaxf(w / mass.sum - q, 0.f) : w;
}
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
  const float inverse = 1.0f / p.temperature[lane_of_row(p, row)];
  const Mass mass = row_mass(masses, row, inverse);
  const float *x = logits + size_t(row) * p.logits_stride, *q = draft + size_t(row) * p.logits_stride;
  const uint32_t child = child_token(p, tree, input_tokens, row);
  bool rejected = false;
  if (child != SAMPLING_NO_TOKEN && child < p.vocabulary) {
    // accept iff u_child * q < p (sampling.metal:790-800)
    const float pc = token_weight(x[child], mass, inverse) / mass.sum;
    rejected = !(uniforms[2 * row + 1] * q[child] < pc);
    if (blockIdx.x % kPerRow == 0 && threadIdx.x == 0) {
      decisions[2 * row] = rejected ? SAMPLING_NO_TOKEN : child;
      decisions[2 * row + 1] = rejected ? 1u : 0u;
    }
  } else if (blockIdx.x % kPerRow == 0 && threadIdx.x == 0) {
    decisions[2 * row] = SAMPLING_NO_TOKEN;
    decisions[2 * row + 1] = 0u;
  }
  if (child != SAMPLING_NO_TOKEN && child < p.vocabulary && !rejected) return;  // accepted: nothing to draw
  // the range's residual: a lane sums its tokens in id order, the lanes are added in order
  const uint32_t size = range_tokens(p.vocabulary), begin = range * size, end = min(p.vocabulary, begin + size);
  const uint32_t per = (size + 63u) / 64u;
  float sum = 0.f;
  for (uint32_t i = 0; i < per; ++i) {
    const uint32_t token = begin + lane * per + i;
    if (token < end) sum += residual_of(x[token], rejected ? q[token] : 0.f, mass, inverse, rejected);
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
  const uint32_t decision = decisions[2 * row];
  if (decision != SAMPLING_NO_TOKEN) {
    if (lane == 0) tokens[row] = decision;
    return;
  }
  const bool rejected = decisions[2 * row + 1] == 1u;
  const float inverse = 1.0f / p.temperature[laneIndex];
  const Mass mass = row_mass(masses, row, inverse);
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
    if (token < end) sum += residual_of(x[token], rejected ? q[token] : 0.f, mass, inverse, rejected);
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
      const float w = residual_of(x[token], rejected ? q[token] : 0.f, mass, inverse, rejected);
      if (w > 0.f) lastToken = token;
      walked += w;
      if (selected == SAMPLING_NO_TOKEN && w > 0.f && target < walked) selected = token;
    }
    tokens[row] = selected != SAMPLING_NO_TOKEN ? selected : lastToken;
  }
}
SP_REGISTER_KERNEL("decode_sample_draw", &decode_sample_draw);

} // namespace splash::kernels
