// The draft selector's candidates (the reference's kernels/decode/sampling.metal: draft_select_top16_sharded :1099-1232,
// top16_merge_shards :1236-1264, draft_select_edges :1271-1356): of every proposal position's logits row the
// DRAFT_CANDIDATES largest, the larger logit first and among equal ones the smaller column, and of each candidate the
// score of its edge from each candidate of the position before it (from the lane's anchor at position 0).
//
// The order is that of one 64-bit key a column: the logit's order-preserving bits above the complement of its column,
// -0 counted as +0, so "the next candidate" is the largest key below the last one and the whole selection is sixteen
// maximum reductions over keys that never leave the wavefronts' registers. A NaN logit is never a candidate; a row of fewer
// columns than candidates ends in empty ones (token 0xFFFFFFFF, logit -infinity).
#include "abi/Sampling.h"
#include "backend/KernelRegistry.hpp"
#include "kernels/device_common.hpp"

namespace splash::kernels {
namespace {

constexpr uint32_t kCandidates = DRAFT_CANDIDATES, kPositions = DRAFT_PROPOSAL_TOKENS, kQueryRows = DRAFT_QUERY_ROWS;
constexpr uint32_t kRank = DRAFT_SELECTOR_RANK;
// The key of an empty candidate: below every column's of a logit that is no NaN, above a NaN's.
constexpr uint64_t kEmpty = uint64_t{0x007FFFFFu} << 32;

__device__ __forceinline__ uint64_t order_key(float value, uint32_t column) {
  uint32_t bits = __float_as_uint(value + 0.0f);
  bits = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
  const uint64_t key = (uint64_t{bits} << 32) | (0xFFFFFFFFu - column);
  return value != value ? 0 : key;
}
__device__ __forceinline__ uint32_t column_of(uint64_t key) { return 0xFFFFFFFFu - static_cast<uint32_t>(key); }

// The largest key of a wavefront, in every lane. Sixteen of these follow one another in a selection, each waiting for the
// last, so they move data between lanes with DPP row shifts and broadcasts, a few cycles each, and never through the LDS
// crossbar: a lane no shift reaches keeps its own key, which a maximum does not mind. After the shifts by 1, 2, 4 and 8 a
// row's last lane holds the row's largest, after the two broadcasts lane 63 the wavefront's.
template <int Control> __device__ __forceinline__ uint64_t dpp_max(uint64_t key) {
  const int low = static_cast<int>(static_cast<uint32_t>(key)), high = static_cast<int>(static_cast<uint32_t>(key >> 32));
  const uint32_t other_low = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(low, low, Control, 0xF, 0xF, false));
  const uint32_t other_high = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(high, high, Control, 0xF, 0xF, false));
  const uint64_t other = (uint64_t{other_high} << 32) | other_low;
  return other > key ? other : key;
}
__device__ __forceinline__ uint64_t wave_max_key(uint64_t key) {
  constexpr int kRowShiftRight = 0x110, kRowBroadcast15 = 0x142, kRowBroadcast31 = 0x143;
  key = dpp_max<kRowShiftRight + 1>(key);
  key = dpp_max<kRowShiftRight + 2>(key);
  key = dpp_max<kRowShiftRight + 4>(key);
  key = dpp_max<kRowShiftRight + 8>(key);
  key = dpp_max<kRowBroadcast15>(key);
  key = dpp_max<kRowBroadcast31>(key);
  const uint32_t low = __builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(key)), 63);
  const uint32_t high = __builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(key >> 32)), 63);
  return (uint64_t{high} << 32) | low;
}

// A wavefront's sixteen largest of its lanes' keys (each lane N of them, all different or empty), best first: lane r < 16
// returns the r-th, the other lanes an empty key. The next one is the largest below the last, so a round is one scan of the
// lane's registers and one maximum over the wavefront, with no barrier.
template <uint32_t N> __device__ __forceinline__ uint64_t wave_top16(const uint64_t (&keys)[N]) {
  const uint32_t l = threadIdx.x & 63u;
  uint64_t last = ~uint64_t{0}, mine = kEmpty;
#pragma unroll 1
  for (uint32_t rank = 0; rank < kCandidates; ++rank) {
    // The lane's largest key below the last: a balanced tree over the keys that are.
    uint64_t below[N];
#pragma unroll
    for (uint32_t j = 0; j < N; ++j) below[j] = keys[j] < last ? keys[j] : kEmpty;
#pragma unroll
    for (uint32_t width = 1; width < N; width *= 2)
#pragma unroll
      for (uint32_t j = 0; j + width < N; j += 2 * width) below[j] = below[j] > below[j + width] ? below[j] : below[j + width];
    last = wave_max_key(below[0]);
    if (l == rank) mine = last;
  }
  return mine;
}

} // namespace

// Grid (lanes * DRAFT_PROPOSAL_TOKENS * shards), 256 threads. A lane's proposal positions are rows 1-7 of its eight
// query rows of the logits. Each wavefront selects among its quarter of the shard's columns, held in registers, and the
// first one among the four's. partials [row][shard][DRAFT_CANDIDATES] keys, best first.
__global__ __launch_bounds__(256) void draft_select_top16_sharded(const float *__restrict__ logits, uint64_t *__restrict__ partials,
                                                                  DraftSelectParams p) {
  constexpr uint32_t kMine = DRAFT_SHARD_COLUMNS / 256;
  __shared__ uint64_t quarters[4 * kCandidates];
  const uint32_t tid = threadIdx.x, shard = blockIdx.x % p.shards, row = blockIdx.x / p.shards;
  const uint32_t lane = row / kPositions, position = row % kPositions;
  const float *x = logits + (size_t(lane) * kQueryRows + position + 1) * p.columns;
  const uint32_t begin = shard * DRAFT_SHARD_COLUMNS;
  // Every load is made (a column past the row's end reads the row's last one and counts as empty), so that a lane's
  // are in flight together.
  float values[kMine];
#pragma unroll
  for (uint32_t j = 0; j < kMine; ++j) values[j] = __builtin_nontemporal_load(x + min(begin + j * 256 + tid, p.columns - 1));
  uint64_t keys[kMine];
#pragma unroll
  for (uint32_t j = 0; j < kMine; ++j) {
    const uint32_t column = begin + j * 256 + tid;
    const uint64_t key = order_key(values[j], column);
    keys[j] = column < p.columns && key ? key : kEmpty;
  }
  const uint64_t mine = wave_top16(keys);
  if ((tid & 63u) < kCandidates) quarters[(tid >> 6) * kCandidates + (tid & 63u)] = mine;
  __syncthreads();
  if (tid < 64) {
    const uint64_t one[1] = {quarters[tid]};
    const uint64_t best = wave_top16(one);
    if (tid < kCandidates) partials[size_t(blockIdx.x) * kCandidates + tid] = best;
  }
}
SP_REGISTER_KERNEL("draft_select_top16_sharded", &draft_select_top16_sharded);

namespace {
// The best DRAFT_CANDIDATES keys of a row's shard partials, by one wavefront: lane r < 16 returns the r-th.
template <uint32_t N> __device__ __forceinline__ uint64_t merge_shards(const uint64_t *__restrict__ partials, uint32_t row, uint32_t shards) {
  const uint32_t entries = shards * kCandidates, l = threadIdx.x & 63u;
  const uint64_t *mine = partials + size_t(row) * entries;
  uint64_t keys[N];
#pragma unroll
  for (uint32_t j = 0; j < N; ++j) keys[j] = l + j * 64 < entries ? mine[l + j * 64] : kEmpty;
  return wave_top16(keys);
}
__device__ __forceinline__ uint32_t token_of(uint64_t key, const DraftSelectParams &p) {
  if (key == kEmpty) return SAMPLING_NO_TOKEN;
  const uint32_t column = column_of(key);
  return column < p.leading ? column : column - p.leading + p.trailing;
}
__device__ __forceinline__ float4 bf16x4_to_float(uint2 v) {
  return make_float4(bf16_bits_to_float(v.x & 0xFFFFu), bf16_bits_to_float(v.x >> 16), bf16_bits_to_float(v.y & 0xFFFFu),
                     bf16_bits_to_float(v.y >> 16));
}
} // namespace

// Grid (lanes * DRAFT_PROPOSAL_TOKENS), 256 threads: one workgroup per proposal row merges its row's candidates (tokens
// and their logits, best first) and those of the row before it, then scores the edges: edges[row][predecessor][candidate]
// = sum over the selector's rank of predecessor_codebook[predecessor token] * hidden[row] * successor_codebook[candidate
// token], bf16 factors multiplied and summed in fp32. Position 0 has the lane's anchor as its one predecessor (row 0 of
// its table; the other rows are left as they were). hidden: bf16 [lanes * 8][rank], a lane's positions rows 1-7.
__global__ __launch_bounds__(256) void draft_select_edges(const float *__restrict__ logits, const uint64_t *__restrict__ partials,
                                                          uint32_t *__restrict__ candidates, float *__restrict__ unary,
                                                          float *__restrict__ edges, const uint16_t *__restrict__ hidden,
                                                          const uint16_t *__restrict__ predecessor_codebook,
                                                          const uint16_t *__restrict__ successor_codebook, DraftSelectParams p) {
  __shared__ uint32_t successors[kCandidates], predecessors[kCandidates];
  const uint32_t tid = threadIdx.x, wave = tid >> 6, l = tid & 63u;
  const uint32_t row = blockIdx.x, lane = row / kPositions, position = row % kPositions;
  // The first wavefront merges the row's candidates, the second those of the row before it.
  if (wave < 2 && (wave == 0 || position > 0)) {
    constexpr uint32_t kFew = 10, kMany = DRAFT_MAXIMUM_SHARDS * DRAFT_CANDIDATES / 64;
    const uint64_t key = p.shards * kCandidates <= kFew * 64 ? merge_shards<kFew>(partials, row - wave, p.shards)
                                                             : merge_shards<kMany>(partials, row - wave, p.shards);
    if (l < kCandidates) {
      const uint32_t token = token_of(key, p);
      if (wave == 0) {
        const float *x = logits + (size_t(lane) * kQueryRows + position + 1) * p.columns;
        candidates[row * kCandidates + l] = token;
        unary[row * kCandidates + l] = key == kEmpty ? -INFINITY : x[column_of(key)];
        successors[l] = min(token, p.vocabulary - 1u);
      } else {
        predecessors[l] = min(token, p.vocabulary - 1u);
      }
    }
  } else if (wave == 1 && l < kCandidates) {
    predecessors[l] = min(p.anchor[lane], p.vocabulary - 1u);
  }
  __syncthreads();
  // The rows meet in LDS as fp32, the predecessors' already times the hidden row: a wavefront every fourth row of each
  // table, a lane four consecutive dimensions, every load requested before the first is used. Then a thread an edge: its
  // 256 products in four running sums of every fourth dimension, added at the end, so no sum crosses lanes. A row's stride
  // of 257 words keeps the sixteen rows a wavefront reads at one dimension in sixteen banks.
  static_assert(kRank == 4 * kWave && kCandidates * kCandidates == 256, "a lane four dimensions, a thread an edge");
  constexpr uint32_t kStride = kRank + 1;
  __shared__ float contexts[kCandidates * kStride], followers[kCandidates * kStride];
  const uint32_t count = position > 0 ? kCandidates : 1u;
  const float4 h = bf16x4_to_float(reinterpret_cast<const uint2 *>(hidden + (size_t(lane) * kQueryRows + position + 1) * kRank)[l]);
  uint2 after[kCandidates / 4], before[kCandidates / 4];
#pragma unroll
  for (uint32_t j = 0; j < kCandidates / 4; ++j) {
    before[j] = reinterpret_cast<const uint2 *>(predecessor_codebook + size_t(predecessors[min(wave + j * 4, count - 1)]) * kRank)[l];
    after[j] = reinterpret_cast<const uint2 *>(successor_codebook + size_t(successors[wave + j * 4]) * kRank)[l];
  }
#pragma unroll
  for (uint32_t j = 0; j < kCandidates / 4; ++j) {
    const float4 c = bf16x4_to_float(before[j]), s = bf16x4_to_float(after[j]);
    float *context = contexts + (wave + j * 4) * kStride + 4 * l, *follower = followers + (wave + j * 4) * kStride + 4 * l;
    context[0] = c.x * h.x, context[1] = c.y * h.y, context[2] = c.z * h.z, context[3] = c.w * h.w;
    follower[0] = s.x, follower[1] = s.y, follower[2] = s.z, follower[3] = s.w;
  }
  __syncthreads();
  const uint32_t predecessor = tid / kCandidates, candidate = tid % kCandidates;
  if (predecessor >= count) return;
  const float *context = contexts + predecessor * kStride, *follower = followers + candidate * kStride;
  float sums[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll 8
  for (uint32_t d = 0; d < kRank; d += 4) {
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) sums[i] += context[d + i] * follower[d + i];
  }
  edges[size_t(row) * kCandidates * kCandidates + tid] = (sums[0] + sums[1]) + (sums[2] + sums[3]);
}
SP_REGISTER_KERNEL("draft_select_edges", &draft_select_edges);

} // namespace splash::kernels
