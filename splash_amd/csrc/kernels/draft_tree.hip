// The draft selector's tree growth (the reference's draft_select_tree, kernels/decode/sampling.metal:1357-1766; its rule,
// runtime/metal/abi/Sampling.h:209-241): over the candidates and edge scores draft_select_edges left, each lane grows a
// tree of up to 16 rows best first by the estimate that the target accepts the path to a row.
//
// One wavefront a lane, and no heap: the tree's open steps ("entries": from a row to a token one deeper) sit in LDS, at
// most five a row, and taking the best is one 64-bit maximum reduction over (estimate bits, complement of the entry's
// number), which is exactly "the largest estimate, the earlier entry among equal ones". A row's expansion runs on sixteen
// lanes, one a candidate: the tempered weights, the Gumbel keys of a sampled lane's draws (a hash of the row's key and the
// candidate's token a lane), each draw a 16-lane maximum reduction. Sums whose order decides a float's bits (a
// distribution's mass) are taken in candidate order, as a sequential statement takes them, so the values agree with it to
// the rounding of exp and log alone.
#include "abi/PagedAttention.h"
#include "abi/Sampling.h"
#include "backend/KernelRegistry.hpp"
#include "kernels/device_common.hpp"

namespace splash::kernels {
namespace {

constexpr uint32_t kPositions = DRAFT_PROPOSAL_TOKENS, kCandidates = DRAFT_CANDIDATES, kChildren = SAMPLING_TREE_CHILDREN;
constexpr uint32_t kRows = DRAFT_TREE_ROWS, kEntries = 96, kDead = 0xFFFFFFFFu, kChainEntry = 1u << 31;

__device__ __forceinline__ uint64_t mix64(uint64_t v) {  // the splitmix64 finalizer
  v = (v ^ (v >> 30)) * 0xbf58476d1ce4e5b9ull;
  v = (v ^ (v >> 27)) * 0x94d049bb133111ebull;
  return v ^ (v >> 31);
}
// The standard Gumbel of candidate `token` under a row of key `key`: of a uniform from the top 23 bits k of a hash of the
// two, (k + 0.5) / 2^23, which fp32 holds exactly, inside (0, 1).
__device__ __forceinline__ float gumbel_of(uint64_t key, uint32_t token) {
  const uint64_t v = mix64(key ^ 0xd1b54a32d192ed03ull * (uint64_t(token) + 1u));
  const float uniform = (float(uint32_t(v >> 41)) + 0.5f) * 0x1p-23f;
  return -logf(-logf(uniform));
}
__device__ __forceinline__ uint32_t order_bits(float value) {
  const uint32_t bits = __float_as_uint(value);
  return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
}
// The largest key of each group of `Width` neighbouring lanes, in every lane of the group.
template <int Width> __device__ __forceinline__ uint64_t group_max(uint64_t key) {
#pragma unroll
  for (int step = 1; step < Width; step <<= 1) {
    const uint32_t lo = uint32_t(__shfl_xor(int(uint32_t(key)), step, 64)), hi = uint32_t(__shfl_xor(int(uint32_t(key >> 32)), step, 64));
    const uint64_t other = uint64_t(hi) << 32 | lo;
    key = other > key ? other : key;
  }
  return key;
}

struct TreeState {
  float probability[kPositions][kCandidates][kCandidates];
  uint8_t likeliest[kPositions][kCandidates][kChildren];
  uint32_t ids[kPositions][kCandidates];
  // rows
  uint32_t token[kRows], ancestors[kRows], parent[kRows], depth[kRows], onChain[kRows];
  float q[kRows], estimate[kRows], cap[kRows];
  uint64_t key[kRows];
  uint8_t draw[kRows][kChildren];
  float left[kRows][kChildren], next[kRows][kCandidates];
  // entries: the steps the tree may still take, in the order made
  float entryScore[kEntries];
  uint32_t entryInfo[kEntries];  // kChainEntry | parent row << 16 | proposal position << 8 | candidate index; kDead once taken
};

} // namespace

__global__ __launch_bounds__(64) void draft_select_tree(const uint32_t *__restrict__ candidates, const float *__restrict__ unary,
                                                        const float *__restrict__ edges, const uint32_t *__restrict__ chain_tokens,
                                                        const float *__restrict__ chain_rates, uint32_t *__restrict__ tokens,
                                                        AttentionTreeRow *__restrict__ tree, float *__restrict__ scores,
                                                        uint32_t *__restrict__ sizes, uint8_t *__restrict__ draws,
                                                        float *__restrict__ next, float *__restrict__ caps, DraftTreeParams p) {
  __shared__ TreeState s;
  const uint32_t lane = blockIdx.x, tid = threadIdx.x, i = tid & 15u;
  const size_t origin = size_t(lane) * kPositions * kCandidates;

  // ---- The lattice: a thread a (position, predecessor candidate); position 0 follows the anchor alone.
  for (uint32_t at = tid; at < kPositions * kCandidates; at += 64u) {
    const uint32_t position = at / kCandidates, predecessor = at % kCandidates;
    s.ids[position][predecessor] = candidates[origin + at];
    if (position == 0 && predecessor != 0) continue;
    const float *edge = edges + (origin + at) * kCandidates;
    float score[kCandidates];
#pragma unroll
    for (uint32_t c = 0; c < kCandidates; ++c) score[c] = unary[origin + position * kCandidates + c] + edge[c];
    float best = score[0];
#pragma unroll
    for (uint32_t c = 1; c < kCandidates; ++c) best = fmaxf(best, score[c]);
    float weight[kCandidates], mass = 0.f;
#pragma unroll
    for (uint32_t c = 0; c < kCandidates; ++c) {
      weight[c] = expf(score[c] - best);
      mass += weight[c];
    }
#pragma unroll
    for (uint32_t c = 0; c < kCandidates; ++c) s.probability[position][predecessor][c] = weight[c] / mass;
    // its four likeliest, the lower index first among equal scores: four passes over a key of (score, complement of index)
    uint64_t last = ~uint64_t{0};
    for (uint32_t child = 0; child < kChildren; ++child) {
      uint64_t pick = 0;
#pragma unroll
      for (uint32_t c = 0; c < kCandidates; ++c) {
        const uint64_t key = uint64_t(order_bits(score[c] + 0.0f)) << 32 | (kCandidates - c);
        pick = key < last && key > pick ? key : pick;
      }
      last = pick;
      s.likeliest[position][predecessor][child] = uint8_t(kCandidates - uint32_t(pick));
    }
  }
  __syncthreads();

  const uint32_t *chain = chain_tokens + size_t(lane) * DRAFT_CHAIN_TOKENS;
  const float *rates = chain_rates + size_t(lane) * DRAFT_CHAIN_TOKENS * DRAFT_CHAIN_AGREEMENTS;
  const uint32_t children = min(p.children[lane], kChildren), deepest = p.depth[lane], chained = min(p.chain[lane], uint32_t(DRAFT_CHAIN_TOKENS));
  const float temperature = p.temperature[lane], slope = p.slope[lane];
  uint32_t made = 1, entryCount = 0;

  // A host chain token's rate at depth d, by its agreement with the draft there: its likeliest candidate, another of its
  // candidates, none of them, or past its positions.
  auto chainRate = [&](uint32_t d) {
    const uint32_t token = chain[d];
    uint32_t agreement = 3;
    if (d < kPositions) {
      const bool mine = tid < kCandidates && s.ids[d][tid] == token;
      const uint64_t among = __builtin_amdgcn_ballot_w64(mine);
      agreement = among & 1u ? 0u : among ? 1u : 2u;
    }
    return rates[d * DRAFT_CHAIN_AGREEMENTS + agreement];
  };
  auto estimateOf = [&](float q, uint32_t position) {
    q = fminf(fmaxf(q, 1.0e-6f), 1.0f - 1.0e-6f);
    const float z = slope * logf(q / (1.0f - q)) + p.intercept[lane][position];
    return 1.0f / (1.0f + expf(-z));
  };
  auto push = [&](float score, uint32_t info) {
    if (entryCount < kEntries) {
      if (tid == 0) {
        s.entryScore[entryCount] = score;
        s.entryInfo[entryCount] = info;
      }
      ++entryCount;
    }
  };
  auto capOf = [&](uint32_t parent, uint32_t index) {
    float cap = 1.0f;
    bool found = false;
    for (uint32_t child = 0; child < kChildren; ++child)
      if (!found && s.draw[parent][child] == index) {
        cap = s.left[parent][child];
        found = true;
      }
    return cap;
  };
  auto clearRow = [&](uint32_t row) {
    if (tid < kChildren) s.draw[row][tid] = uint8_t(SAMPLING_NO_DRAW);
    if (tid < kCandidates) s.next[row][tid] = 0.f;
  };
  // A draft row's children at `position`, after its candidate `predecessor`: its drawn candidates, each an entry.
  auto expand = [&](uint32_t row, uint32_t position, uint32_t predecessor, float score, bool hasChain, uint32_t chainToken, float chainRateHere) {
    const float q = s.probability[position][predecessor][i];
    float top = q;
#pragma unroll
    for (int step = 1; step < 16; step <<= 1) top = fmaxf(top, __shfl_xor(top, step, 64));
    const float weight = temperature == 0.0f || !(q > 0.0f) ? q : expf((logf(q) - logf(top)) / temperature);
    if (tid < kCandidates) s.next[row][i] = weight;
    __syncthreads();
    float mass = 0.f;
#pragma unroll
    for (uint32_t c = 0; c < kCandidates; ++c) mass += s.next[row][c];
    __syncthreads();
    const float mine = weight / mass;
    if (tid < kCandidates) s.next[row][i] = mine;
    __syncthreads();
    const float key = temperature > 0.0f && mine > 0.0f ? logf(mine) + gumbel_of(s.key[row], s.ids[position][i]) : -INFINITY;
    uint32_t taken = 0;
    float bound = score, left = 1.0f - chainRateHere, reserved = chainRateHere;
    for (uint32_t child = 0; child < children; ++child) {
      uint32_t drawn = kCandidates;
      if (temperature == 0.0f) {
        const uint32_t likely = s.likeliest[position][predecessor][child];
        drawn = s.probability[position][predecessor][likely] > 0.0f ? likely : kCandidates;
      } else {
        const bool open = !(taken >> i & 1u) && key > -INFINITY;
        const uint64_t best = group_max<16>(open ? uint64_t(order_bits(key)) << 32 | (kCandidates - i) : 0);
        drawn = best ? kCandidates - uint32_t(best) : kCandidates;
        drawn = uint32_t(__builtin_amdgcn_readfirstlane(int(drawn)));
      }
      if (drawn == kCandidates) break;
      taken |= 1u << drawn;
      const bool joins = hasChain && s.ids[position][drawn] == chainToken;
      const float cap = joins ? left + reserved : left;
      const float own = fminf(estimateOf(s.next[row][drawn], position), cap);
      left = joins ? cap - fmaxf(own, reserved) : left - own;
      reserved = joins ? 0.0f : reserved;
      bound = fminf(bound, score * own);
      if (tid == 0) {
        s.draw[row][child] = uint8_t(drawn);
        s.left[row][child] = cap;
      }
      push(bound, row << 16 | position << 8 | drawn);
    }
    __syncthreads();
  };

  if (tid == 0) {
    s.token[0] = p.anchor[lane];
    s.ancestors[0] = 1u;
    s.parent[0] = SAMPLING_TREE_ROOT;
    s.depth[0] = 0;
    s.onChain[0] = 1u;
    s.q[0] = s.estimate[0] = s.cap[0] = 1.0f;
    s.key[0] = uint64_t(p.noise[lane][1]) << 32 | p.noise[lane][0];
  }
  clearRow(0);
  __syncthreads();
  if (deepest > 0) {
    const float rate = chained ? chainRate(0) : 0.0f;
    expand(0, 0, 0, 1.0f, chained != 0, chained ? chain[0] : 0u, rate);
    if (chained) push(rate, kChainEntry);
  }
  __syncthreads();
  const uint32_t most = min(kRows, deepest + 1u);
  while (made < most) {
    // the best open entry: the largest estimate, the earliest made among equal ones
    uint64_t best = 0;
    for (uint32_t e = tid; e < entryCount; e += 64u)
      if (s.entryInfo[e] != kDead) {
        const uint64_t key = uint64_t(order_bits(s.entryScore[e] + 0.0f)) << 32 | (kDead - e);
        best = key > best ? key : best;
      }
    best = group_max<64>(best);
    if (!best) break;
    const uint32_t entry = kDead - uint32_t(best);
    const float score = s.entryScore[entry];
    const uint32_t info = s.entryInfo[entry];
    __syncthreads();
    if (tid == 0) s.entryInfo[entry] = kDead;
    const bool fromChain = (info & kChainEntry) != 0;
    const uint32_t parent = info >> 16 & 0x7FFFu, position = info >> 8 & 0xFFu, index = info & 0xFFu;
    const uint32_t token = fromChain ? chain[position] : s.ids[position][index];
    // a token path the tree holds already gains no row
    const uint64_t same = __builtin_amdgcn_ballot_w64(tid >= 1u && tid < made && s.parent[tid] == parent && s.token[tid] == token);
    uint32_t row = same ? uint32_t(__builtin_ctzll(same)) : 0u;
    if (!row) {
      row = made++;
      const float cap = fromChain ? 1.0f : capOf(parent, index);
      if (tid == 0) {
        s.token[row] = token;
        s.ancestors[row] = s.ancestors[parent] | 1u << row;
        s.parent[row] = parent;
        s.depth[row] = position + 1u;
        s.onChain[row] = s.onChain[parent] && position < chained && token == chain[position];
        s.q[row] = fromChain ? -1.0f : s.next[parent][index];   // a row a host chain token made is no draft step
        s.estimate[row] = score;
        s.cap[row] = cap;
        s.key[row] = mix64(s.key[parent] + 0x9e3779b97f4a7c15ull * (uint64_t(token) + 1u));
      }
      clearRow(row);
    } else if (!fromChain && s.q[row] < 0.0f) {
      // a draft step that joins a host chain's row gives it its draft probability and cap
      const float cap = capOf(parent, index);
      __syncthreads();
      if (tid == 0) {
        s.q[row] = s.next[parent][index];
        s.cap[row] = cap;
      }
    }
    __syncthreads();
    if (position + 1u >= deepest) continue;   // the row's children would lie too deep
    const bool chainChild = s.onChain[row] && position + 1u < chained;
    if (!fromChain && position + 1u < kPositions)
      expand(row, position + 1u, index, score, chainChild, chainChild ? chain[position + 1u] : 0u, chainChild ? chainRate(position + 1u) : 0.0f);
    else if (fromChain && position + 1u < chained)
      push(score * chainRate(position + 1u), kChainEntry | row << 16 | (position + 1u) << 8);
    __syncthreads();
  }
  __syncthreads();
  if (tid == 0) sizes[lane] = made;
  if (tid < made) {
    const size_t at = size_t(lane) * kRows + tid;
    tokens[at] = s.token[tid];
    tree[at] = AttentionTreeRow{s.ancestors[tid], uint16_t(s.parent[tid]), uint16_t(s.depth[tid])};
    scores[2 * at] = s.q[tid];
    scores[2 * at + 1] = s.estimate[tid];
    caps[at] = s.cap[tid];
    for (uint32_t child = 0; child < kChildren; ++child) draws[at * kChildren + child] = s.draw[tid][child];
    for (uint32_t c = 0; c < kCandidates; ++c) next[at * kCandidates + c] = s.next[tid][c];
  }
}
SP_REGISTER_KERNEL("draft_select_tree", &draft_select_tree);

// The trees' side of a sampled verify step, gathered by the step's rows (abi/Sampling.h, VerifyChildrenParams).
__global__ __launch_bounds__(64) void draft_verify_children(const uint32_t *__restrict__ sources, const SamplingLaneRows *__restrict__ lane_rows,
                                                            const AttentionTreeRow *__restrict__ step_tree, const uint32_t *__restrict__ candidates,
                                                            const float *__restrict__ tree_next, const uint8_t *__restrict__ tree_draws,
                                                            uint32_t *__restrict__ ids, float *__restrict__ probabilities,
                                                            uint8_t *__restrict__ draws, uint32_t *__restrict__ depths, VerifyChildrenParams p) {
  const uint32_t row = blockIdx.x, tid = threadIdx.x;
  if (row >= p.rows) return;
  uint32_t lane = SAMPLING_MAXIMUM_LANES;
  for (uint32_t l = 0; l < min(p.lanes, uint32_t(SAMPLING_MAXIMUM_LANES)); ++l)
    if (row >= lane_rows[l].first && row < lane_rows[l].first + lane_rows[l].rows) lane = l;
  const uint32_t source = sources[row], depth = step_tree[row].depth;
  const bool drafted = lane < SAMPLING_MAXIMUM_LANES && source < kRows && depth < kPositions;
  if (tid == 0) depths[row] = lane < SAMPLING_MAXIMUM_LANES ? depth : 0u;
  if (tid < kCandidates) {
    ids[size_t(row) * kCandidates + tid] = drafted ? candidates[(size_t(lane) * kPositions + depth) * kCandidates + tid] : SAMPLING_NO_TOKEN;
    probabilities[size_t(row) * kCandidates + tid] = drafted ? tree_next[(size_t(lane) * kRows + source) * kCandidates + tid] : 0.f;
  }
  if (tid < kChildren) draws[size_t(row) * kChildren + tid] = drafted ? tree_draws[(size_t(lane) * kRows + source) * kChildren + tid] : uint8_t(SAMPLING_NO_DRAW);
}
SP_REGISTER_KERNEL("draft_verify_children", &draft_verify_children);

} // namespace splash::kernels
