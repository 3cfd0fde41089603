// The draft model's attention block (abi/DraftAttention.h; the reference's kernels/decode/draft.metal,
// kernels/prefill/draft_context.metal, common/draft_context_kv.h and common/draft_context_window.h): the dynamic
// convolutions, the q/k/v preparation of a lane's eight query rows, their attention over the lane's rings and
// themselves, the writers of the rings and the 4-bit context window.
//
// The attention core: a KV head's 32 attention rows (four query heads x eight query rows) against the ring's live
// slots and the eight current rows. A workgroup of the split pass takes one 128-slot tile of the ring, a wave 32 of
// its slots: the scores leave the matrix cores transposed (tokens down, query rows across), which is the operand
// layout of the output product, so nothing passes through LDS between the two; keys and values are read from the
// rings as the operands they are (a key's 8 consecutive dimensions, a value dimension's 4 + 4 consecutive slots). One
// more workgroup takes the current rows. The merge adds the 17 partials in their order, so a row's result depends on
// neither the lanes of the dispatch nor the order the workgroups finished in.
#include "abi/DraftAttention.h"
#include "abi/Sampling.h"
#include "backend/KernelRegistry.hpp"
#include "kernels/device_common.hpp"

namespace splash::kernels {
namespace {

constexpr uint32_t kRows = DRAFT_ATTENTION_QUERY_ROWS, kQueryHeads = DRAFT_ATTENTION_QUERY_HEADS, kKvHeads = DRAFT_ATTENTION_KV_HEADS;
constexpr uint32_t kD = DRAFT_ATTENTION_HEAD_DIMENSION, kWindow = DRAFT_ATTENTION_WINDOW, kM = DRAFT_ATTENTION_ROWS;
constexpr uint32_t kPairs = DRAFT_ATTENTION_ROPE_PAIRS;
// 1 / sqrt(128) and log2(e): scores are kept as exponents of two.
constexpr float kScoreScale = 0.08838834765f * 1.4426950408889634f;

// One head of 128 values at `source`: RMS-normalized, weighed by `weight`, rounded to bf16, then turned by the RoPE
// row (dimension i with i + 64). A wave's lane l holds dimensions l and l + 64; the squares are added lane by lane
// (l's two, then the butterfly 32, 16, ... 1 apart).
__device__ __forceinline__ void head_norm_rope(const uint16_t *__restrict__ source, const uint16_t *__restrict__ weight,
                                               const float *__restrict__ cosines, const float *__restrict__ sines,
                                               uint16_t *__restrict__ destination, uint32_t lane) {
  const float x0 = bf16_bits_to_float(source[lane]), x1 = bf16_bits_to_float(source[lane + 64u]);
  const float total = wave_sum(x0 * x0 + x1 * x1);
  const float inverse = 1.0f / sqrtf(total / float(kD) + 1e-6f);
  const float n0 = round_bf16(x0 * inverse * bf16_bits_to_float(weight[lane]));
  const float n1 = round_bf16(x1 * inverse * bf16_bits_to_float(weight[lane + 64u]));
  const float c = cosines[lane], s = sines[lane];
  destination[lane] = uint16_t(float_to_bf16_bits(n0 * c - n1 * s));
  destination[lane + 64u] = uint16_t(float_to_bf16_bits(n1 * c + n0 * s));
}

// The i-th set bit of `mask` (i below its count).
__device__ __forceinline__ uint32_t nth_set_bit(uint32_t mask, uint32_t i) {
  for (uint32_t earlier = 0; earlier < i; ++earlier) mask &= mask - 1u;
  return uint32_t(__builtin_ctz(mask));
}

} // namespace

__global__ __launch_bounds__(256) void draft_conv(const uint16_t *__restrict__ input, const uint16_t *__restrict__ dynamic,
                                                  const uint16_t *__restrict__ base, const uint16_t *__restrict__ residual,
                                                  uint16_t *__restrict__ output, DraftConvParams p) {
  const uint32_t hidden = p.hidden, groups = hidden / DRAFT_CONVOLUTION_GROUP, dynamicWidth = draft_dynamic_width(hidden);
  const uint32_t element = blockIdx.x * 256u + threadIdx.x;
  if (element >= kRows * hidden) return;
  const size_t lane = blockIdx.y;
  input += lane * kRows * hidden;
  residual += lane * kRows * hidden;
  output += lane * kRows * hidden;
  dynamic += lane * kRows * dynamicWidth;
  const uint32_t row = element / hidden, channel = element % hidden, group = channel / DRAFT_CONVOLUTION_GROUP;
  const uint32_t tap = (p.finish ? 1u : 0u) * DRAFT_CONVOLUTION_TAPS;
  float value = bf16_bits_to_float(input[element]) *
                (bf16_bits_to_float(base[tap * hidden + channel]) + bf16_bits_to_float(dynamic[row * dynamicWidth + tap * groups + group]));
  if (row > 0)
    value += bf16_bits_to_float(input[element - hidden]) *
             (bf16_bits_to_float(base[(tap + 1u) * hidden + channel]) +
              bf16_bits_to_float(dynamic[row * dynamicWidth + (tap + 1u) * groups + group]));
  if (p.finish) value += bf16_bits_to_float(residual[element]);
  output[element] = uint16_t(float_to_bf16_bits(value));
}

__global__ __launch_bounds__(256) void draft_mask_rows(const uint16_t *__restrict__ mask, uint16_t *__restrict__ rows, DraftMaskRowsParams p) {
  const uint32_t column = blockIdx.x * 256u + threadIdx.x;
  if (column < p.width) rows[(size_t(blockIdx.z) * kRows + 1u + blockIdx.y) * p.width + column] = mask[column];
}

__global__ __launch_bounds__(512) void draft_attention_qkv(const uint16_t *__restrict__ qkv, uint16_t *__restrict__ queries,
                                                           const uint16_t *__restrict__ query_norm, const uint16_t *__restrict__ key_norm,
                                                           const float *__restrict__ rope_cos, const float *__restrict__ rope_sin,
                                                           uint16_t *__restrict__ query_keys, uint16_t *__restrict__ query_values, DraftLanesParams) {
  const size_t batch = blockIdx.y;
  qkv += batch * kRows * DRAFT_ATTENTION_QKV_WIDTH;
  queries += batch * kRows * DRAFT_ATTENTION_WIDTH;
  query_keys += batch * kRows * DRAFT_ATTENTION_KV_WIDTH;
  query_values += batch * kRows * DRAFT_ATTENTION_KV_WIDTH;
  // The value rows, transposed to [KV head][dimension][row].
  const uint32_t element = blockIdx.x * 512u + threadIdx.x;
  if (element < kRows * DRAFT_ATTENTION_KV_WIDTH) {
    const uint32_t row = element / DRAFT_ATTENTION_KV_WIDTH, rest = element % DRAFT_ATTENTION_KV_WIDTH;
    query_values[rest * kRows + row] = qkv[row * DRAFT_ATTENTION_QKV_WIDTH + DRAFT_ATTENTION_WIDTH + DRAFT_ATTENTION_KV_WIDTH + rest];
  }
  // Task (row, head): the query heads' first, then the key heads'.
  const uint32_t task = blockIdx.x * 8u + (threadIdx.x >> 6), lane = threadIdx.x & 63u;
  constexpr uint32_t kQueryTasks = kRows * kQueryHeads;
  if (task >= kQueryTasks + kRows * kKvHeads) return;
  const bool query = task < kQueryTasks;
  const uint32_t local = query ? task : task - kQueryTasks, heads = query ? kQueryHeads : kKvHeads;
  const uint32_t row = local / heads, head = local % heads;
  const uint16_t *source = qkv + row * DRAFT_ATTENTION_QKV_WIDTH + (query ? 0u : DRAFT_ATTENTION_WIDTH) + head * kD;
  const size_t rope = (batch * DRAFT_ATTENTION_ROPE_LANE_ROWS + row) * kPairs;
  head_norm_rope(source, query ? query_norm : key_norm, rope_cos + rope, rope_sin + rope,
                 (query ? queries : query_keys) + (head * kRows + row) * kD, lane);
}

__global__ __launch_bounds__(64) void draft_context_kv(const uint16_t *__restrict__ context_kv, const uint16_t *__restrict__ key_norm,
                                                       const float *__restrict__ rope_cos, const float *__restrict__ rope_sin,
                                                       uint8_t *__restrict__ rings, const uint32_t *__restrict__ retained,
                                                       const SamplingLaneRows *__restrict__ lane_rows, DraftContextParams p) {
  const uint32_t batch = blockIdx.y, index = blockIdx.x / kKvHeads, head = blockIdx.x % kKvHeads, lane = threadIdx.x;
  uint32_t sourceRow = index, ropeRow = index;
  if (p.commit) {
    const uint32_t path = retained[batch], count = min(uint32_t(__builtin_popcount(path)), lane_rows[batch].rows);
    if (index >= count) return;
    const uint32_t bit = nth_set_bit(path, index);
    if (bit >= lane_rows[batch].rows) return;  // a mask names rows of its lane alone: a stray bit reads nothing
    sourceRow = lane_rows[batch].first + bit;
    ropeRow = batch * DRAFT_ATTENTION_ROPE_LANE_ROWS + index;
  } else if (index >= p.rows) {
    return;
  }
  const uint32_t slot = (p.start_position[batch] + index) % kWindow;
  const uint16_t *source = context_kv + size_t(sourceRow) * 2u * DRAFT_ATTENTION_KV_WIDTH + head * kD;
  uint16_t *keys = reinterpret_cast<uint16_t *>(rings + p.keys[batch]) + (size_t(head) * kWindow + slot) * kD;
  uint16_t *values = reinterpret_cast<uint16_t *>(rings + p.values[batch]) + size_t(head) * kD * kWindow + slot;
  head_norm_rope(source, key_norm, rope_cos + size_t(ropeRow) * kPairs, rope_sin + size_t(ropeRow) * kPairs, keys, lane);
  values[size_t(lane) * kWindow] = source[DRAFT_ATTENTION_KV_WIDTH + lane];
  values[size_t(lane + 64u) * kWindow] = source[DRAFT_ATTENTION_KV_WIDTH + lane + 64u];
}

__global__ __launch_bounds__(256) void draft_attention_split(const uint16_t *__restrict__ queries, const uint8_t *__restrict__ rings,
                                                             const uint16_t *__restrict__ query_keys,
                                                             const uint16_t *__restrict__ query_values, float *__restrict__ partials,
                                                             DraftAttentionParams p) {
  const uint32_t head = blockIdx.x, batch = blockIdx.y, split = blockIdx.z;
  float *const partial = partials + ((size_t(batch) * kKvHeads + head) * DRAFT_ATTENTION_SPLITS + split) * DRAFT_ATTENTION_PARTIAL_FLOATS;
  const uint16_t *const q = queries + size_t(batch) * kRows * DRAFT_ATTENTION_WIDTH + size_t(head) * kM * kD;
  const uint32_t cache = p.cache_length[batch];
  // The positions every row's window may hold: [commonStart, cache); row r of the eight hides the first hiddenPrefix
  // of them, the positions that have left its own window of 2048.
  const uint32_t commonStart = cache >= kWindow - 1u ? cache - (kWindow - 1u) : 0u, oldCount = cache - commonStart;
  const uint32_t physicalStart = commonStart % kWindow;

  if (split == DRAFT_ATTENTION_RING_TILES) {
    // The eight current rows, every one visible to every row: thread (row, c) holds dimensions 16 c .. 16 c + 15.
    const uint32_t row = threadIdx.x / 8u, c = threadIdx.x % 8u;
    const uint16_t *keys = query_keys + (size_t(batch) * kKvHeads + head) * kRows * kD;
    const uint16_t *values = query_values + (size_t(batch) * kKvHeads + head) * kD * kRows;
    float query[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) query[i] = bf16_bits_to_float(q[row * kD + 16u * c + i]);
    float score[kRows], best = -INFINITY;
#pragma unroll
    for (uint32_t j = 0; j < kRows; ++j) {
      float dot = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) dot += query[i] * bf16_bits_to_float(keys[j * kD + 16u * c + i]);
      dot += __shfl_xor(dot, 1, 64);
      dot += __shfl_xor(dot, 2, 64);
      dot += __shfl_xor(dot, 4, 64);
      score[j] = dot * kScoreScale;
      best = fmaxf(best, score[j]);
    }
    float sum = 0.f, acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
    for (uint32_t j = 0; j < kRows; ++j) {
      const float weight = __builtin_amdgcn_exp2f(score[j] - best);
      sum += weight;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] += weight * bf16_bits_to_float(values[(16u * c + i) * kRows + j]);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) partial[row * kD + 16u * c + i] = acc[i];
    if (c == 0) {
      partial[kM * kD + row] = best;
      partial[kM * kD + kM + row] = sum;
    }
    return;
  }

  // A ring tile: slots [slot0, slot0 + 128), whose logical indices (positions past commonStart) run on from `first`
  // modulo the ring. Live if one of them is below oldCount.
  const uint32_t slot0 = split * DRAFT_ATTENTION_TILE, first = (slot0 - physicalStart) & (kWindow - 1u);
  if (!(oldCount > 0u && (first < oldCount || first + DRAFT_ATTENTION_TILE > kWindow))) {
    if (threadIdx.x < kM) partial[kM * kD + threadIdx.x] = -INFINITY;
    return;
  }
  __shared__ float waveMax[4][kM], waveSum[4][kM];
  __shared__ float combined[kM][kD];
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, col = lane & 15u, kq = lane >> 4;
  const uint32_t base = slot0 + 32u * wave;
  const uint16_t *const keys = reinterpret_cast<const uint16_t *>(rings + p.keys[batch]) + size_t(head) * kWindow * kD;
  const uint16_t *const values = reinterpret_cast<const uint16_t *>(rings + p.values[batch]) + size_t(head) * kD * kWindow;

  // Scores, transposed: s[g][t][i] of token base + 16 t + 4 kq + i and attention row 16 g + col.
  f32x4 s[2][2];
  {
    bf16x8 query[2][4];
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int j = 0; j < 4; ++j) query[g][j] = as_bf16x8(*reinterpret_cast<const uint4 *>(q + (16u * g + col) * kD + 32u * j + 8u * kq));
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      bf16x8 key[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        key[j] = as_bf16x8(load_stream(reinterpret_cast<const uint4 *>(keys + size_t(base + 16u * t + col) * kD + 32u * j + 8u * kq)));
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(key[j], query[g][j], acc, 0, 0, 0);
        s[g][t] = acc;
      }
    }
  }
  float best[2], sum[2];
  bf16x8 weights[2];
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    const uint32_t proposal = (16u * g + col) % kRows, position = cache + proposal;
    const uint32_t rowStart = position >= kWindow - 1u ? position - (kWindow - 1u) : 0u, hiddenPrefix = rowStart - commonStart;
    float most = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t logical = (base + 16u * t + 4u * kq + i - physicalStart) & (kWindow - 1u);
        const bool visible = logical < oldCount && logical >= hiddenPrefix;
        s[g][t][i] = visible ? s[g][t][i] * kScoreScale : -INFINITY;
        most = fmaxf(most, s[g][t][i]);
      }
    most = fmaxf(most, __shfl_xor(most, 16, 64));
    most = fmaxf(most, __shfl_xor(most, 32, 64));
    const float safe = most == -INFINITY ? 0.f : most;
    float total = 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float weight = __builtin_amdgcn_exp2f(s[g][t][i] - safe);
        total += weight;
        weights[g][4 * t + i] = __bf16(weight);
      }
    total += __shfl_xor(total, 16, 64);
    total += __shfl_xor(total, 32, 64);
    best[g] = most;
    sum[g] = total;
    if (kq == 0) {
      waveMax[wave][16u * g + col] = most;
      waveSum[wave][16u * g + col] = total;
    }
  }
  // Outputs, transposed: o[g][d][i] of dimension 16 d + 4 kq + i and attention row 16 g + col. A value operand's
  // eight slots are the tokens of the weights': 4 kq .. + 3 of the wave's first sixteen, then of its second.
  f32x4 o[2][8];
#pragma unroll
  for (int d = 0; d < 8; ++d) {
    const uint16_t *at = values + size_t(16u * d + col) * kWindow + base + 4u * kq;
    const uint2 low = *reinterpret_cast<const uint2 *>(at), high = *reinterpret_cast<const uint2 *>(at + 16);
    const bf16x8 value = as_bf16x8(make_uint4(low.x, low.y, high.x, high.y));
#pragma unroll
    for (int g = 0; g < 2; ++g) o[g][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(value, weights[g], f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
  }
  __syncthreads();
  // The tile's maximum of each row, every wave's outputs and sums brought to it, and added in wave order.
  float factor[2];
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    const uint32_t row = 16u * g + col;
    const float most = fmaxf(fmaxf(waveMax[0][row], waveMax[1][row]), fmaxf(waveMax[2][row], waveMax[3][row]));
    factor[g] = __builtin_amdgcn_exp2f(best[g] - (most == -INFINITY ? 0.f : most));
  }
  for (uint32_t turn = 0; turn < 4u; ++turn) {
    if (wave == turn) {
#pragma unroll
      for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int d = 0; d < 8; ++d)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float &cell = combined[16u * g + col][16u * d + 4u * kq + i];
            cell = turn ? cell + o[g][d][i] * factor[g] : o[g][d][i] * factor[g];
          }
    }
    __syncthreads();
  }
#pragma unroll
  for (int e = 0; e < 16; ++e) partial[threadIdx.x + 256u * e] = (&combined[0][0])[threadIdx.x + 256u * e];
  if (threadIdx.x < kM) {
    const uint32_t row = threadIdx.x;
    const float most = fmaxf(fmaxf(waveMax[0][row], waveMax[1][row]), fmaxf(waveMax[2][row], waveMax[3][row]));
    const float safe = most == -INFINITY ? 0.f : most;
    float total = 0.f;
    for (uint32_t w = 0; w < 4u; ++w) total += waveSum[w][row] * __builtin_amdgcn_exp2f(waveMax[w][row] - safe);
    partial[kM * kD + row] = most;
    partial[kM * kD + kM + row] = total;
  }
}

// The 17 partials of a (lane, KV head) in their order into the lane's rows, [query row][query head][dimension]: the
// output projection's input, in the place of the grouped queries every split has read. A thread holds four dimensions
// of a row: its 17 splits' loads are in flight together, one round trip to memory.
__global__ __launch_bounds__(1024) void draft_attention_merge(const float *__restrict__ partials, uint16_t *__restrict__ output, DraftLanesParams) {
  const uint32_t head = blockIdx.x, batch = blockIdx.y, row = threadIdx.x / 32u, c = threadIdx.x % 32u;
  const float *from = partials + (size_t(batch) * kKvHeads + head) * DRAFT_ATTENTION_SPLITS * DRAFT_ATTENTION_PARTIAL_FLOATS;
  // Every split's maximum, sum and outputs are loaded whatever the split holds, so the loads do not wait for each other;
  // a split with no visible key (a maximum of -inf) wrote no outputs, and what its place holds is set aside, not added.
  float splitMax[DRAFT_ATTENTION_SPLITS], splitSum[DRAFT_ATTENTION_SPLITS], most = -INFINITY;
  float4 four[DRAFT_ATTENTION_SPLITS];
#pragma unroll
  for (uint32_t split = 0; split < DRAFT_ATTENTION_SPLITS; ++split) {
    splitMax[split] = from[split * DRAFT_ATTENTION_PARTIAL_FLOATS + kM * kD + row];
    splitSum[split] = from[split * DRAFT_ATTENTION_PARTIAL_FLOATS + kM * kD + kM + row];
    four[split] = *reinterpret_cast<const float4 *>(from + split * DRAFT_ATTENTION_PARTIAL_FLOATS + row * kD + 4u * c);
    most = fmaxf(most, splitMax[split]);
  }
  float total = 0.f, acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (uint32_t split = 0; split < DRAFT_ATTENTION_SPLITS; ++split) {
    const bool live = splitMax[split] != -INFINITY;
    const float scale = __builtin_amdgcn_exp2f(splitMax[split] - most);
    if (live) total += scale * splitSum[split];
    const float values[4] = {four[split].x, four[split].y, four[split].z, four[split].w};
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] += live ? scale * values[i] : 0.f;
  }
  const uint32_t queryRow = row % kRows, queryHead = head * (kM / kRows) + row / kRows;
  uint16_t *to = output + size_t(batch) * kRows * DRAFT_ATTENTION_WIDTH + (queryRow * kQueryHeads + queryHead) * kD + 4u * c;
  const uint32_t low = float_to_bf16_bits(acc[0] / total) | (float_to_bf16_bits(acc[1] / total) << 16);
  const uint32_t high = float_to_bf16_bits(acc[2] / total) | (float_to_bf16_bits(acc[3] / total) << 16);
  *reinterpret_cast<uint2 *>(to) = make_uint2(low, high);
}

// A wave a (row, group of 64 values): lane l holds value l; the code of x is round((x - minimum) / scale) with the scale
// and minimum as stored (fp16), so loading reads back minimum + code * scale.
__global__ __launch_bounds__(256) void draft_context_store(const uint16_t *__restrict__ context, uint8_t *__restrict__ window,
                                                           const uint32_t *__restrict__ retained,
                                                           const SamplingLaneRows *__restrict__ lane_rows, DraftWindowParams p) {
  const uint32_t groups = p.width / DRAFT_CONTEXT_GROUP, task = blockIdx.x * 4u + (threadIdx.x >> 6), lane = threadIdx.x & 63u;
  const uint32_t row = task / groups, group = task % groups;
  if (row >= p.rows) return;
  uint32_t sourceRow = row;
  if (p.commit) {
    const uint32_t path = retained[0];
    if (row >= min(uint32_t(__builtin_popcount(path)), lane_rows[0].rows)) return;
    const uint32_t bit = nth_set_bit(path, row);
    if (bit >= lane_rows[0].rows) return;
    sourceRow = lane_rows[0].first + bit;
  }
  const uint32_t slot = (p.start_position + row) % kWindow;
  const float x = bf16_bits_to_float(context[size_t(sourceRow) * p.width + group * DRAFT_CONTEXT_GROUP + lane]);
  float low = x, high = x;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    low = fminf(low, __shfl_xor(low, o, 64));
    high = fmaxf(high, __shfl_xor(high, o, 64));
  }
  const uint32_t scaleBits = float_to_half_bits(__fdiv_rn(high - low, 15.0f)), minimumBits = float_to_half_bits(low);
  const float scale = half_bits_to_float(scaleBits), minimum = half_bits_to_float(minimumBits);
  uint32_t code = 0;
  if (scale > 0.f) code = uint32_t(fminf(fmaxf(rintf(__fdiv_rn(x - minimum, scale)), 0.f), 15.f));
  const uint32_t other = uint32_t(__shfl_xor(int(code), 1, 64));
  if (!(lane & 1u)) window[size_t(slot) * (p.width / 2u) + group * (DRAFT_CONTEXT_GROUP / 2u) + lane / 2u] = uint8_t(code | (other << 4));
  if (lane == 0)
    reinterpret_cast<uint32_t *>(window + draft_context_codes_bytes(p.width))[size_t(slot) * groups + group] = scaleBits | (minimumBits << 16);
}

__global__ __launch_bounds__(256) void draft_context_load(const uint8_t *__restrict__ window, uint16_t *__restrict__ context, DraftWindowParams p) {
  const uint32_t groups = p.width / DRAFT_CONTEXT_GROUP, task = blockIdx.x * 4u + (threadIdx.x >> 6), lane = threadIdx.x & 63u;
  const uint32_t row = task / groups, group = task % groups;
  if (row >= p.rows) return;
  const uint32_t slot = (p.start_position + row) % kWindow;
  const uint32_t pair = reinterpret_cast<const uint32_t *>(window + draft_context_codes_bytes(p.width))[size_t(slot) * groups + group];
  const float scale = half_bits_to_float(pair & 0xFFFFu), minimum = half_bits_to_float(pair >> 16);
  const uint32_t byte = window[size_t(slot) * (p.width / 2u) + group * (DRAFT_CONTEXT_GROUP / 2u) + lane / 2u];
  const uint32_t code = lane & 1u ? byte >> 4 : byte & 15u;
  context[size_t(row) * p.width + group * DRAFT_CONTEXT_GROUP + lane] = uint16_t(float_to_bf16_bits(__fmaf_rn(float(code), scale, minimum)));
}

SP_REGISTER_KERNEL("draft_conv", &draft_conv);
SP_REGISTER_KERNEL("draft_mask_rows", &draft_mask_rows);
SP_REGISTER_KERNEL("draft_attention_qkv", &draft_attention_qkv);
SP_REGISTER_KERNEL("draft_context_kv", &draft_context_kv);
SP_REGISTER_KERNEL("draft_attention_split", &draft_attention_split);
SP_REGISTER_KERNEL("draft_attention_merge", &draft_attention_merge);
SP_REGISTER_KERNEL("draft_context_store", &draft_context_store);
SP_REGISTER_KERNEL("draft_context_load", &draft_context_load);

} // namespace splash::kernels
