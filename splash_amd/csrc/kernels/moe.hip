// Mixture-of-experts routing around the grouped expert projections (kernels/gguf_linear.hip):
// top-k selection, grouping of routes by expert, the tiles' activation tables, the weighted sum
// (the reference's kernels/shared/moe.metal).
#include "abi/Moe.h"
#include "backend/KernelRegistry.hpp"
#include "kernels/device_common.hpp"

namespace splash::kernels {

// moe_route_select (moe.metal:23-113): one wave per row; lane l holds experts l, l + 64, ... Each
// rank takes the highest remaining score and, among equals, the lowest expert id.
// A gated shared expert's weight is the sigmoid of the row's product with the scalar gate: lane l sums dimensions l,
// l + 64, ... in order, the lanes' sums add by the wave's exchanges at distances 32, 16, ... 1.
__global__ __launch_bounds__(64) void moe_route_select(const float *__restrict__ scores, const uint16_t *__restrict__ input,
                                                       const float *__restrict__ shared_gate, uint32_t *__restrict__ selected,
                                                       float *__restrict__ weights, MoeRouteParams p) {
  constexpr uint32_t kPerLane = MOE_MAXIMUM_EXPERTS / 64u;
  __shared__ float ordered[MOE_MAXIMUM_TOP];
  const uint32_t row = blockIdx.x, lane = threadIdx.x, perRow = p.top_k + p.shared;
  if (p.shared) {
    float weight = 1.0f;
    if (p.shared_gated) {
      const uint16_t *x = input + size_t(row) * p.input_size;
      float scalar = 0.f;
      for (uint32_t d = lane; d < p.input_size; d += 64u) scalar += bf16_bits_to_float(x[d]) * shared_gate[d];
      scalar = wave_sum(scalar);
      weight = 1.0f / (1.0f + __builtin_amdgcn_exp2f(-1.44269504089f * scalar));
    }
    if (lane < p.shared) {
      selected[size_t(row) * perRow + p.top_k + lane] = p.experts + lane;
      weights[size_t(row) * perRow + p.top_k + lane] = weight;
    }
  }
  float mine[kPerLane];
#pragma unroll
  for (uint32_t slot = 0; slot < kPerLane; ++slot) {
    const uint32_t expert = lane + 64u * slot;
    mine[slot] = expert < p.experts ? scores[size_t(row) * p.score_stride + expert] : -INFINITY;
  }
  for (uint32_t rank = 0; rank < p.top_k; ++rank) {
    float best = -INFINITY;
    uint32_t bestSlot = 0;
#pragma unroll
    for (uint32_t slot = 0; slot < kPerLane; ++slot)
      if (mine[slot] > best) {
        best = mine[slot];
        bestSlot = slot;
      }
    const float rowBest = wave_max(best);
    uint32_t candidate = best == rowBest ? lane + 64u * bestSlot : 0xFFFFFFFFu;
    uint32_t winner = candidate;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) winner = min(winner, uint32_t(__shfl_xor(int(winner), o, 64)));
    if (candidate == winner) {
#pragma unroll
      for (uint32_t slot = 0; slot < kPerLane; ++slot)
        if (slot == bestSlot) mine[slot] = -INFINITY;
    }
    if (lane == 0) {
      ordered[rank] = rowBest;
      selected[size_t(row) * perRow + rank] = winner;
    }
  }
  __syncthreads();
  if (lane < p.top_k) {
    float denominator = 0.f;
    if (p.sigmoid_router) {
      const auto sigmoid = [](float x) { return 1.0f / (1.0f + __builtin_amdgcn_exp2f(-1.44269504089f * x)); };
      for (uint32_t other = 0; other < p.top_k; ++other) denominator += sigmoid(ordered[other]);
      weights[size_t(row) * perRow + lane] = sigmoid(ordered[lane]) / (denominator + 1e-20f);
    } else {
      for (uint32_t other = 0; other < p.top_k; ++other) denominator += __builtin_amdgcn_exp2f((ordered[other] - ordered[0]) * 1.44269504089f);
      weights[size_t(row) * perRow + lane] = __builtin_amdgcn_exp2f((ordered[lane] - ordered[0]) * 1.44269504089f) / denominator;
    }
  }
}
SP_REGISTER_KERNEL("moe_route_select", &moe_route_select);

// moe_group_routes: one workgroup of 1024 threads, work in proportion to the routes. Every route sets its bit
// in its expert's row of a bit matrix (an OR: whatever order the threads run in, the matrix is the same);
// a thread per expert counts its row word by word, which gives the expert's routes before each word and its
// tiles; a route's place among its expert's is then those before its word plus the set bits below its own, so
// an expert's routes keep their route order and the grouping never depends on timing.
__global__ __launch_bounds__(1024) void moe_group_routes(const uint32_t *__restrict__ selected, uint32_t *__restrict__ route_slot,
                                                         uint32_t *__restrict__ slot_row, uint32_t *__restrict__ tile_expert,
                                                         uint32_t *__restrict__ tile_rows, uint32_t *__restrict__ tile_total,
                                                         MoeGroupParams p) {
  __shared__ uint32_t masks[MOE_GROUP_WORDS];   // [expert][word]: bit b of word w: route 32 w + b is the expert's
  __shared__ uint16_t before[MOE_GROUP_WORDS];  // [expert][word]: the expert's routes before word w
  __shared__ uint32_t firstTile[MOE_MAXIMUM_EXPERTS], waveTiles[MOE_MAXIMUM_EXPERTS / 64u];
  constexpr uint32_t kMine = 256u * MOE_MAXIMUM_TOP / 1024u;  // routes a thread may own
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t words = (p.routes + 31u) / 32u;
  for (uint32_t i = tid; i < p.experts * words; i += 1024u) masks[i] = 0u;
  for (uint32_t slot = tid; slot < p.maximum_tiles * MOE_TILE_ROWS; slot += 1024u) slot_row[slot] = MOE_NO_ROW;
  uint32_t mine[kMine];
#pragma unroll
  for (uint32_t i = 0; i < kMine; ++i) {
    const uint32_t route = tid + 1024u * i;
    mine[i] = route < p.routes ? selected[route] : 0u;
  }
  __syncthreads();
#pragma unroll
  for (uint32_t i = 0; i < kMine; ++i) {
    const uint32_t route = tid + 1024u * i;
    if (route < p.routes) atomicOr(&masks[mine[i] * words + route / 32u], 1u << (route % 32u));
  }
  __syncthreads();
  // The expert's routes in all, and before each word of its row.
  uint32_t total = 0;
  if (tid < p.experts)
    for (uint32_t w = 0; w < words; ++w) {
      before[tid * words + w] = uint16_t(total);
      total += uint32_t(__builtin_popcount(masks[tid * words + w]));
    }
  // First tiles: an exclusive sum of the experts' tile counts, by waves and then over the waves' sums.
  const uint32_t tiles = (total + MOE_TILE_ROWS - 1u) / MOE_TILE_ROWS;
  uint32_t running = tiles;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const uint32_t up = uint32_t(__shfl_up(int(running), o, 64));
    if (lane >= uint32_t(o)) running += up;
  }
  if (lane == 63u && tid < MOE_MAXIMUM_EXPERTS) waveTiles[wave] = running;
  __syncthreads();
  if (tid < MOE_MAXIMUM_EXPERTS) {
    uint32_t start = 0;
    for (uint32_t w = 0; w < wave; ++w) start += waveTiles[w];
    firstTile[tid] = start + running - tiles;
    if (tid == MOE_MAXIMUM_EXPERTS - 1u) tile_total[0] = start + running;
    for (uint32_t t = 0; t < tiles; ++t) {
      tile_expert[firstTile[tid] + t] = tid;
      tile_rows[firstTile[tid] + t] = min(MOE_TILE_ROWS, total - t * MOE_TILE_ROWS);
    }
  }
  __syncthreads();
#pragma unroll
  for (uint32_t i = 0; i < kMine; ++i) {
    const uint32_t route = tid + 1024u * i;
    if (route >= p.routes) continue;
    const uint32_t at = mine[i] * words + route / 32u;
    const uint32_t placed = before[at] + uint32_t(__builtin_popcount(masks[at] & ((1u << (route % 32u)) - 1u)));
    const uint32_t slot = (firstTile[mine[i]] + placed / MOE_TILE_ROWS) * MOE_TILE_ROWS + placed % MOE_TILE_ROWS;
    route_slot[route] = slot;
    slot_row[slot] = route / p.top_k;
  }
}
SP_REGISTER_KERNEL("moe_group_routes", &moe_group_routes);

// moe_gather_table: the activation table (abi/Gguf.h) of each tile's gathered rows, as
// gguf_prepare_table writes a block's; empty slots are zero rows.
__global__ __launch_bounds__(64) void moe_gather_table(const uint16_t *__restrict__ input, const uint32_t *__restrict__ slot_row,
                                                       const uint32_t *__restrict__ tile_total, uint8_t *__restrict__ tables,
                                                       MoeGatherParams p) {
  const uint32_t g = blockIdx.x, tile = blockIdx.y, lane = threadIdx.x, r = lane & 15u, kq = lane >> 4;
  if (tile >= tile_total[0]) return;
  const uint32_t row = slot_row[tile * MOE_TILE_ROWS + r];
  uint8_t *table = tables + tile * p.table_bytes;
  float v[8];
  uint32_t bits[8] = {};
#pragma unroll
  for (uint32_t e = 0; e < 8; ++e) v[e] = 0.f;
  if (row != MOE_NO_ROW) {
    const uint16_t *x = input + size_t(row) * p.hidden + 32u * g;
#pragma unroll
    for (uint32_t e = 0; e < 8; ++e) {
      bits[e] = x[gguf_operand_input(kq, e)];
      v[e] = bf16_bits_to_float(bits[e]);
    }
  }
  reinterpret_cast<uint4 *>(table)[size_t(g) * 64u + lane] =
      make_uint4(bits[0] | (bits[1] << 16), bits[2] | (bits[3] << 16), bits[4] | (bits[5] << 16), bits[6] | (bits[7] << 16));
  const float half0 = (v[0] + v[2]) + (v[1] + v[3]), half1 = (v[4] + v[6]) + (v[5] + v[7]);
  float h0[4], h1[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    h0[q] = __shfl(half0, int(r) + 16 * q, 64);
    h1[q] = __shfl(half1, int(r) + 16 * q, 64);
  }
  const float s0 = ((h0[0] + h0[1]) + h0[2]) + h0[3], s1 = ((h1[0] + h1[1]) + h1[2]) + h1[3];
  if (kq == 0) {
    float *sums32 = reinterpret_cast<float *>(table + gguf_table_sums32_offset(p.hidden, 1));
    float *sums16 = reinterpret_cast<float *>(table + gguf_table_sums16_offset(p.hidden, 1));
    sums32[size_t(g) * 16u + r] = s0 + s1;
    sums16[(2u * size_t(g)) * 16u + r] = s0;
    sums16[(2u * size_t(g) + 1u) * 16u + r] = s1;
  }
}
SP_REGISTER_KERNEL("moe_gather_table", &moe_gather_table);

// moe_combine (moe.metal:367-392): out = bf16(residual + sum over the row's routes of w y) in rank order, fp32.
__global__ __launch_bounds__(256) void moe_combine(const uint16_t *__restrict__ expert_output, const uint32_t *__restrict__ route_slot,
                                                   const float *__restrict__ weights, const uint16_t *__restrict__ residual,
                                                   uint16_t *__restrict__ output, const uint16_t *__restrict__ norm_weight,
                                                   uint8_t *__restrict__ table, MoeCombineParams p) {
  const uint32_t row = blockIdx.x, d = blockIdx.y * 256u + threadIdx.x;
  const bool live = d < p.hidden;  // always, where a table is written
  uint32_t bits = 0;
  if (live) {
    float value = bf16_bits_to_float(residual[size_t(row) * p.hidden + d]);
    for (uint32_t rank = 0; rank < p.top_k; ++rank) {
      const size_t route = size_t(row) * p.top_k + rank;
      value += weights[route] * bf16_bits_to_float(expert_output[size_t(route_slot[route]) * p.hidden + d]);
    }
    bits = float_to_bf16_bits(value);
    output[size_t(row) * p.hidden + d] = uint16_t(bits);
  }
  if (!p.table_tiles) return;
  // The row's piece of the table: lane l of a wave holds input 64 j + l of column group j. Runs of four
  // inputs are one 8-byte piece of a table entry; lanes 4 i lead them.
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, r = row % 16u, G = p.hidden / 32u;
  const uint32_t piece = row / 16u / GGUF_PIECE_TILES, tile = row / 16u % GGUF_PIECE_TILES;
  const uint32_t tiles = min(uint32_t(GGUF_PIECE_TILES), p.table_tiles - piece * GGUF_PIECE_TILES);
  table += piece * gguf_table_bytes(p.hidden, GGUF_PIECE_TILES);
  const float hidden = bf16_bits_to_float(bits);
  const uint32_t scaled = float_to_bf16_bits(hidden * bf16_bits_to_float(norm_weight[d]));
  const float v = bf16_bits_to_float(scaled);
  const uint32_t b1 = uint32_t(__shfl_down(int(scaled), 1, 64)), b2 = uint32_t(__shfl_down(int(scaled), 2, 64)),
                 b3 = uint32_t(__shfl_down(int(scaled), 3, 64));
  const float v1 = __shfl_down(v, 1, 64), v2 = __shfl_down(v, 2, 64), v3 = __shfl_down(v, 3, 64);
  // sums of 16 inputs in input order: the four runs of a half are led by lanes 4 apart
  float s = (v + v1) + (v2 + v3);
  const float s1 = __shfl_down(s, 4, 64), s2 = __shfl_down(s, 8, 64), s3 = __shfl_down(s, 12, 64);
  s = ((s + s1) + s2) + s3;
  const float other = __shfl_down(s, 16, 64);
  float square = hidden * hidden;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) square += __shfl_xor(square, o, 64);
  const uint32_t q = d / 4u, g = q / 8u, half = (q / 4u) % 2u, kq = q % 4u;  // the run of input d
  if ((lane & 3u) == 0) {
    // operand elements 4 half + {0,1,2,3} are inputs 4 kq + {0,2,1,3} of the half
    reinterpret_cast<uint2 *>(table)[((size_t(tile) * G + g) * 64u + kq * 16u + r) * 2u + half] =
        make_uint2(scaled | (b2 << 16), b1 | (b3 << 16));
    if (kq == 0) {
      float *sums32 = reinterpret_cast<float *>(table + gguf_table_sums32_offset(p.hidden, tiles));
      float *sums16 = reinterpret_cast<float *>(table + gguf_table_sums16_offset(p.hidden, tiles));
      sums16[(size_t(tile) * 2u * G + 2u * g + half) * 16u + r] = s;
      if (half == 0) sums32[(size_t(tile) * G + g) * 16u + r] = s + other;
    }
  }
  if (lane == 0) {
    float *squares = reinterpret_cast<float *>(table + gguf_table_squares_offset(p.hidden, tiles));
    squares[size_t(blockIdx.y * 4u + wave) * gguf_squares_stride(tiles) + 16u * tile + r] = square;
  }
}
SP_REGISTER_KERNEL("moe_combine", &moe_combine);

} // namespace splash::kernels
