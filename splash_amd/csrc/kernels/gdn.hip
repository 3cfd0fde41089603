// Gated DeltaNet verify step for gfx950 (the reference's kernels/decode/gdn.metal and
// common/gdn_primitives.h): one workgroup per (value head, lane) runs the short convolution + SiLU,
// the q/k norms and gates of the block's rows, folds the lane's pending (previously accepted) rows
// into the head's 128 x 128 fp32 state, writes THAT state (the one before the block's rows, so a
// rejected row never has to be undone), runs the block's rows for their outputs and gates them.
//
// Sixteen waves. In the prologue and the gate a wave takes a row: lane l holds channels l and 64 + l,
// and a sum over the head's 128 channels is four tree sums over 32 lanes added in channel
// order, the reference's simdgroup sums (gdn.metal:215-222). In the recurrence a wave advances
// two state rows at once, one per half-wave, lane j of a half holding key columns 4 j .. 4 j + 3;
// the row's products with k and q are tree sums over the half's 32 lanes, and each token keeps
// the decay, memory, delta, update, output order of gdn.metal:270-298.
//
// The block's rows never advance the state: every row, of a chain block as of a tree block, takes its
// output from the committed state (the reference does so for tree blocks, gdn.metal:417-478; a chain is
// the tree whose every row follows the row before it): with S_j the state after the j-th token of a
// row's path, S_j z = S_j-1 (d_j (z - c k_j)) + c v_j for c = beta_j (k_j . z), so the row's output is
// S_-1 z_-1 + sum_j c_j v_j; a wave per row walks its path upward for z_-1 and the coefficients, and
// the recurrence's waves add the path terms to the state's product with z_-1: one product with the
// state a row instead of the four passes over it that advancing it takes.
#include "abi/Gdn.h"
#include "abi/Gguf.h"
#include "abi/PagedAttention.h"  // AttentionTreeRow
#include "backend/KernelRegistry.hpp"
#include "kernels/device_common.hpp"

namespace splash::kernels {

namespace {

constexpr uint32_t kDim = GDN_HEAD_DIMENSION, kTaps = GDN_CONVOLUTION_TAPS, kRows = GDN_MAXIMUM_ROWS;
constexpr float kLog2e = 1.44269504089f;

// The sum over each half-wave's 32 lanes (lanes 0..31 and 32..63 apart), in every lane of the half: a
// binary tree over neighbours (pairs, quads, eights, sixteens, the two rows of sixteen), four of its
// levels as row-local DPP operands of the add itself.
template <int Control> __device__ __forceinline__ float dpp_of(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), Control, 0xF, 0xF, false));
}
__device__ __forceinline__ float half_sum(float v) {
  v += dpp_of<0xB1>(v);   // quad_perm [1, 0, 3, 2]
  v += dpp_of<0x4E>(v);   // quad_perm [2, 3, 0, 1]
  v += dpp_of<0x141>(v);  // row_half_mirror: the other quad of the eight
  v += dpp_of<0x140>(v);  // row_mirror: the other eight of the row
  v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));  // lane ^ 16
  return v;
}
// The sum of a head's 128 values, lane l holding a = value[l] and b = value[64 + l]: the four
// 32-channel groups' sums added in channel order.
__device__ __forceinline__ float head_sum(float a, float b) {
  const float first = half_sum(a), second = half_sum(b);
  const float s0 = __shfl(first, 0, 64), s1 = __shfl(first, 32, 64), s2 = __shfl(second, 0, 64), s3 = __shfl(second, 32, 64);
  return ((s0 + s1) + s2) + s3;
}
__device__ __forceinline__ uint32_t path_row(uint32_t path, uint32_t depth) {
  for (uint32_t i = 0; i < depth; ++i) path &= path - 1u;
  return uint32_t(__builtin_ctz(path));
}
__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float silu_of(float x) { return x / (1.0f + exp2_fast(-kLog2e * x)); }
__device__ __forceinline__ float sigmoid_of(float x) { return 1.0f / (1.0f + exp2_fast(-kLog2e * x)); }

struct Tape {
  uint16_t *inputs, *kv;
  float *decay;
  uint16_t *beta;
};
__device__ __forceinline__ Tape tape_at(uint8_t *tape, uint64_t offset, const GdnShapeParams &s) {
  const uint32_t kvWidth = (s.key_heads + s.value_heads) * kDim;
  uint8_t *layer = tape + offset;
  return {reinterpret_cast<uint16_t *>(layer), reinterpret_cast<uint16_t *>(layer + gdn_tape_kv_offset(s.conv_dim)),
          reinterpret_cast<float *>(layer + gdn_tape_decay_offset(s.conv_dim, kvWidth)),
          reinterpret_cast<uint16_t *>(layer + gdn_tape_beta_offset(s.conv_dim, kvWidth, s.value_heads))};
}

// The rows a head folds into its state: k, v and gates, in LDS.
struct Pending {
  uint16_t keys[kRows][kDim];
  uint16_t values[kRows][kDim];
  float decay[kRows];
  uint16_t beta[kRows];
};

// Path row `row` of a tape to slot `slot`: one wave, lane l the channels l and 64 + l.
__device__ __forceinline__ void load_pending(const Tape &tape, Pending &pending, uint32_t slot, uint32_t row, uint32_t head,
                                             const GdnShapeParams &s, uint32_t lane) {
  const uint32_t keyWidth = s.key_heads * kDim, kvWidth = keyWidth + s.value_heads * kDim;
  const uint32_t keyHead = head / (s.value_heads / s.key_heads);
  const uint16_t *source = tape.kv + size_t(row) * kvWidth;
#pragma unroll
  for (uint32_t part = 0; part < 2; ++part) {
    const uint32_t d = lane + 64u * part;
    pending.keys[slot][d] = source[keyHead * kDim + d];
    pending.values[slot][d] = source[keyWidth + head * kDim + d];
  }
  if (lane == 0) {
    pending.decay[slot] = tape.decay[row * s.value_heads + head];
    pending.beta[slot] = tape.beta[row * s.value_heads + head];
  }
}

// The three rows of convolution inputs before a command's first row, after `consumed` rows of
// `path` of `rows` (gdn_primitives.h:20-35).
struct History {
  const uint16_t *row[kTaps - 1];
};
__device__ __forceinline__ History history_of(const uint16_t *carried, const uint16_t *rows, uint32_t conv_dim, uint32_t consumed,
                                              uint32_t path) {
  History h;
#pragma unroll
  for (uint32_t r = 0; r < kTaps - 1; ++r) {
    const uint32_t source = consumed + r;
    h.row[r] = source < kTaps - 1 ? carried + size_t(source) * conv_dim : rows + size_t(path_row(path, source - (kTaps - 1))) * conv_dim;
  }
  return h;
}

// One token's delta-rule step on the wave's state rows (R pairs, a row per half-wave): decay,
// memory, delta, update (gdn.metal:270-298).
template <int R>
__device__ __forceinline__ void advance(float (&state)[R][4], const uint16_t *key, const uint16_t *value_row, const uint32_t (&value_dim)[R],
                                        float decay, float beta, uint32_t column) {
  const uint2 kb = *reinterpret_cast<const uint2 *>(key + column);
  const float k[4] = {bf16_bits_to_float(kb.x & 0xFFFFu), bf16_bits_to_float(kb.x >> 16), bf16_bits_to_float(kb.y & 0xFFFFu),
                      bf16_bits_to_float(kb.y >> 16)};
  float memory[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    memory[r] = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      state[r][i] *= decay;
      memory[r] += state[r][i] * k[i];
    }
    memory[r] = half_sum(memory[r]);
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const float delta = (bf16_bits_to_float(value_row[value_dim[r]]) - memory[r]) * beta;
#pragma unroll
    for (int i = 0; i < 4; ++i) state[r][i] += k[i] * delta;
  }
}

constexpr int kInFlight = 4;  // row pairs a wave advances together, to overlap their reductions
constexpr uint32_t kWaves = 16;  // of a workgroup: with four pairs each they hold the head's 128 state rows at once

} // namespace

// gdn_decode: grid (value_heads, lanes), 1024 threads. `tree` holds the step's rows' places in their
// blocks (bit j of a row's ancestors: row j of its block is on its path, itself included).
__global__ __launch_bounds__(64 * kWaves) void gdn_decode(const uint16_t *__restrict__ packed, const uint16_t *__restrict__ conv_weights,
                                                  uint8_t *__restrict__ states, uint8_t *__restrict__ tape,
                                                  const float *__restrict__ a_scale, const uint16_t *__restrict__ dt_bias,
                                                  const void *__restrict__ norm_weight, uint16_t *__restrict__ hidden,
                                                  const AttentionTreeRow *__restrict__ tree, uint8_t *__restrict__ table,
                                                  GdnDecodeParams p) {
  __shared__ __align__(16) uint16_t queries[kRows][kDim], keys[kRows][kDim], values[kRows][kDim], outputs[kRows][kDim];
  __shared__ __align__(16) float transformed[kRows][kDim];
  __shared__ float coefficients[kRows][kRows];
  __shared__ float decays[kRows];
  __shared__ uint16_t betas[kRows];
  __shared__ uint32_t paths[kRows];
  __shared__ __align__(16) Pending pending;

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, head = blockIdx.x;
  const GdnShapeParams s = p.shape;
  const GdnLane L = p.lane[blockIdx.y];
  const uint32_t perKey = s.value_heads / s.key_heads, keyHead = head / perKey, keyWidth = s.key_heads * kDim;
  const uint32_t kvWidth = keyWidth + s.value_heads * kDim, C = s.conv_dim, P = s.packed_width;
  const uint32_t zOffset = C, bOffset = C + s.value_heads * kDim, aOffset = bOffset + s.value_heads;
  const bool sharedWriter = head % perKey == 0;
  const uint32_t rows = L.rows, pendingRows = uint32_t(__builtin_popcount(L.pending_path));
  const uint16_t *rowsIn = packed + size_t(L.first_row) * P;

  const uint8_t *current = states + L.current_cell;
  uint8_t *next = states + L.next_cell;
  const uint16_t *convIn = reinterpret_cast<const uint16_t *>(current + uint64_t(p.layer) * p.conv_layer_bytes);
  uint16_t *convOut = reinterpret_cast<uint16_t *>(next + uint64_t(p.layer) * p.conv_layer_bytes);
  const float *stateIn = reinterpret_cast<const float *>(current + p.convolution_state_bytes + uint64_t(p.layer) * p.recurrent_layer_bytes);
  float *stateOut = reinterpret_cast<float *>(next + p.convolution_state_bytes + uint64_t(p.layer) * p.recurrent_layer_bytes);
  const Tape pendingTape = tape_at(tape, L.pending_tape, s), stepTape = tape_at(tape, L.step_tape, s);
  const History history = history_of(convIn, pendingTape.inputs, C, pendingRows, L.pending_path);

  // ---- prologue ----
  // channels of this head: q and k of its key head, its v; lane l the dimensions l and 64 + l
  const uint32_t qChannel = keyHead * kDim, kChannel = keyWidth + keyHead * kDim, vChannel = 2 * keyWidth + head * kDim;
  // The state's carried rows after the pending path: waves 0..2 hold one each until the block's rows are done.
  uint16_t carryV[2] = {0, 0}, carryQ[2] = {0, 0}, carryK[2] = {0, 0};
  if (wave < kTaps - 1) {
#pragma unroll
    for (uint32_t part = 0; part < 2; ++part) {
      const uint32_t d = lane + 64u * part;
      carryV[part] = history.row[wave][vChannel + d];
      if (sharedWriter) {
        carryQ[part] = history.row[wave][qChannel + d];
        carryK[part] = history.row[wave][kChannel + d];
      }
    }
  }
  for (uint32_t token = wave; token < pendingRows; token += kWaves)
    load_pending(pendingTape, pending, token, path_row(L.pending_path, token), head, s, lane);
  for (uint32_t token = wave; token < rows; token += kWaves) {
    // The row's path within the block (its own row the last), its depth, and the block rows of its
    // last four path tokens; taps before the block's first row read the history (gdn.metal:198-206).
    const uint32_t path = (tree[L.first_row + token].ancestors & ((1u << token) - 1u)) | (1u << token);
    const uint32_t depth = uint32_t(__builtin_popcount(path)) - 1u;
    const uint16_t *taps[kTaps];
    {
      uint32_t up = path;
#pragma unroll
      for (uint32_t tap = kTaps; tap-- > 0;) {
        const uint32_t row = up ? 31u - uint32_t(__builtin_clz(up)) : 0u;
        up &= ~(1u << row);
        taps[tap] = depth + tap < kTaps - 1 ? history.row[depth + tap] : rowsIn + size_t(row) * P;
      }
    }
    auto conv = [&](uint32_t channel) -> float {
      float value = 0.f;
#pragma unroll
      for (uint32_t tap = 0; tap < kTaps; ++tap)
        value += bf16_bits_to_float(taps[tap][channel]) * bf16_bits_to_float(conv_weights[size_t(channel) * kTaps + tap]);
      value = round_bf16(value);
      return round_bf16(silu_of(value));
    };
    float q[2], k[2], v[2];
#pragma unroll
    for (uint32_t part = 0; part < 2; ++part) {
      const uint32_t d = lane + 64u * part;
      q[part] = conv(qChannel + d);
      k[part] = conv(kChannel + d);
      v[part] = conv(vChannel + d);
    }
    const float qScale = 1.0f / sqrtf(head_sum(q[0] * q[0], q[1] * q[1]) / float(kDim) + 1e-6f);
    const float kScale = 1.0f / sqrtf(head_sum(k[0] * k[0], k[1] * k[1]) / float(kDim) + 1e-6f);
    const uint16_t *inputs = rowsIn + size_t(token) * P;
#pragma unroll
    for (uint32_t part = 0; part < 2; ++part) {
      const uint32_t d = lane + 64u * part;
      const uint32_t query = float_to_bf16_bits(round_bf16(q[part] * qScale) * 0.0078125f);
      const uint32_t key = float_to_bf16_bits(round_bf16(k[part] * kScale) * 0.08838834765f);
      const uint32_t value = float_to_bf16_bits(v[part]);
      queries[token][d] = uint16_t(query);
      keys[token][d] = uint16_t(key);
      values[token][d] = uint16_t(value);
      stepTape.inputs[size_t(token) * C + vChannel + d] = inputs[vChannel + d];
      stepTape.kv[size_t(token) * kvWidth + keyWidth + head * kDim + d] = uint16_t(value);
      if (sharedWriter) {
        stepTape.inputs[size_t(token) * C + qChannel + d] = inputs[qChannel + d];
        stepTape.inputs[size_t(token) * C + kChannel + d] = inputs[kChannel + d];
        stepTape.kv[size_t(token) * kvWidth + keyHead * kDim + d] = uint16_t(key);
      }
    }
    if (lane == 0) {
      // gdn_primitives.h:65-73: beta = bf16(sigmoid(b)); decay = exp(a_scale bf16(softplus(bf16(a + dt_bias))))
      const uint32_t beta = float_to_bf16_bits(sigmoid_of(bf16_bits_to_float(inputs[bOffset + head])));
      const float x = round_bf16(bf16_bits_to_float(inputs[aOffset + head]) + bf16_bits_to_float(dt_bias[head]));
      const float softplus = round_bf16(fmaxf(x, 0.0f) + __builtin_amdgcn_logf(1.0f + exp2_fast(-kLog2e * fabsf(x))) * 0.69314718056f);
      const float decay = exp2_fast(kLog2e * (a_scale[head] * softplus));
      stepTape.beta[token * s.value_heads + head] = uint16_t(beta);
      stepTape.decay[token * s.value_heads + head] = decay;
      betas[token] = uint16_t(beta);
      decays[token] = decay;
      paths[token] = path;
    }
  }
  if (wave < kTaps - 1) {
#pragma unroll
    for (uint32_t part = 0; part < 2; ++part) {
      const uint32_t d = lane + 64u * part;
      convOut[size_t(wave) * C + vChannel + d] = carryV[part];
      if (sharedWriter) {
        convOut[size_t(wave) * C + qChannel + d] = carryQ[part];
        convOut[size_t(wave) * C + kChannel + d] = carryK[part];
      }
    }
  }
  __syncthreads();

  {
    // ---- tree rows: transformed queries and path coefficients, a wave per row ----
    const uint32_t j = lane & 31u, column = 4u * j;
    for (uint32_t token = wave; token < rows; token += kWaves) {
      const uint2 qb = *reinterpret_cast<const uint2 *>(&queries[token][column]);
      float z[4] = {bf16_bits_to_float(qb.x & 0xFFFFu), bf16_bits_to_float(qb.x >> 16), bf16_bits_to_float(qb.y & 0xFFFFu),
                    bf16_bits_to_float(qb.y >> 16)};
      float coefficient = 0.f;
      for (uint32_t up = paths[token]; up;) {
        const uint32_t row = 31u - uint32_t(__builtin_clz(up));
        up &= ~(1u << row);
        const uint2 kb = *reinterpret_cast<const uint2 *>(&keys[row][column]);
        const float k[4] = {bf16_bits_to_float(kb.x & 0xFFFFu), bf16_bits_to_float(kb.x >> 16), bf16_bits_to_float(kb.y & 0xFFFFu),
                            bf16_bits_to_float(kb.y >> 16)};
        float product = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) product += k[i] * z[i];
        const float c = bf16_bits_to_float(betas[row]) * half_sum(product);
        const float d = decays[row];
#pragma unroll
        for (int i = 0; i < 4; ++i) z[i] = d * (z[i] - c * k[i]);
        if (j == row) coefficient = c;
      }
      if (lane < 32u) {
        *reinterpret_cast<float4 *>(&transformed[token][column]) = make_float4(z[0], z[1], z[2], z[3]);
        if (j < kRows) coefficients[token][j] = coefficient;
      }
    }
    __syncthreads();
  }

  // ---- recurrence ----
  {
    const uint32_t half = lane >> 5, column = 4u * (lane & 31u);
    for (uint32_t batch = 0; batch < kDim / (2u * kWaves); batch += kInFlight) {
      uint32_t valueDim[kInFlight];
      float state[kInFlight][4], result[kInFlight];
#pragma unroll
      for (int r = 0; r < kInFlight; ++r) {
        valueDim[r] = (batch + r) * 2u * kWaves + wave * 2u + half;
        const float4 loaded = *reinterpret_cast<const float4 *>(stateIn + (size_t(head) * kDim + valueDim[r]) * kDim + column);
        state[r][0] = loaded.x;
        state[r][1] = loaded.y;
        state[r][2] = loaded.z;
        state[r][3] = loaded.w;
      }
      for (uint32_t token = 0; token < pendingRows; ++token)
        advance<kInFlight>(state, pending.keys[token], pending.values[token], valueDim, pending.decay[token],
                           bf16_bits_to_float(pending.beta[token]), column);
#pragma unroll
      for (int r = 0; r < kInFlight; ++r)
        *reinterpret_cast<float4 *>(stateOut + (size_t(head) * kDim + valueDim[r]) * kDim + column) =
            make_float4(state[r][0], state[r][1], state[r][2], state[r][3]);
      for (uint32_t token = 0; token < rows; ++token) {
        // The path's terms, a lane per block row, beside the committed state's product with the
        // transformed query (gdn.metal:363-377).
        const uint32_t j = lane & 31u, pathRowIndex = j & (kRows - 1u);
        const bool onPath = j < kRows && ((paths[token] >> j) & 1u);
        const float coefficient = coefficients[token][pathRowIndex];
        const float4 zq = *reinterpret_cast<const float4 *>(&transformed[token][column]);
#pragma unroll
        for (int r = 0; r < kInFlight; ++r) {
          result[r] = onPath ? coefficient * bf16_bits_to_float(values[pathRowIndex][valueDim[r]]) : 0.0f;
          result[r] += state[r][0] * zq.x;
          result[r] += state[r][1] * zq.y;
          result[r] += state[r][2] * zq.z;
          result[r] += state[r][3] * zq.w;
          result[r] = half_sum(result[r]);
        }
        if ((lane & 31u) == 0) {
#pragma unroll
          for (int r = 0; r < kInFlight; ++r) outputs[token][valueDim[r]] = uint16_t(float_to_bf16_bits(result[r]));
        }
      }
    }
  }
  __syncthreads();

  // ---- gated output norm (gdn.metal:489-526) ----
  const uint32_t outHead = (p.flags & GDN_TILED_HEADS) ? (head % perKey) * s.key_heads + head / perKey : head;
  for (uint32_t token = wave; token < rows; token += kWaves) {
    float value[2];
#pragma unroll
    for (uint32_t part = 0; part < 2; ++part) value[part] = bf16_bits_to_float(outputs[token][lane + 64u * part]);
    const float inverse = 1.0f / sqrtf(head_sum(value[0] * value[0], value[1] * value[1]) / float(kDim) + 1e-6f);
#pragma unroll
    for (uint32_t part = 0; part < 2; ++part) {
      const uint32_t d = lane + 64u * part;
      const float weight = (p.flags & GDN_FLOAT_NORM) ? static_cast<const float *>(norm_weight)[d]
                                                       : bf16_bits_to_float(static_cast<const uint16_t *>(norm_weight)[d]);
      const float normalized = round_bf16((value[part] * inverse) * weight);
      const float z = bf16_bits_to_float(rowsIn[size_t(token) * P + zOffset + head * kDim + d]);
      const float gated = (normalized * ((p.flags & GDN_SIGMOID_GATE) ? 1.0f : z)) / (1.0f + exp2_fast(-kLog2e * z));
      const uint32_t bits = float_to_bf16_bits(gated);
      hidden[(size_t(L.first_row + token) * s.value_heads + outHead) * kDim + d] = uint16_t(bits);
      outputs[token][d] = uint16_t(bits);  // this wave's row: read above, and below for the table
    }
    if (p.table_tiles) {
      // The row's 128 values of this head as 32 runs of four inputs, a lane a run: the pieces, and the sums of 16
      // and 32 inputs in input order, that gguf_prepare_table would write of the hidden rows.
      const uint32_t packedRow = L.first_row + token, r = packedRow % 16u, width = s.value_heads * kDim, G = width / 32u;
      const uint32_t piece = packedRow / 16u / GGUF_PIECE_TILES, tile = packedRow / 16u % GGUF_PIECE_TILES;
      const uint32_t tiles = min(uint32_t(GGUF_PIECE_TILES), p.table_tiles - piece * GGUF_PIECE_TILES);
      uint8_t *mine = table + piece * gguf_table_bytes(width, GGUF_PIECE_TILES);
      const uint32_t run = lane & 31u, q = outHead * (kDim / 4u) + run, g = q / 8u, half = (q / 4u) % 2u, kq = q % 4u;
      const uint2 raw = *reinterpret_cast<const uint2 *>(&outputs[token][4u * run]);
      const uint32_t x0 = raw.x & 0xFFFFu, x1 = raw.x >> 16, x2 = raw.y & 0xFFFFu, x3 = raw.y >> 16;
      float sum = (bf16_bits_to_float(x0) + bf16_bits_to_float(x1)) + (bf16_bits_to_float(x2) + bf16_bits_to_float(x3));
      const float s1 = __shfl_down(sum, 1, 64), s2 = __shfl_down(sum, 2, 64), s3 = __shfl_down(sum, 3, 64);
      sum = ((sum + s1) + s2) + s3;
      const float other = __shfl_down(sum, 4, 64);
      if (lane < 32u) {
        // operand elements 4 half + {0,1,2,3} are inputs 4 kq + {0,2,1,3} of the half
        reinterpret_cast<uint2 *>(mine)[((size_t(tile) * G + g) * 64u + kq * 16u + r) * 2u + half] = make_uint2(x0 | (x2 << 16), x1 | (x3 << 16));
        if (kq == 0) {
          float *sums32 = reinterpret_cast<float *>(mine + gguf_table_sums32_offset(width, tiles));
          float *sums16 = reinterpret_cast<float *>(mine + gguf_table_sums16_offset(width, tiles));
          sums16[(size_t(tile) * 2u * G + 2u * g + half) * 16u + r] = sum;
          if (half == 0) sums32[(size_t(tile) * G + g) * 16u + r] = sum + other;
        }
      }
    }
  }
}
SP_REGISTER_KERNEL("gdn_decode", &gdn_decode);

// gdn_fold: grid (value_heads, layers), 1024 threads (gdn.metal:630-698, exact cells).
__global__ __launch_bounds__(64 * kWaves) void gdn_fold(uint8_t *__restrict__ states, uint8_t *__restrict__ tape,
                                                const uint32_t *__restrict__ retained, GdnFoldParams p) {
  __shared__ __align__(16) Pending pending;
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, head = blockIdx.x, layer = blockIdx.y;
  const GdnShapeParams s = p.shape;
  const uint32_t rows = p.rows, path = retained[0];
  if (uint32_t(__builtin_popcount(path)) < rows) return;
  const uint32_t perKey = s.value_heads / s.key_heads, keyHead = head / perKey, keyWidth = s.key_heads * kDim, C = s.conv_dim;
  const Tape step = tape_at(tape, p.step_tape + uint64_t(layer) * p.tape_layer_bytes, s);
  const uint8_t *cell = states + p.state_cell;
  uint8_t *fold = states + p.fold_cell;
  for (uint32_t token = wave; token < rows; token += kWaves) load_pending(step, pending, token, path_row(path, token), head, s, lane);
  if (wave < kTaps - 1) {
    const History history = history_of(reinterpret_cast<const uint16_t *>(cell + uint64_t(layer) * p.conv_layer_bytes), step.inputs, C, rows, path);
    uint16_t *carried = reinterpret_cast<uint16_t *>(fold + uint64_t(layer) * p.conv_layer_bytes) + size_t(wave) * C;
    const uint32_t qChannel = keyHead * kDim, kChannel = keyWidth + keyHead * kDim, vChannel = 2 * keyWidth + head * kDim;
#pragma unroll
    for (uint32_t part = 0; part < 2; ++part) {
      const uint32_t d = lane + 64u * part;
      carried[vChannel + d] = history.row[wave][vChannel + d];
      if (head % perKey == 0) {
        carried[qChannel + d] = history.row[wave][qChannel + d];
        carried[kChannel + d] = history.row[wave][kChannel + d];
      }
    }
  }
  __syncthreads();
  const float *stateIn = reinterpret_cast<const float *>(cell + p.convolution_state_bytes + uint64_t(layer) * p.recurrent_layer_bytes);
  float *stateOut = reinterpret_cast<float *>(fold + p.convolution_state_bytes + uint64_t(layer) * p.recurrent_layer_bytes);
  const uint32_t half = lane >> 5, column = 4u * (lane & 31u);
  for (uint32_t batch = 0; batch < kDim / (2u * kWaves); batch += kInFlight) {
    uint32_t valueDim[kInFlight];
    float state[kInFlight][4];
#pragma unroll
    for (int r = 0; r < kInFlight; ++r) {
      valueDim[r] = (batch + r) * 2u * kWaves + wave * 2u + half;
      const float4 loaded = *reinterpret_cast<const float4 *>(stateIn + (size_t(head) * kDim + valueDim[r]) * kDim + column);
      state[r][0] = loaded.x;
      state[r][1] = loaded.y;
      state[r][2] = loaded.z;
      state[r][3] = loaded.w;
    }
    for (uint32_t token = 0; token < rows; ++token)
      advance<kInFlight>(state, pending.keys[token], pending.values[token], valueDim, pending.decay[token],
                         bf16_bits_to_float(pending.beta[token]), column);
#pragma unroll
    for (int r = 0; r < kInFlight; ++r)
      *reinterpret_cast<float4 *>(stateOut + (size_t(head) * kDim + valueDim[r]) * kDim + column) =
          make_float4(state[r][0], state[r][1], state[r][2], state[r][3]);
  }
}
SP_REGISTER_KERNEL("gdn_fold", &gdn_fold);

} // namespace splash::kernels
