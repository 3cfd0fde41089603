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

// A row's convolution + SiLU of one channel from its four taps, oldest first (gdn_primitives.h:37-50).
__device__ __forceinline__ float conv_silu(const uint16_t *const (&taps)[kTaps], const uint16_t *conv_weights, uint32_t channel) {
  float value = 0.f;
#pragma unroll
  for (uint32_t tap = 0; tap < kTaps; ++tap)
    value += bf16_bits_to_float(taps[tap][channel]) * bf16_bits_to_float(conv_weights[size_t(channel) * kTaps + tap]);
  value = round_bf16(value);
  return round_bf16(silu_of(value));
}

// A row's normalized, scaled query and key and its value of one head as bf16 bits, lane l the
// dimensions l and 64 + l (gdn.metal:198-232): q and k are RMS-normed over the head, rounded, then
// scaled by 1/128 and 1/sqrt(128).
struct HeadRow {
  uint32_t query[2], key[2], value[2];
};
__device__ __forceinline__ HeadRow head_row(const uint16_t *const (&taps)[kTaps], const uint16_t *conv_weights, uint32_t qChannel,
                                            uint32_t kChannel, uint32_t vChannel, uint32_t lane) {
  float q[2], k[2], v[2];
#pragma unroll
  for (uint32_t part = 0; part < 2; ++part) {
    const uint32_t d = lane + 64u * part;
    q[part] = conv_silu(taps, conv_weights, qChannel + d);
    k[part] = conv_silu(taps, conv_weights, kChannel + d);
    v[part] = conv_silu(taps, conv_weights, vChannel + d);
  }
  const float qScale = 1.0f / sqrtf(head_sum(q[0] * q[0], q[1] * q[1]) / float(kDim) + 1e-6f);
  const float kScale = 1.0f / sqrtf(head_sum(k[0] * k[0], k[1] * k[1]) / float(kDim) + 1e-6f);
  HeadRow row;
#pragma unroll
  for (uint32_t part = 0; part < 2; ++part) {
    row.query[part] = float_to_bf16_bits(round_bf16(q[part] * qScale) * 0.0078125f);
    row.key[part] = float_to_bf16_bits(round_bf16(k[part] * kScale) * 0.08838834765f);
    row.value[part] = float_to_bf16_bits(v[part]);
  }
  return row;
}

// A row's gates of one value head (gdn_primitives.h:65-73): beta = bf16(sigmoid(b)); decay =
// exp(a_scale bf16(softplus(bf16(a + dt_bias)))).
struct Gates {
  uint32_t beta;
  float decay;
};
__device__ __forceinline__ Gates gates_of(const uint16_t *inputs, uint32_t bOffset, uint32_t aOffset, uint32_t head,
                                          const float *a_scale, const uint16_t *dt_bias) {
  Gates g;
  g.beta = float_to_bf16_bits(sigmoid_of(bf16_bits_to_float(inputs[bOffset + head])));
  const float x = round_bf16(bf16_bits_to_float(inputs[aOffset + head]) + bf16_bits_to_float(dt_bias[head]));
  const float softplus = round_bf16(fmaxf(x, 0.0f) + __builtin_amdgcn_logf(1.0f + exp2_fast(-kLog2e * fabsf(x))) * 0.69314718056f);
  g.decay = exp2_fast(kLog2e * (a_scale[head] * softplus));
  return g;
}

// The gated output norm of a row's 128 recurrent values of one head, lane l the dimensions l and
// 64 + l, as bf16 bits (gdn.metal:489-526): RMS norm with the mixer's weight, rounded, times silu(z)
// (or sigmoid(z)) of the row's gate columns `z`.
__device__ __forceinline__ void gated_norm(const float (&value)[2], const void *norm_weight, uint32_t flags, const uint16_t *z_row,
                                           uint32_t lane, uint32_t (&bits)[2]) {
  const float inverse = 1.0f / sqrtf(head_sum(value[0] * value[0], value[1] * value[1]) / float(kDim) + 1e-6f);
#pragma unroll
  for (uint32_t part = 0; part < 2; ++part) {
    const uint32_t d = lane + 64u * part;
    const float weight = (flags & GDN_FLOAT_NORM) ? static_cast<const float *>(norm_weight)[d]
                                                  : bf16_bits_to_float(static_cast<const uint16_t *>(norm_weight)[d]);
    const float normalized = round_bf16((value[part] * inverse) * weight);
    const float z = bf16_bits_to_float(z_row[d]);
    const float gated = (normalized * ((flags & GDN_SIGMOID_GATE) ? 1.0f : z)) / (1.0f + exp2_fast(-kLog2e * z));
    bits[part] = float_to_bf16_bits(gated);
  }
}

// One token's delta-rule step on the wave's state rows (R pairs, a row per half-wave): decay,
// memory, delta, update (gdn.metal:270-298). k: the lane's four key columns; value: each row's value.
template <int R>
__device__ __forceinline__ void advance_rows(float (&state)[R][4], const float (&k)[4], const float (&value)[R], float decay, float beta) {
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
    const float delta = (value[r] - memory[r]) * beta;
#pragma unroll
    for (int i = 0; i < 4; ++i) state[r][i] += k[i] * delta;
  }
}
// The same from a token's staged key row and value row (bf16 in LDS).
template <int R>
__device__ __forceinline__ void advance(float (&state)[R][4], const uint16_t *key, const uint16_t *value_row, const uint32_t (&value_dim)[R],
                                        float decay, float beta, uint32_t column) {
  const uint2 kb = *reinterpret_cast<const uint2 *>(key + column);
  const float k[4] = {bf16_bits_to_float(kb.x & 0xFFFFu), bf16_bits_to_float(kb.x >> 16), bf16_bits_to_float(kb.y & 0xFFFFu),
                      bf16_bits_to_float(kb.y >> 16)};
  float value[R];
#pragma unroll
  for (int r = 0; r < R; ++r) value[r] = bf16_bits_to_float(value_row[value_dim[r]]);
  advance_rows<R>(state, k, value, decay, beta);
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
    const HeadRow row = head_row(taps, conv_weights, qChannel, kChannel, vChannel, lane);
    const uint16_t *inputs = rowsIn + size_t(token) * P;
#pragma unroll
    for (uint32_t part = 0; part < 2; ++part) {
      const uint32_t d = lane + 64u * part;
      queries[token][d] = uint16_t(row.query[part]);
      keys[token][d] = uint16_t(row.key[part]);
      values[token][d] = uint16_t(row.value[part]);
      stepTape.inputs[size_t(token) * C + vChannel + d] = inputs[vChannel + d];
      stepTape.kv[size_t(token) * kvWidth + keyWidth + head * kDim + d] = uint16_t(row.value[part]);
      if (sharedWriter) {
        stepTape.inputs[size_t(token) * C + qChannel + d] = inputs[qChannel + d];
        stepTape.inputs[size_t(token) * C + kChannel + d] = inputs[kChannel + d];
        stepTape.kv[size_t(token) * kvWidth + keyHead * kDim + d] = uint16_t(row.key[part]);
      }
    }
    if (lane == 0) {
      const Gates gates = gates_of(inputs, bOffset, aOffset, head, a_scale, dt_bias);
      stepTape.beta[token * s.value_heads + head] = uint16_t(gates.beta);
      stepTape.decay[token * s.value_heads + head] = gates.decay;
      betas[token] = uint16_t(gates.beta);
      decays[token] = gates.decay;
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
    uint32_t gated[2];
    gated_norm(value, norm_weight, p.flags, rowsIn + size_t(token) * P + zOffset + head * kDim, lane, gated);
#pragma unroll
    for (uint32_t part = 0; part < 2; ++part) {
      const uint32_t d = lane + 64u * part;
      hidden[(size_t(L.first_row + token) * s.value_heads + outHead) * kDim + d] = uint16_t(gated[part]);
      outputs[token][d] = uint16_t(gated[part]);  // this wave's row: read above, and below for the table
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

// ---- prefill: a prompt chunk, whose rows all enter the state (the reference's kernels/prefill/gdn.metal) ----
//
// Three passes over a run of `tokens` rows of one lane and layer. The rows' k, v and gates are those
// a verify step would leave on its tape for the same rows (the same device functions compute both) and
// a state row's recurrence is `advance`, the fold's: a prompt that enters the state through these
// kernels leaves the cell, bit for bit, that the same rows leave when they enter as accepted verify
// blocks. Only the outputs differ in form: here a row reads the state after its own token, o = S_t q_t
// (gdn.metal:291-298), where a verify block's rows read the state before the block.

// gdn_prefill_prepare: grid (value_heads, ceil(tokens / 4)), 256 threads, a wave per (row, value head),
// lane l the dimensions l and 64 + l: convolution + SiLU, q/k norms, gates (prefill/gdn.metal:196-262).
// The head's value rows, its gates and, from the first value head of a key head, the key head's query
// and key rows leave to the run's buffers; the workgroups of the first rows also write the convolution
// carry after the run's last row.
__global__ __launch_bounds__(256) void gdn_prefill_prepare(const uint16_t *__restrict__ packed, const uint16_t *__restrict__ conv_weights,
                                                           uint8_t *__restrict__ states, const float *__restrict__ a_scale,
                                                           const uint16_t *__restrict__ dt_bias, uint16_t *__restrict__ queries,
                                                           uint16_t *__restrict__ keys, uint16_t *__restrict__ values,
                                                           float *__restrict__ decay, uint16_t *__restrict__ beta, GdnPrefillParams p) {
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, head = blockIdx.x, token = blockIdx.y * 4u + wave;
  const GdnShapeParams s = p.shape;
  const uint32_t perKey = s.value_heads / s.key_heads, keyHead = head / perKey, keyWidth = s.key_heads * kDim;
  const uint32_t valueWidth = s.value_heads * kDim, C = s.conv_dim, P = s.packed_width;
  const uint32_t bOffset = C + valueWidth, aOffset = bOffset + s.value_heads;
  const bool sharedWriter = head % perKey == 0;
  const uint16_t *convIn = reinterpret_cast<const uint16_t *>(states + p.current_cell + uint64_t(p.layer) * p.conv_layer_bytes);
  uint16_t *convOut = reinterpret_cast<uint16_t *>(states + p.next_cell + uint64_t(p.layer) * p.conv_layer_bytes);
  const uint32_t qChannel = keyHead * kDim, kChannel = keyWidth + keyHead * kDim, vChannel = 2 * keyWidth + head * kDim;
  // input position i of the run's history: the carried rows, then the run's own (gdn_primitives.h:20-35)
  auto input = [&](uint32_t position) __attribute__((always_inline)) -> const uint16_t * {
    return position < kTaps - 1 ? convIn + size_t(position) * C : packed + size_t(p.first + position - (kTaps - 1)) * P;
  };
  if (blockIdx.y == 0 && wave < kTaps - 1) {
    const uint16_t *source = input(p.tokens + wave);
#pragma unroll
    for (uint32_t part = 0; part < 2; ++part) {
      const uint32_t d = lane + 64u * part;
      convOut[size_t(wave) * C + vChannel + d] = source[vChannel + d];
      if (sharedWriter) {
        convOut[size_t(wave) * C + qChannel + d] = source[qChannel + d];
        convOut[size_t(wave) * C + kChannel + d] = source[kChannel + d];
      }
    }
  }
  if (token >= p.tokens) return;
  const uint16_t *taps[kTaps];
#pragma unroll
  for (uint32_t tap = 0; tap < kTaps; ++tap) taps[tap] = input(token + tap);
  const HeadRow row = head_row(taps, conv_weights, qChannel, kChannel, vChannel, lane);
  const size_t at = size_t(p.first) + token;  // the row's place in the chunk's buffers
#pragma unroll
  for (uint32_t part = 0; part < 2; ++part) {
    const uint32_t d = lane + 64u * part;
    values[at * valueWidth + head * kDim + d] = uint16_t(row.value[part]);
    if (sharedWriter) {
      queries[at * keyWidth + keyHead * kDim + d] = uint16_t(row.query[part]);
      keys[at * keyWidth + keyHead * kDim + d] = uint16_t(row.key[part]);
    }
  }
  if (lane == 0) {
    const Gates gates = gates_of(packed + at * P, bOffset, aOffset, head, a_scale, dt_bias);
    beta[at * s.value_heads + head] = uint16_t(gates.beta);
    decay[at * s.value_heads + head] = gates.decay;
  }
}
SP_REGISTER_KERNEL("gdn_prefill_prepare", &gdn_prefill_prepare);

// gdn_prefill_scan: grid (value_heads * 128 / GDN_SCAN_STATE_ROWS), 256 threads. A workgroup carries GDN_SCAN_STATE_ROWS
// rows of a head's state through the run in registers, token by token (prefill/gdn.metal:11-23): a wave holds a
// pair of rows, a row per half-wave, lane j of a half the key columns 4 j .. 4 j + 3, as the fold does.
// Blocks of GDN_SCAN_BLOCK tokens of k, q, v and gates are staged in LDS while the block after them is
// in flight to registers, so the dependent chain of a token reads LDS only; a block's outputs collect
// in LDS and leave as whole 16-byte runs. Eight rows a workgroup put two workgroups on a compute unit and
// two waves on a SIMD, each other's cover for the chain's latencies.
__global__ __launch_bounds__(256) void gdn_prefill_scan(const uint16_t *__restrict__ queries, const uint16_t *__restrict__ keys,
                                                        const uint16_t *__restrict__ values, const float *__restrict__ decay,
                                                        const uint16_t *__restrict__ beta, uint8_t *__restrict__ states,
                                                        uint16_t *__restrict__ recurrent_rows, GdnPrefillParams p) {
  constexpr uint32_t B = GDN_SCAN_BLOCK, R = GDN_SCAN_STATE_ROWS, kGroups = kDim / R, kPairs = R / 8, kPieces = R / 8;
  static_assert(B * kDim * 2 == 256 * 16, "a thread stages sixteen bytes of a block's keys and of its queries");
  static_assert(R == 4 * 2 * kPairs && R % 8 == 0, "four waves of kPairs pairs of rows hold a workgroup's state rows, whole 16-byte pieces of a token's values");
  __shared__ __align__(16) uint16_t sk[2][B][kDim], sq[2][B][kDim];
  __shared__ __align__(16) uint16_t sv[2][B][R], so[B][R];
  __shared__ float sd[2][B];
  __shared__ uint16_t sb[2][B];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const GdnShapeParams s = p.shape;
  const uint32_t head = blockIdx.x / kGroups, rowBase = (blockIdx.x % kGroups) * R;
  const uint32_t keyHead = head / (s.value_heads / s.key_heads), keyWidth = s.key_heads * kDim, valueWidth = s.value_heads * kDim;
  const uint32_t half = lane >> 5, column = 4u * (lane & 31u), tokens = p.tokens;
  const float *stateIn = reinterpret_cast<const float *>(states + p.current_cell + p.convolution_state_bytes + uint64_t(p.layer) * p.recurrent_layer_bytes);
  float *stateOut = reinterpret_cast<float *>(states + p.next_cell + p.convolution_state_bytes + uint64_t(p.layer) * p.recurrent_layer_bytes);
  uint32_t local[kPairs];
  float state[kPairs][4];
#pragma unroll
  for (uint32_t r = 0; r < kPairs; ++r) {
    local[r] = (r * 4u + wave) * 2u + half;
    const float4 loaded = *reinterpret_cast<const float4 *>(stateIn + (size_t(head) * kDim + rowBase + local[r]) * kDim + column);
    state[r][0] = loaded.x;
    state[r][1] = loaded.y;
    state[r][2] = loaded.z;
    state[r][3] = loaded.w;
  }
  // Rows at or past `tokens` keep what the registers held and are staged as they are: the loop below stops at the
  // run's last token, so those slots are never read.
  uint4 keyFetch = make_uint4(0, 0, 0, 0), queryFetch = keyFetch, valueFetch = keyFetch;
  float decayFetch = 0.f;
  uint16_t betaFetch = 0;
  auto fetch = [&](uint32_t start) __attribute__((always_inline)) {
    const uint32_t token = start + tid / 16u;
    if (token < tokens) {
      const size_t at = (size_t(p.first) + token) * keyWidth + keyHead * kDim + (tid % 16u) * 8u;
      keyFetch = *reinterpret_cast<const uint4 *>(keys + at);
      queryFetch = *reinterpret_cast<const uint4 *>(queries + at);
    }
    if (tid < kPieces * B && start + tid / kPieces < tokens)
      valueFetch = *reinterpret_cast<const uint4 *>(values + (size_t(p.first) + start + tid / kPieces) * valueWidth + head * kDim + rowBase + (tid % kPieces) * 8u);
    if (tid < B && start + tid < tokens) {
      decayFetch = decay[(size_t(p.first) + start + tid) * s.value_heads + head];
      betaFetch = beta[(size_t(p.first) + start + tid) * s.value_heads + head];
    }
  };
  auto stage = [&](uint32_t buffer) __attribute__((always_inline)) {
    *reinterpret_cast<uint4 *>(&sk[buffer][tid / 16u][(tid % 16u) * 8u]) = keyFetch;
    *reinterpret_cast<uint4 *>(&sq[buffer][tid / 16u][(tid % 16u) * 8u]) = queryFetch;
    if (tid < kPieces * B) *reinterpret_cast<uint4 *>(&sv[buffer][tid / kPieces][(tid % kPieces) * 8u]) = valueFetch;
    if (tid < B) {
      sd[buffer][tid] = decayFetch;
      sb[buffer][tid] = betaFetch;
    }
  };
  fetch(0);
  stage(0);
  __syncthreads();
  for (uint32_t start = 0, buffer = 0; start < tokens; start += B, buffer ^= 1u) {
    const bool more = start + B < tokens;
    if (more) fetch(start + B);
    const uint32_t count = min(B, tokens - start);
    // A token's operands leave LDS one token ahead of their use, and a token's output is off the state's dependent
    // chain: its lanes' products wait one token, and their sum over the half-wave runs beside the next token's update.
    struct Operands {
      uint2 key, query;
      float decay;
      uint32_t beta, value[kPairs];
    };
    auto operands = [&](uint32_t t) __attribute__((always_inline)) {
      Operands o;
      o.key = *reinterpret_cast<const uint2 *>(&sk[buffer][t][column]);
      o.query = *reinterpret_cast<const uint2 *>(&sq[buffer][t][column]);
      o.decay = sd[buffer][t];
      o.beta = sb[buffer][t];
#pragma unroll
      for (uint32_t r = 0; r < kPairs; ++r) o.value[r] = sv[buffer][t][local[r]];
      return o;
    };
    float partial[kPairs] = {};
    Operands ahead = operands(0);
    for (uint32_t t = 0; t <= count; ++t) {
      float sum[kPairs];
#pragma unroll
      for (uint32_t r = 0; r < kPairs; ++r) sum[r] = partial[r];
      if (t < count) {
        const Operands now = ahead;
        ahead = operands(min(t + 1u, B - 1u));  // past the block's last token: a staged slot nobody uses
        const float k[4] = {bf16_bits_to_float(now.key.x & 0xFFFFu), bf16_bits_to_float(now.key.x >> 16),
                            bf16_bits_to_float(now.key.y & 0xFFFFu), bf16_bits_to_float(now.key.y >> 16)};
        const float q[4] = {bf16_bits_to_float(now.query.x & 0xFFFFu), bf16_bits_to_float(now.query.x >> 16),
                            bf16_bits_to_float(now.query.y & 0xFFFFu), bf16_bits_to_float(now.query.y >> 16)};
        float value[kPairs];
#pragma unroll
        for (uint32_t r = 0; r < kPairs; ++r) value[r] = bf16_bits_to_float(now.value[r]);
        advance_rows<kPairs>(state, k, value, now.decay, bf16_bits_to_float(now.beta));
#pragma unroll
        for (uint32_t r = 0; r < kPairs; ++r) {
          partial[r] = 0.f;
#pragma unroll
          for (int i = 0; i < 4; ++i) partial[r] += state[r][i] * q[i];
        }
      }
      if (t > 0) {
#pragma unroll
        for (uint32_t r = 0; r < kPairs; ++r) sum[r] = half_sum(sum[r]);
        if ((lane & 31u) == 0) {
#pragma unroll
          for (uint32_t r = 0; r < kPairs; ++r) so[t - 1][local[r]] = uint16_t(float_to_bf16_bits(sum[r]));
        }
      }
    }
    __syncthreads();  // the block's outputs are whole, and no wave reads its staged rows any more
    if (tid < kPieces * count)
      *reinterpret_cast<uint4 *>(recurrent_rows + (size_t(p.first) + start + tid / kPieces) * valueWidth + head * kDim + rowBase + (tid % kPieces) * 8u) =
          *reinterpret_cast<const uint4 *>(&so[tid / kPieces][(tid % kPieces) * 8u]);
    if (more) stage(buffer ^ 1u);
    __syncthreads();
  }
#pragma unroll
  for (uint32_t r = 0; r < kPairs; ++r)
    *reinterpret_cast<float4 *>(stateOut + (size_t(head) * kDim + rowBase + local[r]) * kDim + column) =
        make_float4(state[r][0], state[r][1], state[r][2], state[r][3]);
}
SP_REGISTER_KERNEL("gdn_prefill_scan", &gdn_prefill_scan);

// gdn_prefill_gate: grid (value_heads, ceil(tokens / 4)), 256 threads, a wave per (row, value head): the gated
// output norm of the scan's rows (prefill/gdn.metal:312-341, gdn.metal:489-526).
__global__ __launch_bounds__(256) void gdn_prefill_gate(const uint16_t *__restrict__ recurrent_rows, const uint16_t *__restrict__ packed,
                                                        const void *__restrict__ norm_weight, uint16_t *__restrict__ hidden,
                                                        GdnPrefillParams p) {
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, head = blockIdx.x;
  if (blockIdx.y * 4u + wave >= p.tokens) return;
  const size_t token = size_t(p.first) + blockIdx.y * 4u + wave;
  const GdnShapeParams s = p.shape;
  const uint32_t perKey = s.value_heads / s.key_heads, valueWidth = s.value_heads * kDim;
  const uint32_t outHead = (p.flags & GDN_TILED_HEADS) ? (head % perKey) * s.key_heads + head / perKey : head;
  float value[2];
#pragma unroll
  for (uint32_t part = 0; part < 2; ++part)
    value[part] = bf16_bits_to_float(recurrent_rows[token * valueWidth + head * kDim + lane + 64u * part]);
  uint32_t gated[2];
  gated_norm(value, norm_weight, p.flags, packed + token * s.packed_width + s.conv_dim + head * kDim, lane, gated);
#pragma unroll
  for (uint32_t part = 0; part < 2; ++part)
    hidden[(token * s.value_heads + outHead) * kDim + lane + 64u * part] = uint16_t(gated[part]);
}
SP_REGISTER_KERNEL("gdn_prefill_gate", &gdn_prefill_gate);

} // namespace splash::kernels
