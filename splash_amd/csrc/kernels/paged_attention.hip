// Block-causal attention of a verify block over the paged INT8 KV cache, for gfx950 (the
// reference's kernels/shared/attention_qkv.metal, paged_attention.metal, kv_path_commit.metal and
// common/paged_attention_tile.h, attention_qkv_prepare.h, attention_store.h).
//
//   attention_q8_qkv_d<D>     per (head, row, sequence): RMS-norm q and k, partial RoPE, stage the
//                             query rows, quantize k and v into the row's page slot.
//   attention_q8_split_d<D>_g<G>  per (KV head, history split, sequence): flash-decoding page loop
//                             over the split's 64-token steps for all 16 G fused rows of the head.
//   attention_reduce_d<D>     per (query head, row, sequence): merge the splits in split order.
//   attention_q8_commit_d<D>  per (KV head, sequence): move the retained path's slots to their depths.
//
// The page loop keeps the reference's rules (paged_attention_tile.h:179-285): score =
// (q . k_codes) key_scale / sqrt(D), computed on the stored integer codes; online softmax per step;
// P is folded with value_scale before the P.V product, which also runs on the stored codes. Both
// products are fp16 MFMAs on exact integer operands: a stored code c becomes the fp16 number
// 1152 + c by one byte permute (0x6400 | (c ^ 0x80), no conversion instruction), and the constant
// 1152 is removed exactly afterwards with the row's sum of q (scores) and of P (outputs), the latter
// from one more MFMA against a tile of ones. Scores are kept transposed (tokens x rows) so that a
// lane owns one fused row from the first MFMA to the last: row maxima, sums and rescales never
// cross lanes except over the four lanes that share a row.
#include "abi/Gguf.h"
#include "abi/PagedAttention.h"
#include "backend/KernelRegistry.hpp"
#include "kernels/device_common.hpp"
#include <type_traits>

namespace splash::kernels {

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;

constexpr float kCodeOffset = 1152.0f;  // fp16(0x6400 | u) = 1024 + u, u = code + 128
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kPScale = 1024.0f;  // P is carried times 2^10 so that small weights stay normal fp16

// Bytes b0..b3 of x as two registers of fp16 numbers 1024 + b: [b0, b1] and [b2, b3].
__device__ __forceinline__ uint2 bytes_to_f16(uint32_t x) {
  return make_uint2(__builtin_amdgcn_perm(0x64646464u, x, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u));
}

template <int N> __device__ __forceinline__ float block_sum(float v, float *scratch, uint32_t tid) {
  v = wave_sum(v);
  if constexpr (N > 64) {
    if ((tid & 63u) == 0) scratch[tid >> 6] = v;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < N / 64; ++w) total += scratch[w];
    __syncthreads();
    return total;
  }
  return v;
}
template <int N> __device__ __forceinline__ float block_max(float v, float *scratch, uint32_t tid) {
  v = wave_max(v);
  if constexpr (N > 64) {
    if ((tid & 63u) == 0) scratch[tid >> 6] = v;
    __syncthreads();
    float total = scratch[0];
#pragma unroll
    for (int w = 1; w < N / 64; ++w) total = fmaxf(total, scratch[w]);
    __syncthreads();
    return total;
  }
  return v;
}

// The page of logical page `index` of a sequence.
__device__ __forceinline__ uint8_t *page_of(uint8_t *pool, const uint64_t *page_table, const AttentionSequence &seq,
                                            uint64_t page_bytes, uint32_t index) {
  return pool + page_table[seq.table_first + index] * page_bytes;
}

// ---------------------------------------------------------------------------------------------
// attention_q8_qkv: grid (q_heads + kv_heads, 16, sequences), D threads.
// Staged queries: fp16 [sequence][kv head][group head][16 rows][D] (rows past the block zero) and
// their fp32 sums [sequence][kv head][group head][16].
// ---------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(D) void attention_q8_qkv(const uint16_t *__restrict__ qkv, const uint16_t *__restrict__ q_norm,
                                                      const uint16_t *__restrict__ k_norm, const float *__restrict__ rope_cos,
                                                      const float *__restrict__ rope_sin, _Float16 *__restrict__ queries,
                                                      float *__restrict__ qsums, const uint64_t *__restrict__ page_table,
                                                      uint8_t *__restrict__ pool, AttentionParams p) {
  __shared__ float scratch[4];
  __shared__ float normalized[D];
  const uint32_t tid = threadIdx.x, head = blockIdx.x, row = blockIdx.y, z = blockIdx.z;
  const AttentionSequence seq = p.sequence[z];
  const bool query = head < p.q_heads;
  const uint32_t group = p.q_heads / p.kv_heads;
  if (row >= seq.rows) {
    if (query) {
      const uint32_t kv = head / group, g = head % group;
      const size_t at = ((size_t(z) * p.kv_heads + kv) * group + g) * 16u + row;
      if (p.int8_queries) reinterpret_cast<int8_t *>(queries)[at * D + tid] = 0;
      else queries[at * D + tid] = _Float16(0.f);
      if (tid == 0) qsums[at] = 0.f;
    }
    return;
  }
  const uint32_t index = query ? head : head - p.q_heads;
  const size_t packed = size_t(seq.first_row) + row;
  // A gated layer's row holds each query head's queries, then its gate (attention_gate.h:27-31).
  const uint32_t queryStride = p.gated ? 2u * D : uint32_t(D);
  const uint16_t *source = qkv + packed * p.qkv_stride + (query ? index * queryStride : p.q_heads * queryStride + index * D);
  const float element = bf16_bits_to_float(source[tid]);
  float result = element;
  if (p.normalize) {
    // attention_qkv_prepare.h:59-66: inv = rsqrt(sum x^2 / D + 1e-6); n = bf16(x inv w)
    const float total = block_sum<D>(element * element, scratch, tid);
    const float inverse = 1.0f / sqrtf(total / float(D) + 1e-6f);  // correctly rounded, as the CPU oracle's
    result = round_bf16(element * inverse * bf16_bits_to_float((query ? q_norm : k_norm)[tid]));
  }
  if (p.rotary_pairs) {
    normalized[tid] = result;
    __syncthreads();
    if (tid < 2 * p.rotary_pairs) {
      const uint32_t pair = tid % p.rotary_pairs;
      const float first = normalized[pair], second = normalized[pair + p.rotary_pairs];
      const float cosine = rope_cos[packed * p.rotary_pairs + pair], sine = rope_sin[packed * p.rotary_pairs + pair];
      result = tid < p.rotary_pairs ? round_bf16(first * cosine - second * sine) : round_bf16(second * cosine + first * sine);
    }
  }
  if (query) {
    const uint32_t kv = index / group, g = index % group;
    const size_t at = ((size_t(z) * p.kv_heads + kv) * group + g) * 16u + row;
    if (p.int8_queries) {
      // common/int8_activations.h:22-28: code = clamp(rint(x (127 / m))), the quotient rounded first; scale = m / 127; a
      // head at or below 2^-100 codes as zeros with scale 0; one that is not finite takes a NaN scale. The codes lie
      // where the fp16 queries would, one byte a dimension, and the scale in the sums' slot.
      const uint32_t bits = __builtin_bit_cast(uint32_t, result);
      const float notFinite = block_max<D>((bits & 0x7F800000u) == 0x7F800000u ? 1.f : 0.f, scratch, tid);
      const float largest = block_max<D>(fabsf(result), scratch, tid);
      const bool coded = largest > 0x1p-100f;
      const float inverse = coded ? 127.0f / largest : 0.0f;
      const float code = fminf(fmaxf(rintf(result * inverse), -127.0f), 127.0f);
      reinterpret_cast<int8_t *>(queries)[at * D + tid] = notFinite != 0.f ? int8_t(0) : int8_t(code);
      if (tid == 0) qsums[at] = notFinite != 0.f ? __builtin_bit_cast(float, 0x7FC00000u) : coded ? largest / 127.0f : 0.0f;
      return;
    }
    const _Float16 staged = _Float16(result);
    queries[at * D + tid] = staged;
    const float sum = block_sum<D>(float(staged), scratch, tid);
    if (tid == 0) qsums[at] = sum;
    return;
  }
  // attention_store.h:52-85: scale = max / 127, code = clamp(rint(v 127 / max)); the scale is stored fp16.
  const float value = bf16_bits_to_float(source[p.kv_heads * D + tid]);
  const float keyMax = block_max<D>(fabsf(result), scratch, tid), valueMax = block_max<D>(fabsf(value), scratch, tid);
  const uint32_t slot = seq.committed + row, token = slot % ATTENTION_PAGE_TOKENS;
  uint8_t *page = page_of(pool, page_table, seq, p.page_bytes, slot / ATTENTION_PAGE_TOKENS);
  auto code = [](float v, float maximum) -> int8_t {
    if (maximum == 0.0f) return 0;
    const int q = int(rintf(v * 127.0f / maximum));
    return int8_t(q < -127 ? -127 : q > 127 ? 127 : q);
  };
  reinterpret_cast<int8_t *>(page)[attention_key_index(index, token, tid, D)] = code(result, keyMax);
  reinterpret_cast<int8_t *>(page + attention_page_values_offset(p.kv_heads, D))[attention_value_index(index, token, tid, D)] =
      code(value, valueMax);
  if (tid == 0) {
    uint16_t *ks = reinterpret_cast<uint16_t *>(page + attention_page_key_scales_offset(p.kv_heads, D));
    uint16_t *vs = reinterpret_cast<uint16_t *>(page + attention_page_value_scales_offset(p.kv_heads, D));
    ks[attention_scale_index(index, token)] = uint16_t(float_to_half_bits(keyMax == 0.0f ? 0.0f : keyMax / 127.0f));
    vs[attention_scale_index(index, token)] = uint16_t(float_to_half_bits(valueMax == 0.0f ? 0.0f : valueMax / 127.0f));
  }
}
SP_REGISTER_KERNEL("attention_q8_qkv_d128", &attention_q8_qkv<128>);
SP_REGISTER_KERNEL("attention_q8_qkv_d64", &attention_q8_qkv<64>);

// ---------------------------------------------------------------------------------------------
// attention_q8_split: grid (kv_heads, splits, sequences), 256 threads.
// Partials: O fp32 [sequence][kv head][split][16 G fused rows][D], (max, sum) fp32 pairs
// [sequence][kv head][split][16 G]; the max is in the log2 domain of the scaled scores.
// ---------------------------------------------------------------------------------------------
// I8: the queries are INT8 codes with a scale a fused row (attention_q8_qkv staged them so): the score product is one
// v_mfma_i32_16x16x64_i8 per 64 dimensions on the keys' stored bytes, which pass through LDS as they are (no widening,
// no offset to remove), and a row's scale multiplies its scores after the product.
typedef __attribute__((ext_vector_type(4))) int i32x4;
template <int D, int G, bool I8>
__global__ __launch_bounds__(256, 2) void attention_q8_split(const _Float16 *__restrict__ queries, const float *__restrict__ qsums,
                                                          const AttentionTreeRow *__restrict__ tree,
                                                          const uint64_t *__restrict__ page_table, uint8_t *__restrict__ pool,
                                                          _Float16 *__restrict__ partialO, float *__restrict__ partialML,
                                                          AttentionParams p) {
  constexpr int kStep = 64, JD = D / 32, DT = D / 16;
  constexpr int kTiles = (G + 3) / 4;  // fused-row tiles (one query head's 16 rows each) per wave
  constexpr int kKeyVectors = kStep * D / 16 / 256, kValueVectors = kKeyVectors;
  static_assert(kKeyVectors >= 1, "a step's keys fill the workgroup's loads");
  // keys: fp16 numbers 1152 + code, or (I8) the stored bytes, a token's row padded by 16 bytes either way
  constexpr int kKeyRow = I8 ? (D + 16) / 2 : D + 8;  // in fp16 units
  __shared__ __align__(16) _Float16 ldsK[2][kStep][kKeyRow];
  __shared__ __align__(16) _Float16 ldsV[2][D][kStep + 8];
  __shared__ __align__(16) float ldsKS[2][kStep], ldsVS[2][kStep];

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, row = lane & 15u, kq = lane >> 4;
  const uint32_t h = blockIdx.x, split = blockIdx.y, z = blockIdx.z;
  const AttentionSequence seq = p.sequence[z];
  const uint32_t total = seq.committed + seq.rows;
  // The sequence's own splits: ceil(steps / steps_per_split) of them; later grid rows are empty.
  static_assert(kStep == int(ATTENTION_STEP_TOKENS) && ATTENTION_PAGE_TOKENS % ATTENTION_STEP_TOKENS == 0, "a page holds whole steps");
  const uint32_t span = uint32_t(seq.steps_per_split) * ATTENTION_STEP_TOKENS;
  const uint32_t first = min(total, split * span), last = min(total, (split + 1) * span);
  const uint32_t steps = first < last ? (last - first + kStep - 1) / kStep : 0;
  const float scale2 = kLog2e / sqrtf(float(D));

  // This wave's query rows as MFMA operands, their sums and their rows' visibility masks.
  constexpr int JQ = D / 64;  // INT8 products of 64 dimensions
  f16x8 q[I8 ? 1 : kTiles][I8 ? 1 : JD];
  i32x4 q8[I8 ? kTiles : 1][I8 ? JQ : 1];
  float qsum[kTiles];  // fp16 queries: the code offset's share of a score; INT8 queries: the row's scale
  bool owns[kTiles];
#pragma unroll
  for (int k = 0; k < kTiles; ++k) {
    const uint32_t g = wave + 4u * k;
    owns[k] = g < uint32_t(G);
    const size_t at = ((size_t(z) * p.kv_heads + h) * G + (owns[k] ? g : 0u)) * 16u + row;
    if constexpr (I8) {
      const int8_t *codes = reinterpret_cast<const int8_t *>(queries) + at * D;
#pragma unroll
      for (int j = 0; j < JQ; ++j) q8[k][j] = *reinterpret_cast<const i32x4 *>(codes + 64 * j + 16 * kq);
      qsum[k] = qsums[at];
    } else {
#pragma unroll
      for (int j = 0; j < JD; ++j) q[k][j] = *reinterpret_cast<const f16x8 *>(queries + at * D + 32 * j + 8 * kq);
      qsum[k] = -(qsums[at] * kCodeOffset);
    }
  }
  const uint32_t ancestors = row < seq.rows ? tree[seq.first_row + row].ancestors : 0u;

  float m[kTiles], l[kTiles];
  f32x4 o[kTiles][DT + 1];
#pragma unroll
  for (int k = 0; k < kTiles; ++k) {
    m[k] = -INFINITY;
    l[k] = 0.f;
#pragma unroll
    for (int dt = 0; dt <= DT; ++dt) o[k][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // A step's loads of this thread: kKeyVectors 16-byte vectors of keys, as many of values, a scale.
  uint4 keyLoad[kKeyVectors], valueLoad[kValueVectors];
  uint32_t scaleLoad = 0;
  // The page table is read one page ahead of the page loop, so that a step's loads never wait
  // for a table entry first (all of this is wave-uniform).
  const uint64_t *entries = page_table + seq.table_first;
  const uint32_t lastPage = total ? (total - 1u) / ATTENTION_PAGE_TOKENS : 0u;
  uint32_t heldPage = min(first / ATTENTION_PAGE_TOKENS, lastPage);
  uint64_t heldEntry = entries[heldPage], nextEntry = entries[min(heldPage + 1u, lastPage)];
  auto load = [&](uint32_t step) {
    const uint32_t token0 = first + step * kStep;
    if (token0 / ATTENTION_PAGE_TOKENS != heldPage) {
      heldPage = token0 / ATTENTION_PAGE_TOKENS;
      heldEntry = nextEntry;
      nextEntry = entries[min(heldPage + 1u, lastPage)];
    }
    uint8_t *page = pool + heldEntry * p.page_bytes;
    const uint32_t inPage = token0 % ATTENTION_PAGE_TOKENS;
    const uint4 *keys = reinterpret_cast<const uint4 *>(page + attention_key_index(h, inPage, 0, D));
    const uint4 *values = reinterpret_cast<const uint4 *>(page + attention_page_values_offset(p.kv_heads, D) +
                                                          attention_value_index(h, inPage, 0, D));
#pragma unroll
    for (int n = 0; n < kKeyVectors; ++n) keyLoad[n] = load_stream(keys + tid + 256u * n);
#pragma unroll
    for (int n = 0; n < kValueVectors; ++n) valueLoad[n] = load_stream(values + tid + 256u * n);
    if (tid < 2 * kStep) {
      const uint16_t *scales = reinterpret_cast<const uint16_t *>(
          page + (tid < kStep ? attention_page_key_scales_offset(p.kv_heads, D) : attention_page_value_scales_offset(p.kv_heads, D)));
      scaleLoad = scales[attention_scale_index(h, inPage + (tid & (kStep - 1)))];
    }
  };
  auto stage = [&](uint32_t buffer) {
#pragma unroll
    for (int n = 0; n < kKeyVectors; ++n) {
      const uint32_t v = tid + 256u * n, token = v / (D / 16), dq = v % (D / 16);
      if constexpr (I8) {
        *reinterpret_cast<uint4 *>(reinterpret_cast<int8_t *>(&ldsK[buffer][token][0]) + 16 * dq) = keyLoad[n];
      } else {
        const uint4 x = make_uint4(keyLoad[n].x ^ 0x80808080u, keyLoad[n].y ^ 0x80808080u, keyLoad[n].z ^ 0x80808080u,
                                   keyLoad[n].w ^ 0x80808080u);
        const uint2 a = bytes_to_f16(x.x), b = bytes_to_f16(x.y), c = bytes_to_f16(x.z), d = bytes_to_f16(x.w);
        uint4 *out = reinterpret_cast<uint4 *>(&ldsK[buffer][token][16 * dq]);
        out[0] = make_uint4(a.x, a.y, b.x, b.y);
        out[1] = make_uint4(c.x, c.y, d.x, d.y);
      }
    }
#pragma unroll
    for (int n = 0; n < kValueVectors; ++n) {
      // 16 tokens (tile tt of the step) of dimension d: token 4 kq' + i of the tile is operand
      // element 4 (tt % 2) + i of lane quarter kq' in token pair-block tt / 2.
      const uint32_t v = tid + 256u * n, d = v / 4u, tt = v % 4u;
      const uint32_t words[4] = {valueLoad[n].x ^ 0x80808080u, valueLoad[n].y ^ 0x80808080u, valueLoad[n].z ^ 0x80808080u,
                                 valueLoad[n].w ^ 0x80808080u};
#pragma unroll
      for (uint32_t quarter = 0; quarter < 4; ++quarter)
        *reinterpret_cast<uint2 *>(&ldsV[buffer][d][((tt >> 1) * 4u + quarter) * 8u + 4u * (tt & 1u)]) = bytes_to_f16(words[quarter]);
    }
    // Key scales carry the softmax scale (log2 domain), value scales the 2^10 of P.
    if (tid < 2 * kStep) (tid < kStep ? ldsKS[buffer] : ldsVS[buffer])[tid & (kStep - 1)] = half_bits_to_float(scaleLoad) * (tid < kStep ? scale2 : kPScale);
  };

  if (steps) {
    load(0);
    stage(0);
  }
  __syncthreads();
  const f16x8 ones = {_Float16(1.f), _Float16(1.f), _Float16(1.f), _Float16(1.f), _Float16(1.f), _Float16(1.f), _Float16(1.f), _Float16(1.f)};
  // One 64-token step. Masked steps (those that reach the block's own rows or the end of the
  // sequence) test every score's visibility; the steps before them, all of the history, do not.
  auto compute = [&](uint32_t buffer, uint32_t token0, auto maskedTag) {
    constexpr bool kMasked = decltype(maskedTag)::value;
    // Scores, transposed: tile tt holds tokens 16 tt + 4 kq + i of the step for fused row `row`.
    // The accumulator starts at -1152 sum(q), which takes the code offset out of the product.
    f32x4 s[kTiles][4];
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
      if constexpr (I8) {
        // the keys' bytes against the queries' codes, exact in int32; the row's scale follows with the key's
        i32x4 key[JQ];
        const int8_t *bytes = reinterpret_cast<const int8_t *>(&ldsK[buffer][16 * tt + row][0]);
#pragma unroll
        for (int j = 0; j < JQ; ++j) key[j] = *reinterpret_cast<const i32x4 *>(bytes + 64 * j + 16 * kq);
#pragma unroll
        for (int k = 0; k < kTiles; ++k) {
          i32x4 acc = {0, 0, 0, 0};
#pragma unroll
          for (int j = 0; j < JQ; ++j) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(key[j], q8[k][j], acc, 0, 0, 0);
#pragma unroll
          for (int i = 0; i < 4; ++i) s[k][tt][i] = float(acc[i]) * qsum[k];
        }
      } else {
        f16x8 key[JD];
#pragma unroll
        for (int j = 0; j < JD; ++j) key[j] = *reinterpret_cast<const f16x8 *>(&ldsK[buffer][16 * tt + row][32 * j + 8 * kq]);
#pragma unroll
        for (int k = 0; k < kTiles; ++k) {
          f32x4 acc = {qsum[k], qsum[k], qsum[k], qsum[k]};
#pragma unroll
          for (int j = 0; j < JD; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(key[j], q[k][j], acc, 0, 0, 0);
          s[k][tt] = acc;
        }
      }
    }
    f32x4 keyScale[4], valueScale[4];
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
      keyScale[tt] = *reinterpret_cast<const f32x4 *>(&ldsKS[buffer][16 * tt + 4 * kq]);
      valueScale[tt] = *reinterpret_cast<const f32x4 *>(&ldsVS[buffer][16 * tt + 4 * kq]);
    }
    f16x8 pOperand[kTiles][2];
#pragma unroll
    for (int k = 0; k < kTiles; ++k) {
      float stepMax = -INFINITY;
#pragma unroll
      for (int tt = 0; tt < 4; ++tt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float score = s[k][tt][i] * keyScale[tt][i];
          if constexpr (kMasked) {
            const uint32_t token = token0 + 16u * tt + 4u * kq + i;
            const bool visible = token < seq.committed || (token < total && ((ancestors >> (token - seq.committed)) & 1u));
            score = visible ? score : -INFINITY;
          }
          s[k][tt][i] = score;
          stepMax = fmaxf(stepMax, score);
        }
      stepMax = fmaxf(stepMax, __shfl_xor(stepMax, 16, 64));
      stepMax = fmaxf(stepMax, __shfl_xor(stepMax, 32, 64));
      const float newMax = fmaxf(m[k], stepMax), safeMax = newMax == -INFINITY ? 0.f : newMax;
      const float alpha = __builtin_amdgcn_exp2f(m[k] - safeMax);
      m[k] = newMax;
      float sum = 0.f;
      float folded[16];
#pragma unroll
      for (int tt = 0; tt < 4; ++tt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float pr = __builtin_amdgcn_exp2f(s[k][tt][i] - safeMax);
          sum += pr;
          const float f = pr * valueScale[tt][i];
          // A slot past the sequence's end may hold any scale: its weight is zero whatever it is.
          folded[4 * tt + i] = kMasked ? (pr > 0.f ? f : 0.f) : f;
        }
      l[k] = l[k] * alpha + sum;
      // rescale the running output only when some row's maximum grew (paged_attention_tile.h:450-458)
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {
#pragma unroll
        for (int dt = 0; dt <= DT; ++dt)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[k][dt][i] *= alpha;
      }
#pragma unroll
      for (int pair = 0; pair < 2; ++pair)
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          typedef __attribute__((ext_vector_type(2))) float f32x2;
          typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
          const f16x2 two = __builtin_convertvector(f32x2{folded[8 * pair + e], folded[8 * pair + e + 1]}, f16x2);
          pOperand[k][pair][e] = two[0];
          pOperand[k][pair][e + 1] = two[1];
        }
    }
    // Outputs, transposed: o[dt] holds dimensions 16 dt + 4 kq + i of fused row `row`.
#pragma unroll
    for (int pair = 0; pair < 2; ++pair) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const f16x8 value = *reinterpret_cast<const f16x8 *>(&ldsV[buffer][16 * dt + row][(pair * 4 + kq) * 8]);
#pragma unroll
        for (int k = 0; k < kTiles; ++k) o[k][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(value, pOperand[k][pair], o[k][dt], 0, 0, 0);
      }
#pragma unroll
      for (int k = 0; k < kTiles; ++k) o[k][DT] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, pOperand[k][pair], o[k][DT], 0, 0, 0);
    }
  };
  // Steps wholly inside the committed history come first, in a loop of their own.
  const uint32_t plain = first < seq.committed ? min(steps, (seq.committed - first) / kStep) : 0u;
  uint32_t step = 0;
  // A SIMD holds one wave of each of a compute unit's two workgroups and issues the older one's instructions first, so
  // the workgroup placed second runs every step behind the first and then finishes alone on an idle unit. The waves
  // take turns instead: a wave's priority is up on the steps whose parity is its wave slot's.
  const uint32_t slot = __builtin_amdgcn_s_getreg((3 << 11) | 4) & 1u;   // HW_ID's wave slot, bit 0
  auto takeTurn = [&](uint32_t s) {
    if ((s + slot) & 1u) __builtin_amdgcn_s_setprio(2);
    else __builtin_amdgcn_s_setprio(0);
  };
  for (; step < plain; ++step) {
    takeTurn(step);
    const uint32_t buffer = step & 1u;
    if (step + 1 < steps) load(step + 1);
    compute(buffer, first + step * kStep, std::false_type{});
    if (step + 1 < steps) stage(buffer ^ 1u);
    __syncthreads();
  }
  for (; step < steps; ++step) {
    takeTurn(step);
    const uint32_t buffer = step & 1u;
    if (step + 1 < steps) load(step + 1);
    compute(buffer, first + step * kStep, std::true_type{});
    if (step + 1 < steps) stage(buffer ^ 1u);
    __syncthreads();
  }

  // The split's partials: the code offset leaves with the row's sum of P, the 2^10 with a scale. The
  // outputs leave divided by the row's sum, a weighted mean of value rows whatever the split's
  // length, as fp16: a lane's 4 DT values are contiguous (position 4 DT kq + 4 dt + i of the row
  // holds dimension 16 dt + 4 kq + i), so a row's 2 D bytes go out as whole 16-byte stores.
#pragma unroll
  for (int k = 0; k < kTiles; ++k) {
    if (!owns[k]) continue;
    const uint32_t g = wave + 4u * k;
    float sum = l[k];
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    const size_t fused = ((size_t(z) * p.kv_heads + h) * p.splits + split) * (16u * G) + 16u * g + row;
    const float rowSum = o[k][DT][0] * kCodeOffset;
    const float norm = sum > 0.f ? 1.0f / (sum * kPScale) : 0.f;
    uint4 *mine = reinterpret_cast<uint4 *>(partialO + fused * D + 4u * DT * kq);
#pragma unroll
    for (int dt = 0; dt < DT; dt += 2) {
      f16x8 out;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        out[i] = _Float16((o[k][dt][i] - rowSum) * norm);
        out[4 + i] = _Float16((o[k][dt + 1][i] - rowSum) * norm);
      }
      mine[dt / 2] = __builtin_bit_cast(uint4, out);
    }
    if (kq == 0) {
      partialML[2 * fused] = m[k];
      partialML[2 * fused + 1] = sum;
    }
  }
}
SP_REGISTER_KERNEL("attention_q8_split_d128_g8", &attention_q8_split<128, 8, false>);
SP_REGISTER_KERNEL("attention_q8_split_d128_g4", &attention_q8_split<128, 4, false>);
SP_REGISTER_KERNEL("attention_q8_split_d64_g2", &attention_q8_split<64, 2, false>);
SP_REGISTER_KERNEL("attention_q8q_split_d128_g8", &attention_q8_split<128, 8, true>);
SP_REGISTER_KERNEL("attention_q8q_split_d128_g4", &attention_q8_split<128, 4, true>);
SP_REGISTER_KERNEL("attention_q8q_split_d64_g2", &attention_q8_split<64, 2, true>);

// ---------------------------------------------------------------------------------------------
// attention_reduce: grid (q_heads, 16, sequences), 256 threads. Merges the splits of one (head,
// row) in a fixed order (paged_attention_tile.h:499-535) and writes bf16 [packed row][q_heads * D].
// Thread (part, quad) sums splits part, part + P, ... of the row's positions 4 quad .. 4 quad + 3
// (four dimensions in a row, in the order the split kernel leaves them), all its loads in flight
// together; the P parts are then added in part order. A split weighs exp2(its maximum - the
// largest) times its sum: its outputs arrive divided by that sum.
// ---------------------------------------------------------------------------------------------
// The _t variant also writes the rows as the activation table (abi/Gguf.h) of the projection that
// follows, as gguf_prepare_table would from `out`; p.table_tiles is the table's row tiles. Rows of
// a tile past the packed rows keep what the table held.
template <int D, bool Table>
__global__ __launch_bounds__(256) void attention_reduce(const _Float16 *__restrict__ partialO, const float *__restrict__ partialML,
                                                        uint16_t *__restrict__ out, uint8_t *__restrict__ table,
                                                        const uint16_t *__restrict__ qkv, AttentionParams p) {
  constexpr uint32_t kQuads = D / 4, kParts = 256 / kQuads;
  __shared__ float weights[ATTENTION_MAXIMUM_SPLITS];
  __shared__ float scratch[4];
  __shared__ __align__(16) float4 sums[kParts][kQuads];
  __shared__ uint16_t staged[D];
  const uint32_t tid = threadIdx.x, head = blockIdx.x, row = blockIdx.y, z = blockIdx.z;
  const AttentionSequence seq = p.sequence[z];
  if (row >= seq.rows) return;
  const uint32_t group = p.q_heads / p.kv_heads, h = head / group, g = head % group, fusedRows = 16u * group;
  const size_t base = (size_t(z) * p.kv_heads + h) * p.splits;
  auto fusedOf = [&](uint32_t s) { return (base + s) * fusedRows + 16u * g + row; };

  // Split tid's maximum and sum; the block's maximum; the split's weight and its share of the denominator.
  float ms = -INFINITY, ls = 0.f;
  if (tid < p.splits) {
    const float2 ml = *reinterpret_cast<const float2 *>(partialML + 2 * fusedOf(tid));
    ms = ml.x;
    ls = ml.y;
  }
  const float maximum = block_max<256>(ms, scratch, tid);
  const float weight = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - maximum);
  if (tid < ATTENTION_MAXIMUM_SPLITS) weights[tid] = weight * ls;
  const float denominator = block_sum<256>(weight * ls, scratch, tid);  // block_sum's barriers publish the weights too

  const uint32_t part = tid / kQuads, quad = tid % kQuads;
  float4 total = make_float4(0.f, 0.f, 0.f, 0.f);
  typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
  for (uint32_t s0 = part; s0 < p.splits; s0 += 4u * kParts) {
    uint2 held[4];
#pragma unroll
    for (uint32_t i = 0; i < 4u; ++i) {
      const uint32_t s = s0 + i * kParts;
      held[i] = s < p.splits ? reinterpret_cast<const uint2 *>(partialO + fusedOf(s) * D)[quad] : make_uint2(0u, 0u);
    }
#pragma unroll
    for (uint32_t i = 0; i < 4u; ++i) {
      const uint32_t s = s0 + i * kParts;
      const float w = s < p.splits ? weights[s] : 0.f;
      if (w != 0.f) {  // a split without a visible token may hold anything
        const f16x4 x = __builtin_bit_cast(f16x4, held[i]);
        total.x += w * float(x[0]);
        total.y += w * float(x[1]);
        total.z += w * float(x[2]);
        total.w += w * float(x[3]);
      }
    }
  }
  // position quad of the row is dimensions 16 (quad % DT) + 4 (quad / DT) ..
  sums[part][4u * (quad % (D / 16u)) + quad / (D / 16u)] = total;
  __syncthreads();
  if (tid < D) {
    const float *flat = reinterpret_cast<const float *>(&sums[0][0]);
    float numerator = 0.f;
#pragma unroll
    for (uint32_t q = 0; q < kParts; ++q) numerator += flat[q * D + tid];
    const float value = denominator > 0.f ? numerator / denominator : 0.f;
    uint32_t bits = float_to_bf16_bits(value);
    if (p.gated) {
      // attention_gate.h:27-31: bf16(value) times the sigmoid of the head's gate in the row's packed projection.
      const float gate = bf16_bits_to_float(qkv[(size_t(seq.first_row) + row) * p.qkv_stride + head * 2u * D + D + tid]);
      bits = float_to_bf16_bits(bf16_bits_to_float(bits) * (1.0f / (1.0f + __builtin_amdgcn_exp2f(-kLog2e * gate))));
    }
    out[(size_t(seq.first_row) + row) * (p.q_heads * D) + head * D + tid] = uint16_t(bits);
    if constexpr (Table) staged[tid] = uint16_t(bits);
  }
  if constexpr (Table) {
    __syncthreads();
    if (tid < D / 4u) {
      // Run q: inputs 4 q .. 4 q + 3 of the packed row (norm_rms_table16 writes the same pieces).
      const uint32_t width = p.q_heads * D, G = width / 32u, q = head * (D / 4u) + tid;
      // Row tile packed / 16 is a tile of its 64-row piece's table, which holds `tiles` row tiles.
      const uint32_t packed = seq.first_row + row, r = packed % 16u;
      const uint32_t piece = packed / 16u / GGUF_PIECE_TILES, tile = packed / 16u % GGUF_PIECE_TILES;
      const uint32_t tiles = min(uint32_t(GGUF_PIECE_TILES), p.table_tiles - piece * GGUF_PIECE_TILES);
      uint8_t *mine = table + piece * gguf_table_bytes(width, GGUF_PIECE_TILES);
      const uint32_t x0 = staged[4 * tid], x1 = staged[4 * tid + 1], x2 = staged[4 * tid + 2], x3 = staged[4 * tid + 3];
      const uint32_t g = q / 8u, half = (q / 4u) % 2u, kq = q % 4u;
      reinterpret_cast<uint2 *>(mine)[((size_t(tile) * G + g) * 64u + kq * 16u + r) * 2u + half] = make_uint2(x0 | (x2 << 16), x1 | (x3 << 16));
      float s = (bf16_bits_to_float(x0) + bf16_bits_to_float(x1)) + (bf16_bits_to_float(x2) + bf16_bits_to_float(x3));
      const float s1 = __shfl_down(s, 1, 64), s2 = __shfl_down(s, 2, 64), s3 = __shfl_down(s, 3, 64);
      s = ((s + s1) + s2) + s3;
      const float other = __shfl_down(s, 4, 64);
      if (kq == 0) {
        float *sums32 = reinterpret_cast<float *>(mine + gguf_table_sums32_offset(width, tiles));
        float *sums16 = reinterpret_cast<float *>(mine + gguf_table_sums16_offset(width, tiles));
        sums16[(size_t(tile) * 2u * G + 2u * g + half) * 16u + r] = s;
        if (half == 0) sums32[(size_t(tile) * G + g) * 16u + r] = s + other;
      }
    }
  }
}
SP_REGISTER_KERNEL("attention_reduce_d128", &attention_reduce<128, false>);
SP_REGISTER_KERNEL("attention_reduce_d64", &attention_reduce<64, false>);
SP_REGISTER_KERNEL("attention_reduce_d128_t", &attention_reduce<128, true>);
SP_REGISTER_KERNEL("attention_reduce_d64_t", &attention_reduce<64, true>);

// ---------------------------------------------------------------------------------------------
// attention_q8_commit: grid (kv_heads, sequences, layers), D threads. retained[z] is the mask of the block
// rows on the accepted path; its k-th set bit (row r) moves from slot committed + r to committed + k.
// ---------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(D) void attention_q8_commit(const uint32_t *__restrict__ retained,
                                                         const uint64_t *__restrict__ page_table, uint8_t *__restrict__ pool,
                                                         AttentionCommitParams p) {
  const uint32_t tid = threadIdx.x, h = blockIdx.x, z = blockIdx.y;
  const AttentionSequence seq = p.sequence[z];
  pool += uint64_t(blockIdx.z) * p.layer_bytes;
  uint32_t mask = retained[z];
  uint32_t depth = 0;
  while (mask) {
    const uint32_t r = uint32_t(__builtin_ctz(mask));
    mask &= mask - 1u;
    if (r != depth && r < seq.rows) {
      const uint32_t from = seq.committed + r, to = seq.committed + depth;
      uint8_t *source = page_of(pool, page_table, seq, p.page_bytes, from / ATTENTION_PAGE_TOKENS);
      uint8_t *target = page_of(pool, page_table, seq, p.page_bytes, to / ATTENTION_PAGE_TOKENS);
      const uint32_t ft = from % ATTENTION_PAGE_TOKENS, tt = to % ATTENTION_PAGE_TOKENS;
      target[attention_key_index(h, tt, tid, D)] = source[attention_key_index(h, ft, tid, D)];
      const uint64_t values = attention_page_values_offset(p.kv_heads, D);
      target[values + attention_value_index(h, tt, tid, D)] = source[values + attention_value_index(h, ft, tid, D)];
      if (tid < 2) {
        const uint64_t scales = tid ? attention_page_value_scales_offset(p.kv_heads, D) : attention_page_key_scales_offset(p.kv_heads, D);
        reinterpret_cast<uint16_t *>(target + scales)[attention_scale_index(h, tt)] =
            reinterpret_cast<const uint16_t *>(source + scales)[attention_scale_index(h, ft)];
      }
    }
    ++depth;
    __syncthreads();
  }
}
SP_REGISTER_KERNEL("attention_q8_commit_d128", &attention_q8_commit<128>);
SP_REGISTER_KERNEL("attention_q8_commit_d64", &attention_q8_commit<64>);

} // namespace splash::kernels
