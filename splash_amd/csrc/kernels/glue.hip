// Glue kernels of the verify path: RMS norm (with the projection's activation table fused in),
// RoPE tables per packed row, token embedding from native K-quant rows (the reference's
// kernels/shared/normalization.metal, rope.metal, embedding.metal).
#include "abi/Glue.h"
#include "abi/Gguf.h"
#include "backend/KernelRegistry.hpp"
#include "kernels/device_common.hpp"

namespace splash::kernels {

// Rows of up to kStagedWidth columns are staged in LDS with every global load in flight at once
// (a row's columns are read twice, in an order no vector load gives directly).
constexpr uint32_t kStagedWidth = 8192;

// Copies `width` bf16 values (a multiple of 8, 16-byte aligned) to LDS; no barrier.
__device__ __forceinline__ void stage_row(const uint16_t *__restrict__ source, uint32_t width, uint16_t *lds) {
  const uint32_t vectors = width / 8u;
  uint4 held[kStagedWidth / 8u / 256u];
#pragma unroll
  for (uint32_t i = 0; i < kStagedWidth / 8u / 256u; ++i) {
    const uint32_t v = threadIdx.x + 256u * i;
    if (v < vectors) held[i] = reinterpret_cast<const uint4 *>(source)[v];
  }
#pragma unroll
  for (uint32_t i = 0; i < kStagedWidth / 8u / 256u; ++i) {
    const uint32_t v = threadIdx.x + 256u * i;
    if (v < vectors) reinterpret_cast<uint4 *>(lds)[v] = held[i];
  }
}

// The row's inverse RMS: 256 threads sum the squares of columns tid, tid + 256, ... in column
// order; a wavefront sums its lanes by butterfly, the four wavefronts' sums are added in order
// (normalization.metal:59-99 and common/rms_inverse.h:15-33, on 64-lane wavefronts).
__device__ __forceinline__ float rms_inverse(const uint16_t *row, uint32_t width, float *scratch) {
  float sum = 0.f;
  for (uint32_t c = threadIdx.x; c < width; c += 256) {
    const float v = bf16_bits_to_float(row[c]);
    sum += v * v;
  }
  sum = wave_sum(sum);
  if ((threadIdx.x & 63u) == 0) scratch[threadIdx.x >> 6] = sum;
  __syncthreads();
  const float total = ((scratch[0] + scratch[1]) + scratch[2]) + scratch[3];
  return 1.0f / sqrtf(total / float(width) + SPLASH_RMS_EPSILON);
}

__global__ __launch_bounds__(256) void norm_rms(const uint16_t *__restrict__ input, const uint16_t *__restrict__ weight,
                                                uint16_t *__restrict__ output, NormParams p) {
  __shared__ float scratch[4];
  __shared__ __align__(16) uint16_t rowX[kStagedWidth], rowW[kStagedWidth];
  const uint32_t row = blockIdx.x;
  const uint16_t *x = input + size_t(row) * p.width, *w = weight;
  if (p.width <= kStagedWidth && p.width % 8u == 0) {
    stage_row(x, p.width, rowX);
    stage_row(w, p.width, rowW);
    __syncthreads();
    x = rowX;
    w = rowW;
  }
  const float inverse = rms_inverse(x, p.width, scratch);
  for (uint32_t c = threadIdx.x; c < p.width; c += 256)
    output[size_t(row) * p.width + c] = uint16_t(float_to_bf16_bits((bf16_bits_to_float(x[c]) * inverse) * bf16_bits_to_float(w[c])));
}
SP_REGISTER_KERNEL("norm_rms", &norm_rms);

// The same, and the activation table of the normalized rows: grid (tiles * 16) so that the rows
// past the live ones are written as zeros. Each thread normalizes runs of four inputs
// (4 kq .. 4 kq + 3 of a group's half), which are one 8-byte piece of a table entry.
__global__ __launch_bounds__(256) void norm_rms_table16(const uint16_t *__restrict__ input, const uint16_t *__restrict__ weight,
                                                        uint16_t *__restrict__ output, uint8_t *__restrict__ table, NormParams p) {
  __shared__ float scratch[4];
  __shared__ __align__(16) uint16_t rowX[kStagedWidth], rowW[kStagedWidth];
  const uint32_t row = blockIdx.x, r = row % 16u, G = p.width / 32u;
  // Row tile row / 16 is tile `tile` of its piece's table, which holds `tiles` row tiles.
  const uint32_t piece = row / 16u / GGUF_PIECE_TILES, tile = row / 16u % GGUF_PIECE_TILES;
  const uint32_t tiles = min(uint32_t(GGUF_PIECE_TILES), p.tiles - piece * GGUF_PIECE_TILES);
  table += piece * gguf_table_bytes(p.width, GGUF_PIECE_TILES);
  const bool live = row < p.rows;
  const uint16_t *x = input + size_t(live ? row : 0) * p.width, *w = weight;
  if (live && p.width <= kStagedWidth) {  // the width is a multiple of 256
    stage_row(x, p.width, rowX);
    stage_row(w, p.width, rowW);
    __syncthreads();
    x = rowX;
    w = rowW;
  }
  const float inverse = live ? rms_inverse(x, p.width, scratch) : 0.f;
  uint2 *values = reinterpret_cast<uint2 *>(table);
  float *sums32 = reinterpret_cast<float *>(table + gguf_table_sums32_offset(p.width, tiles));
  float *sums16 = reinterpret_cast<float *>(table + gguf_table_sums16_offset(p.width, tiles));
  // run q covers inputs 4 q .. 4 q + 3: group g = q / 8, half = (q / 4) % 2, kq = q % 4
  for (uint32_t q = threadIdx.x; q < p.width / 4u; q += 256) {
    uint32_t bits[4] = {0, 0, 0, 0};
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (live) {
      const uint2 xs = *reinterpret_cast<const uint2 *>(x + 4u * q), ws = *reinterpret_cast<const uint2 *>(w + 4u * q);
      const uint32_t xb[4] = {xs.x & 0xFFFFu, xs.x >> 16, xs.y & 0xFFFFu, xs.y >> 16};
      const uint32_t wb[4] = {ws.x & 0xFFFFu, ws.x >> 16, ws.y & 0xFFFFu, ws.y >> 16};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        bits[i] = float_to_bf16_bits((bf16_bits_to_float(xb[i]) * inverse) * bf16_bits_to_float(wb[i]));
        v[i] = bf16_bits_to_float(bits[i]);
      }
      *reinterpret_cast<uint2 *>(output + size_t(row) * p.width + 4u * q) = make_uint2(bits[0] | (bits[1] << 16), bits[2] | (bits[3] << 16));
    }
    const uint32_t g = q / 8u, half = (q / 4u) % 2u, kq = q % 4u;
    // operand elements 4 half + {0,1,2,3} are inputs 4 kq + {0,2,1,3} of the half
    const uint2 piece = make_uint2(bits[0] | (bits[2] << 16), bits[1] | (bits[3] << 16));
    values[((size_t(tile) * G + g) * 64u + kq * 16u + r) * 2u + half] = piece;
    // sums of 16 inputs in input order: the four runs of a half sit in four consecutive lanes
    float s = (v[0] + v[1]) + (v[2] + v[3]);
    const float s1 = __shfl_down(s, 1, 64), s2 = __shfl_down(s, 2, 64), s3 = __shfl_down(s, 3, 64);
    s = ((s + s1) + s2) + s3;
    const float other = __shfl_down(s, 4, 64);
    if (kq == 0) {
      sums16[(size_t(tile) * 2u * G + 2u * g + half) * 16u + r] = s;
      if (half == 0) sums32[(size_t(tile) * G + g) * 16u + r] = s + other;
    }
  }
}
SP_REGISTER_KERNEL("norm_rms_table16", &norm_rms_table16);

// copy_rows_bf16: grid (ceil(rows * width / 256)), 256 threads.
__global__ __launch_bounds__(256) void copy_rows_bf16(const uint16_t *__restrict__ source, uint16_t *__restrict__ destination, RowCopyParams p) {
  const uint64_t index = uint64_t(blockIdx.x) * 256u + threadIdx.x;
  if (index >= uint64_t(p.rows) * p.width) return;
  const uint32_t row = uint32_t(index / p.width), column = uint32_t(index % p.width);
  destination[(size_t(p.to_row) + row) * p.to_stride + p.to_column + column] =
      source[(size_t(p.from_row) + row) * p.from_stride + p.from_column + column];
}
SP_REGISTER_KERNEL("copy_rows_bf16", &copy_rows_bf16);

__global__ __launch_bounds__(256) void swiglu_rows(const uint16_t *__restrict__ gate, const uint16_t *__restrict__ up,
                                                   uint16_t *__restrict__ output, SwiGluRowsParams p) {
  const uint64_t first = (uint64_t(blockIdx.x) * 256u + threadIdx.x) * 8u;
  if (first >= p.count) return;
  if (first + 8u <= p.count) {
    const uint4 g = *reinterpret_cast<const uint4 *>(gate + first), u = *reinterpret_cast<const uint4 *>(up + first);
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t out[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t low = float_to_bf16_bits(bf16_bits_to_float(uw[i] & 0xFFFFu) * silu(bf16_bits_to_float(gw[i] & 0xFFFFu)));
      const uint32_t high = float_to_bf16_bits(bf16_bits_to_float(uw[i] >> 16) * silu(bf16_bits_to_float(gw[i] >> 16)));
      out[i] = low | (high << 16);
    }
    *reinterpret_cast<uint4 *>(output + first) = make_uint4(out[0], out[1], out[2], out[3]);
  } else {
    for (uint64_t i = first; i < p.count; ++i)
      output[i] = uint16_t(float_to_bf16_bits(bf16_bits_to_float(up[i]) * silu(bf16_bits_to_float(gate[i]))));
  }
}
SP_REGISTER_KERNEL("swiglu_rows", &swiglu_rows);

__global__ void rope_build_tree_tables(const float *__restrict__ inverse_frequency, const uint32_t *__restrict__ depth,
                                       float *__restrict__ cosines, float *__restrict__ sines, RopeTreeParams p) {
  const uint32_t row = blockIdx.x, pair = threadIdx.x;
  if (row >= p.rows || pair >= p.pairs) return;
  uint32_t anchor = 0;
  for (uint32_t s = 0; s < p.sequences; ++s)
    if (row >= p.first_row[s] && row < p.first_row[s] + p.row_count[s]) anchor = p.anchor[s];
  const float angle = float(anchor + depth[row]) * inverse_frequency[pair];
  cosines[size_t(row) * p.pairs + pair] = cosf(angle);
  sines[size_t(row) * p.pairs + pair] = sinf(angle);
}
SP_REGISTER_KERNEL("rope_build_tree_tables", &rope_build_tree_tables);

// gguf_float_<weights>_<output>: the fp32 projection of weights kept as rows (abi/Glue.h; the reference's
// kernels/shared/gguf_float.metal): a workgroup owns 16 rows x 16 columns and walks K in steps of 64 inputs staged in
// LDS (the rows' bf16 values widened, the weights as stored or widened: every operand exact in fp32); thread (r, c)
// runs the four chains of its output. The weights' rows are padded by one word in LDS so that the sixteen columns a
// half-wave reads at one input fall in sixteen banks.
template <bool kBf16Weights, bool kBf16Output>
__global__ __launch_bounds__(256) void gguf_float(const uint16_t *__restrict__ input, const void *__restrict__ weights,
                                                   void *__restrict__ output, GgufFloatParams p) {
  constexpr uint32_t S = GGUF_FLOAT_STEP;
  __shared__ float xs[16][S], ws[16][S + 1];
  const uint32_t tid = threadIdx.x, c = tid & 15u, r = tid >> 4;
  const uint32_t column0 = blockIdx.x * 16u, row0 = blockIdx.y * 16u, K = p.input_size;
  float chain[4] = {0.f, 0.f, 0.f, 0.f};
  for (uint32_t k0 = 0; k0 < K; k0 += S) {
    // stage: thread t the four inputs 4 (t % 16) .. of row / column t / 16; zeros past the rows, the columns and K
    {
      const uint32_t line = tid >> 4, at = (tid & 15u) * 4u;
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) {
        const uint32_t k = k0 + at + i;
        const bool inside = k < K;
        float x = 0.f, w = 0.f;
        if (inside && row0 + line < p.rows) x = bf16_bits_to_float(input[size_t(row0 + line) * K + k]);
        if (inside && column0 + line < p.output_size) {
          if constexpr (kBf16Weights) w = bf16_bits_to_float(static_cast<const uint16_t *>(weights)[size_t(column0 + line) * K + k]);
          else w = static_cast<const float *>(weights)[size_t(column0 + line) * K + k];
        }
        xs[line][at + i] = x;
        ws[line][at + i] = w;
      }
    }
    __syncthreads();
#pragma unroll 4
    for (uint32_t k = 0; k < S; k += 4) {
#pragma unroll
      for (uint32_t j = 0; j < 4; ++j) chain[j] = __builtin_fmaf(xs[r][k + j], ws[c][k + j], chain[j]);
    }
    __syncthreads();
  }
  const float sum = (chain[0] + chain[1]) + (chain[2] + chain[3]);
  if (row0 + r >= p.rows || column0 + c >= p.output_size) return;
  const size_t at = size_t(row0 + r) * p.out_stride + p.out_offset + column0 + c;
  if constexpr (kBf16Output) static_cast<uint16_t *>(output)[at] = uint16_t(float_to_bf16_bits(sum));
  else static_cast<float *>(output)[at] = sum;
}
SP_REGISTER_KERNEL("gguf_float_f32_f32", (&gguf_float<false, false>));
SP_REGISTER_KERNEL("gguf_float_f32_bf16", (&gguf_float<false, true>));
SP_REGISTER_KERNEL("gguf_float_bf16_f32", (&gguf_float<true, false>));
SP_REGISTER_KERNEL("gguf_float_bf16_bf16", (&gguf_float<true, true>));

// gguf_embed_<fmt>: out[r][:] = bf16(decode(native row tokens[r])); a token at or past the
// vocabulary gives zeros (embedding.metal:10-18). Grid (rows, hidden / 256), 64 threads: a thread
// decodes four values of a super-block.
template <uint32_t FMT>
__global__ __launch_bounds__(64) void gguf_embed(const uint8_t *__restrict__ table, const uint32_t *__restrict__ tokens,
                                                 uint16_t *__restrict__ out, GgufEmbedParams p) {
  const uint32_t row = blockIdx.x, block = blockIdx.y, tid = threadIdx.x;
  const uint32_t token = tokens[row];
  uint16_t *o = out + size_t(row) * p.hidden + size_t(block) * 256u;
  if (token >= p.vocabulary) {
#pragma unroll
    for (int i = 0; i < 4; ++i) o[tid + 64 * i] = 0;
    return;
  }
  const uint32_t blocks = p.hidden / 256u;
  if constexpr (FMT == GGUF_FMT_Q4K || FMT == GGUF_FMT_Q5K) {
    constexpr bool kFifth = FMT == GGUF_FMT_Q5K;   // Q5_K: 32 bytes of fifth bits between the scales and the nibbles
    const uint8_t *blk = table + (size_t(token) * blocks + block) * (kFifth ? GGUF_Q5K_NATIVE : GGUF_Q4K_NATIVE);
    const float d = half_bits_to_float(blk[0] | (blk[1] << 8)), dmin = half_bits_to_float(blk[2] | (blk[3] << 8));
    const uint8_t *sc = blk + 4, *qh = blk + 16, *qs = blk + (kFifth ? 48 : 16);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t k = tid + 64u * i, j = k / 32u, e = k % 32u;
      uint32_t s, m;
      if (j < 4) { s = sc[j] & 63u; m = sc[j + 4] & 63u; }
      else { s = (sc[j + 4] & 0xFu) | ((sc[j - 4] >> 6) << 4); m = (sc[j + 4] >> 4) | ((sc[j] >> 6) << 4); }
      uint32_t code = (qs[32u * (j / 2u) + e] >> (4u * (j % 2u))) & 15u;
      if constexpr (kFifth) code |= ((qh[e] >> j) & 1u) << 4;
      o[k] = uint16_t(float_to_bf16_bits(__fmaf_rn(d * float(s), float(code), -(dmin * float(m)))));
    }
  } else if constexpr (FMT == GGUF_FMT_IQ4XS || FMT == GGUF_FMT_IQ4NL) {
    // value = scale * codebook[nibble]: byte e % 16 of the group's 16 holds inputs e (low nibble) and 16 + e (high)
    constexpr int kCodebook[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
    constexpr bool kXs = FMT == GGUF_FMT_IQ4XS;
    const uint8_t *blk = table + (size_t(token) * blocks + block) * (kXs ? GGUF_IQ4XS_NATIVE : GGUF_IQ4NL_NATIVE);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t k = tid + 64u * i, j = k / 32u, e = k % 32u;
      float scale;
      const uint8_t *qs;
      if constexpr (kXs) {
        const uint32_t high = blk[2] | (blk[3] << 8), ls = ((blk[4u + j / 2u] >> (4u * (j % 2u))) & 15u) | (((high >> (2u * j)) & 3u) << 4);
        scale = half_bits_to_float(blk[0] | (blk[1] << 8)) * float(int(ls) - 32);
        qs = blk + 8u + 16u * j;
      } else {
        scale = half_bits_to_float(blk[18u * j] | (blk[18u * j + 1u] << 8));
        qs = blk + 18u * j + 2u;
      }
      const uint32_t code = e < 16u ? qs[e] & 15u : qs[e - 16u] >> 4;
      o[k] = uint16_t(float_to_bf16_bits(scale * float(kCodebook[code])));
    }
  } else if constexpr (FMT == GGUF_FMT_Q80) {
    const uint8_t *blk = table + (size_t(token) * blocks + block) * GGUF_Q80_NATIVE;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t k = tid + 64u * i, j = k / 32u, e = k % 32u;
      const uint8_t *group = blk + 34u * j;
      const float d = half_bits_to_float(group[0] | (group[1] << 8));
      o[k] = uint16_t(float_to_bf16_bits(d * float(int(int8_t(group[2u + e])))));
    }
  } else {
    const uint8_t *blk = table + (size_t(token) * blocks + block) * GGUF_Q6K_NATIVE;
    const float d = half_bits_to_float(blk[208] | (blk[209] << 8));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t k = tid + 64u * i, n = k / 128u, r = (k % 128u) / 32u, e = k % 32u;
      const uint32_t l4 = (blk[64u * n + e + 32u * (r & 1u)] >> (4u * (r >> 1))) & 15u, h2 = (blk[128u + 32u * n + e] >> (2u * r)) & 3u;
      const int q = int(l4 | (h2 << 4)) - 32;
      const float scale = float(int(int8_t(blk[192u + 8u * n + 2u * r + e / 16u])));
      o[k] = uint16_t(float_to_bf16_bits(d * scale * float(q)));
    }
  }
}
SP_REGISTER_KERNEL("gguf_embed_q4k", &gguf_embed<GGUF_FMT_Q4K>);
SP_REGISTER_KERNEL("gguf_embed_q6k", &gguf_embed<GGUF_FMT_Q6K>);
SP_REGISTER_KERNEL("gguf_embed_q5k", &gguf_embed<GGUF_FMT_Q5K>);
SP_REGISTER_KERNEL("gguf_embed_q80", &gguf_embed<GGUF_FMT_Q80>);
SP_REGISTER_KERNEL("gguf_embed_iq4xs", &gguf_embed<GGUF_FMT_IQ4XS>);
SP_REGISTER_KERNEL("gguf_embed_iq4nl", &gguf_embed<GGUF_FMT_IQ4NL>);

} // namespace splash::kernels
