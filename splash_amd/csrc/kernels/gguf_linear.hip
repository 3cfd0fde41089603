// Q4_K / Q6_K dequant-GEMM for a verify block of 1..64 rows (the reference's decode tiles:
// kernels/shared/gguf_linear.metal, kernels/decode/linear_gguf_sgmatrix.metal), written for gfx950.
//
// The projection is weight streaming: every weight byte is read once from HBM with 128-bit loads
// of a re-tiled image (abi/Gguf.h), its codes become exact bf16 operands 128 + code in registers
// (two integer ops per register of two codes, no conversion), and one 16x16x32 bf16 MFMA per
// 32-input group multiplies them with the block's rows from the activation table. The group's
// fp32 scale closes the chain as acc = fma(dot, s, acc), the arithmetic of the reference's register
// tile (linear_gguf_sgmatrix.metal:140-151); the group's constant term sum(x) * (m - 128 s) is a
// K = 4 fp32 MFMA over four groups' row sums, which costs no vector ALU. Q6_K runs one 16x16x16
// MFMA per 16 inputs (one int8 scale each) and the term -160 s sum16(x) the same way.
//
// Work split: a wave owns GGUF_DECODE_UNIT_TILES column tiles over a K range; the `k_waves` waves of
// a workgroup that share tiles sum their ranges through LDS in wave order, and `splits` workgroups
// (grid.y) sum theirs through fp32 partials in split order, the last arriver applying the
// epilogue (the reference's split_reduce.h:28-54), so a result never depends on arrival order.
#include "abi/Gguf.h"
#include "backend/KernelRegistry.hpp"
#include "kernels/gguf_device.hpp"

namespace splash::kernels {

constexpr int kUnitTiles = 2;  // column tiles per wave
#define GGUF_DECODE_UNIT_TILES 2

// ---------------------------------------------------------------------------------------------
// gguf_prepare_table: bf16 rows -> the activation table (abi/Gguf.h).
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(64) void gguf_prepare_table(const uint16_t *__restrict__ input, uint8_t *__restrict__ table,
                                                         GgufPrepareParams p) {
  const uint32_t g = blockIdx.x, t = blockIdx.y, lane = threadIdx.x, r = lane & 15u, kq = lane >> 4;
  const uint32_t G = p.input_size / 32u, row = 16u * t + r;
  float v[8];
#pragma unroll
  for (uint32_t e = 0; e < 8; ++e) v[e] = 0.f;
  uint32_t bits[8] = {};
  if (row < p.rows) {
    const uint16_t *x = input + size_t(row) * p.row_stride + 32u * g;
#pragma unroll
    for (uint32_t e = 0; e < 8; ++e) {
      bits[e] = x[gguf_operand_input(kq, e)];
      v[e] = bf16_bits_to_float(bits[e]);
    }
  }
  uint4 packed;
  packed.x = bits[0] | (bits[1] << 16);
  packed.y = bits[2] | (bits[3] << 16);
  packed.z = bits[4] | (bits[5] << 16);
  packed.w = bits[6] | (bits[7] << 16);
  reinterpret_cast<uint4 *>(table)[(size_t(t) * G + g) * 64u + lane] = packed;
  // Sums of the 16 inputs of each half, in input order: lane kq holds inputs 4 kq + {0,2,1,3}.
  float half0 = (v[0] + v[2]) + (v[1] + v[3]);  // inputs 4kq, 4kq+1, 4kq+2, 4kq+3
  float half1 = (v[4] + v[6]) + (v[5] + v[7]);
  // across kq = 0..3 (lanes r, r + 16, r + 32, r + 48), in order
  float h0[4], h1[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    h0[q] = __shfl(half0, int(r) + 16 * q, 64);
    h1[q] = __shfl(half1, int(r) + 16 * q, 64);
  }
  const float s0 = ((h0[0] + h0[1]) + h0[2]) + h0[3], s1 = ((h1[0] + h1[1]) + h1[2]) + h1[3];
  if (kq == 0) {
    float *sums32 = reinterpret_cast<float *>(table + gguf_table_sums32_offset(p.input_size, p.tiles));
    float *sums16 = reinterpret_cast<float *>(table + gguf_table_sums16_offset(p.input_size, p.tiles));
    sums32[(size_t(t) * G + g) * 16u + r] = s0 + s1;
    sums16[(size_t(t) * 2u * G + 2u * g) * 16u + r] = s0;
    sums16[(size_t(t) * 2u * G + 2u * g + 1u) * 16u + r] = s1;
  }
}
SP_REGISTER_KERNEL("gguf_prepare_table", &gguf_prepare_table);

// ---------------------------------------------------------------------------------------------
// Records in registers.
// ---------------------------------------------------------------------------------------------
template <uint32_t FMT> struct Record;
template <> struct Record<GGUF_FMT_Q4K> {
  uint4 n0, n1, meta;
  __device__ __forceinline__ void load(const uint8_t *rec, uint32_t lane) {
    const uint4 *p = reinterpret_cast<const uint4 *>(rec);
    n0 = load_stream(p + lane);
    n1 = load_stream(p + 64 + lane);
    meta = load_stream(p + 128 + (lane & 15u));
  }
};
template <> struct Record<GGUF_FMT_Q6K> {
  uint4 n0, n1, high, scales;
  uint32_t d;
  __device__ __forceinline__ void load(const uint8_t *rec, uint32_t lane) {
    const uint4 *p = reinterpret_cast<const uint4 *>(rec);
    n0 = load_stream(p + lane);
    n1 = load_stream(p + 64 + lane);
    high = load_stream(p + 128 + lane);
    scales = load_stream(p + 192 + (lane & 15u));
    d = __builtin_nontemporal_load(reinterpret_cast<const uint16_t *>(rec + GGUF_Q6K_D) + (lane & 15u));
  }
};

// The eight groups' operand registers of a record, group g's in ops[g].
__device__ __forceinline__ void record_operands(const Record<GGUF_FMT_Q4K> &r, uint4 ops[8]) {
  ops[0] = q4_operands<false>(r.n0.x, r.n0.y);
  ops[1] = q4_operands<true>(r.n0.x, r.n0.y);
  ops[2] = q4_operands<false>(r.n0.z, r.n0.w);
  ops[3] = q4_operands<true>(r.n0.z, r.n0.w);
  ops[4] = q4_operands<false>(r.n1.x, r.n1.y);
  ops[5] = q4_operands<true>(r.n1.x, r.n1.y);
  ops[6] = q4_operands<false>(r.n1.z, r.n1.w);
  ops[7] = q4_operands<true>(r.n1.z, r.n1.w);
}
__device__ __forceinline__ void record_operands(const Record<GGUF_FMT_Q6K> &r, uint4 ops[8]) {
  ops[0] = q6_operands<false, 0>(r.n0.x, r.n0.y, r.high.x);
  ops[1] = q6_operands<true, 4>(r.n0.x, r.n0.y, r.high.x);
  ops[2] = q6_operands<false, 0>(r.n0.z, r.n0.w, r.high.y);
  ops[3] = q6_operands<true, 4>(r.n0.z, r.n0.w, r.high.y);
  ops[4] = q6_operands<false, 0>(r.n1.x, r.n1.y, r.high.z);
  ops[5] = q6_operands<true, 4>(r.n1.x, r.n1.y, r.high.z);
  ops[6] = q6_operands<false, 0>(r.n1.z, r.n1.w, r.high.w);
  ops[7] = q6_operands<true, 4>(r.n1.z, r.n1.w, r.high.w);
}

__device__ __forceinline__ float q6_scale(const uint4 &scales, uint32_t index) {
  const uint32_t word = index < 4 ? scales.x : index < 8 ? scales.y : index < 12 ? scales.z : scales.w;
  return float(int(int8_t((word >> (8u * (index & 3u))) & 0xFFu)));
}

// ---------------------------------------------------------------------------------------------
// gguf_dequant_<fmt>: fp32 values of the image. One wave per record.
// ---------------------------------------------------------------------------------------------
template <uint32_t FMT> __global__ __launch_bounds__(64) void gguf_dequant(const uint8_t *__restrict__ image,
                                                                          float *__restrict__ out, GgufDequantParams p) {
  const uint32_t b = blockIdx.x, tile = blockIdx.y, lane = threadIdx.x, c = lane & 15u, kq = lane >> 4;
  const uint32_t blocks = p.input_size / GGUF_BLOCK;
  Record<FMT> rec;
  rec.load(image + (size_t(tile) * blocks + b) * gguf_record_bytes(FMT), lane);
  uint4 ops[8];
  record_operands(rec, ops);
  float *row = out + size_t(16u * tile + c) * p.input_size + size_t(b) * GGUF_BLOCK;
  if constexpr (FMT == GGUF_FMT_Q4K) {
    const Q4KScales sc = q4k_scales(rec.meta);
#pragma unroll
    for (uint32_t g = 0; g < 8; ++g) {
      const float s = sc.d * byte_of(g < 4 ? sc.sc_lo : sc.sc_hi, g & 3u);
      const float m = -(sc.dmin * byte_of(g < 4 ? sc.mn_lo : sc.mn_hi, g & 3u));
      const uint32_t regs[4] = {ops[g].x, ops[g].y, ops[g].z, ops[g].w};
#pragma unroll
      for (uint32_t e = 0; e < 8; ++e) {
        const float code = float(operand_code(regs[e >> 1], e & 1u) & 0xFu);
        // d*sc*code is exact in fp32, so this is the one rounding of d*sc*code - dmin*mn.
        row[32u * g + gguf_operand_input(kq, e)] = __fmaf_rn(s, code, m);
      }
    }
  } else {
    const float d = half_bits_to_float(rec.d);
#pragma unroll
    for (uint32_t g = 0; g < 8; ++g) {
      const uint32_t regs[4] = {ops[g].x, ops[g].y, ops[g].z, ops[g].w};
#pragma unroll
      for (uint32_t e = 0; e < 8; ++e) {
        const float s = d * q6_scale(rec.scales, 2u * g + (e >> 2));
        const int q = int(operand_code(regs[e >> 1], e & 1u) & 0x3Fu) - 32;
        row[32u * g + gguf_operand_input(kq, e)] = s * float(q);  // exact: 11 + 7 + 6 bits
      }
    }
  }
}
SP_REGISTER_KERNEL("gguf_dequant_q4k", &gguf_dequant<GGUF_FMT_Q4K>);
SP_REGISTER_KERNEL("gguf_dequant_q6k", &gguf_dequant<GGUF_FMT_Q6K>);

// ---------------------------------------------------------------------------------------------
// The decode projection.
// ---------------------------------------------------------------------------------------------
struct TileRef {
  const uint8_t *image;  // the tile's first record; null for a tile past the dispatch's last
  uint32_t column;       // its first destination column
};

// Tile `index` of the dispatch's concatenated segments.
__device__ __forceinline__ TileRef find_tile(uint32_t index, const uint8_t *const seg[3], const GgufDecodeParams &p,
                                             uint32_t record_bytes) {
  const uint32_t blocks = p.input_size / GGUF_BLOCK;
  TileRef ref{nullptr, 0};
  uint32_t rest = index;
  bool found = false;
#pragma unroll
  for (int s = 0; s < 3; ++s) {
    const uint32_t tiles = p.cols[s] / GGUF_TILE_COLUMNS;
    if (!found && rest < tiles) {
      ref.image = seg[s] + size_t(rest) * blocks * record_bytes;
      ref.column = p.offset[s] + rest * GGUF_TILE_COLUMNS;
      found = true;
    }
    rest -= found ? 0u : tiles;
  }
  return ref;
}

template <uint32_t FMT, int RT>
__device__ __forceinline__ void accumulate_record(const Record<FMT> &rec, const uint4 (&a)[RT][8], const float (&sums)[RT][4],
                                                  f32x4 (&acc)[RT], uint32_t kq) {
  uint4 ops[8];
  record_operands(rec, ops);
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  if constexpr (FMT == GGUF_FMT_Q4K) {
    const Q4KScales sc = q4k_scales(rec.meta);
    float s[8];
#pragma unroll
    for (uint32_t g = 0; g < 8; ++g) s[g] = sc.d * byte_of(g < 4 ? sc.sc_lo : sc.sc_hi, g & 3u);
    // Constant terms of groups kq and 4 + kq: m - 128 s.
    const float s_lo = sc.d * byte_of(sc.sc_lo, kq), s_hi = sc.d * byte_of(sc.sc_hi, kq);
    const float c_lo = __fmaf_rn(-128.f, s_lo, -(sc.dmin * byte_of(sc.mn_lo, kq)));
    const float c_hi = __fmaf_rn(-128.f, s_hi, -(sc.dmin * byte_of(sc.mn_hi, kq)));
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[t][0], c_lo, acc[t], 0, 0, 0);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[t][1], c_hi, acc[t], 0, 0, 0);
    }
#pragma unroll
    for (uint32_t g = 0; g < 8; ++g) {
      const bf16x8 b = as_bf16x8(ops[g]);
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        const f32x4 dot = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a[t][g]), b, zero, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[t][i] = __fmaf_rn(dot[i], s[g], acc[t][i]);
      }
    }
  } else {
    const float d = half_bits_to_float(rec.d);
    // Constant terms of 16-input blocks 4 j + kq: -160 d sc (operand 128 + q, value q - 32).
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
      const uint32_t word = j == 0 ? rec.scales.x : j == 1 ? rec.scales.y : j == 2 ? rec.scales.z : rec.scales.w;
      const float coef = -160.f * (d * float(int(int8_t((word >> (8u * kq)) & 0xFFu))));
#pragma unroll
      for (int t = 0; t < RT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[t][j], coef, acc[t], 0, 0, 0);
    }
#pragma unroll
    for (uint32_t g = 0; g < 8; ++g) {
#pragma unroll
      for (uint32_t h = 0; h < 2; ++h) {
        const float s = d * q6_scale(rec.scales, 2u * g + h);
        const uint2 bw = h ? make_uint2(ops[g].z, ops[g].w) : make_uint2(ops[g].x, ops[g].y);
        const s16x4 b = __builtin_bit_cast(s16x4, bw);
#pragma unroll
        for (int t = 0; t < RT; ++t) {
          const uint2 aw = h ? make_uint2(a[t][g].z, a[t][g].w) : make_uint2(a[t][g].x, a[t][g].y);
          const f32x4 dot = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, aw), b, zero, 0, 0, 0);
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[t][i] = __fmaf_rn(dot[i], s, acc[t][i]);
        }
      }
    }
  }
}

template <uint32_t FMT, int RT, uint32_t EP>
__global__ __launch_bounds__(256) void gguf_decode(const uint8_t *__restrict__ seg0, const uint8_t *__restrict__ seg1,
                                                   const uint8_t *__restrict__ seg2, const uint8_t *__restrict__ table,
                                                   void *__restrict__ out, const uint16_t *__restrict__ residual,
                                                   float *__restrict__ partials, uint32_t *__restrict__ counters,
                                                   GgufDecodeParams p) {
  constexpr uint32_t kRecord = FMT == GGUF_FMT_Q4K ? GGUF_Q4K_RECORD : GGUF_Q6K_RECORD;
  constexpr uint32_t kSumsPerBlock = FMT == GGUF_FMT_Q4K ? 2 : 4;  // K = 4 MFMAs of row sums per super-block
  __shared__ float reduce[3][kUnitTiles][RT][4][64];
  __shared__ uint32_t arrived;

  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, c = lane & 15u, kq = lane >> 4;
  const uint32_t kw = p.k_waves, ks = wave % kw, across = 4u / kw;
  const uint32_t unit = blockIdx.x * across + wave / kw;
  const uint32_t split = blockIdx.y;
  const uint32_t blocks = p.input_size / GGUF_BLOCK, G = p.input_size / 32u;
  const uint32_t tiles = gguf_row_tiles(p.rows);
  const uint8_t *const seg[3] = {seg0, seg1, seg2};

  TileRef tile[kUnitTiles];
  if (unit < p.units) {
    if constexpr (EP == GGUF_EPILOGUE_GATE_UP) {
      tile[0] = {seg0 + size_t(unit) * blocks * kRecord, p.offset[0] + unit * GGUF_TILE_COLUMNS};
      tile[1] = {seg1 + size_t(unit) * blocks * kRecord, p.offset[0] + unit * GGUF_TILE_COLUMNS};
    } else {
#pragma unroll
      for (int i = 0; i < kUnitTiles; ++i) tile[i] = find_tile(unit * kUnitTiles + i, seg, p, kRecord);
    }
  } else {
#pragma unroll
    for (int i = 0; i < kUnitTiles; ++i) tile[i] = {nullptr, 0};
  }

  // This wave's super-blocks: part ks of its workgroup's part `split`.
  const uint32_t parts = p.splits * kw, part = split * kw + ks;
  const uint32_t b0 = uint32_t(uint64_t(blocks) * part / parts), b1 = uint32_t(uint64_t(blocks) * (part + 1) / parts);

  f32x4 acc[kUnitTiles][RT];
#pragma unroll
  for (int i = 0; i < kUnitTiles; ++i)
#pragma unroll
    for (int t = 0; t < RT; ++t) acc[i][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  const uint4 *values = reinterpret_cast<const uint4 *>(table);
  const float *sumsBase = reinterpret_cast<const float *>(
      table + (FMT == GGUF_FMT_Q4K ? gguf_table_sums32_offset(p.input_size, tiles) : gguf_table_sums16_offset(p.input_size, tiles)));
  const uint32_t sumGroups = FMT == GGUF_FMT_Q4K ? G : 2u * G;  // row-sum entries per row tile

  if (tile[0].image && b0 < b1) {
    Record<FMT> cur[kUnitTiles], next[kUnitTiles];
#pragma unroll
    for (int i = 0; i < kUnitTiles; ++i)
      if (tile[i].image) cur[i].load(tile[i].image + size_t(b0) * kRecord, lane);
    for (uint32_t b = b0; b < b1; ++b) {
      // Activations of this super-block first, then the next one's weights: the loads return in
      // order, so the weights may stay in flight while the MFMAs wait for the activations only.
      uint4 a[RT][8];
      float sums[RT][4];
#pragma unroll
      for (int t = 0; t < RT; ++t) {
#pragma unroll
        for (uint32_t g = 0; g < 8; ++g) a[t][g] = values[(size_t(t) * G + 8u * b + g) * 64u + lane];
#pragma unroll
        for (uint32_t j = 0; j < kSumsPerBlock; ++j)
          sums[t][j] = sumsBase[(size_t(t) * sumGroups + kSumsPerBlock * 4u * b + 4u * j + kq) * 16u + c];
      }
      if (b + 1 < b1) {
#pragma unroll
        for (int i = 0; i < kUnitTiles; ++i)
          if (tile[i].image) next[i].load(tile[i].image + size_t(b + 1) * kRecord, lane);
      }
#pragma unroll
      for (int i = 0; i < kUnitTiles; ++i)
        if (tile[i].image) accumulate_record<FMT, RT>(cur[i], a, sums, acc[i], kq);
#pragma unroll
      for (int i = 0; i < kUnitTiles; ++i) cur[i] = next[i];
    }
  }

  // Waves that share tiles: wave ks = 0 adds the others' sums in wave order.
  if (kw > 1) {
    if (ks > 0) {
#pragma unroll
      for (int i = 0; i < kUnitTiles; ++i)
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
          for (int v = 0; v < 4; ++v) reduce[wave - 1][i][t][v][lane] = acc[i][t][v];
    }
    __syncthreads();
    if (ks == 0) {
      for (uint32_t other = 1; other < kw; ++other)
#pragma unroll
        for (int i = 0; i < kUnitTiles; ++i)
#pragma unroll
          for (int t = 0; t < RT; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[i][t][v] += reduce[wave + other - 1][i][t][v][lane];
    }
  }

  // Element (i, t, v) of this lane is row 16 t + 4 kq + v, column tile[i].column + c.
  const uint32_t paddedRows = tiles * GGUF_ROW_TILE;
  bool finish = ks == 0 && tile[0].image;
  if (p.splits > 1) {
    if (finish) {
#pragma unroll
      for (int i = 0; i < kUnitTiles; ++i) {
        if (!tile[i].image) continue;
        const uint32_t column = (EP == GGUF_EPILOGUE_GATE_UP ? uint32_t(i) * p.out_stride : 0u) + tile[i].column + c;
        const uint32_t width = EP == GGUF_EPILOGUE_GATE_UP ? 2u * p.out_stride : p.out_stride;
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
          for (int v = 0; v < 4; ++v)
            partials[(size_t(split) * paddedRows + 16u * t + 4u * kq + v) * width + column] = acc[i][t][v];
      }
    }
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) arrived = atomicAdd(&counters[blockIdx.x], 1u);
    __syncthreads();
    if (arrived != p.splits - 1) return;
    __threadfence();
    if (finish) {
#pragma unroll
      for (int i = 0; i < kUnitTiles; ++i) {
        if (!tile[i].image) continue;
        const uint32_t column = (EP == GGUF_EPILOGUE_GATE_UP ? uint32_t(i) * p.out_stride : 0u) + tile[i].column + c;
        const uint32_t width = EP == GGUF_EPILOGUE_GATE_UP ? 2u * p.out_stride : p.out_stride;
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            float sum = 0.f;
            for (uint32_t s = 0; s < p.splits; ++s)
              sum += partials[(size_t(s) * paddedRows + 16u * t + 4u * kq + v) * width + column];
            acc[i][t][v] = sum;
          }
      }
    }
    if (threadIdx.x == 0) counters[blockIdx.x] = 0;
  }
  if (!finish) return;

  if constexpr (EP == GGUF_EPILOGUE_GATE_UP) {
    uint16_t *o = static_cast<uint16_t *>(out);
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const uint32_t row = 16u * t + 4u * kq + v;
        if (row >= p.rows) continue;
        const float gate = round_bf16(acc[0][t][v]), up = round_bf16(acc[1][t][v]);
        o[size_t(row) * p.out_stride + tile[0].column + c] = uint16_t(float_to_bf16_bits(up * silu(gate)));
      }
  } else {
#pragma unroll
    for (int i = 0; i < kUnitTiles; ++i) {
      if (!tile[i].image) continue;
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const uint32_t row = 16u * t + 4u * kq + v;
          if (row >= p.rows) continue;
          const size_t at = size_t(row) * p.out_stride + tile[i].column + c;
          if constexpr (EP == GGUF_EPILOGUE_PLAIN_F32) static_cast<float *>(out)[at] = acc[i][t][v];
          else if constexpr (EP == GGUF_EPILOGUE_RESIDUAL)
            static_cast<uint16_t *>(out)[at] = uint16_t(float_to_bf16_bits(acc[i][t][v] + bf16_bits_to_float(residual[at])));
          else static_cast<uint16_t *>(out)[at] = uint16_t(float_to_bf16_bits(acc[i][t][v]));
        }
    }
  }
}

#define SP_GGUF_DECODE(fmt, FMT, rows, RT)                                                              \
  SP_REGISTER_KERNEL("gguf_decode_" fmt "_m" #rows "_a", &gguf_decode<FMT, RT, GGUF_EPILOGUE_PLAIN>);   \
  SP_REGISTER_KERNEL("gguf_decode_" fmt "_m" #rows "_a_f32", &gguf_decode<FMT, RT, GGUF_EPILOGUE_PLAIN_F32>); \
  SP_REGISTER_KERNEL("gguf_decode_" fmt "_m" #rows "_r", &gguf_decode<FMT, RT, GGUF_EPILOGUE_RESIDUAL>); \
  SP_REGISTER_KERNEL("gguf_decode_" fmt "_m" #rows "_g", &gguf_decode<FMT, RT, GGUF_EPILOGUE_GATE_UP>)
SP_GGUF_DECODE("q4k", GGUF_FMT_Q4K, 16, 1);
SP_GGUF_DECODE("q4k", GGUF_FMT_Q4K, 32, 2);
SP_GGUF_DECODE("q4k", GGUF_FMT_Q4K, 64, 4);
SP_GGUF_DECODE("q6k", GGUF_FMT_Q6K, 16, 1);
SP_GGUF_DECODE("q6k", GGUF_FMT_Q6K, 32, 2);
SP_GGUF_DECODE("q6k", GGUF_FMT_Q6K, 64, 4);

} // namespace splash::kernels
