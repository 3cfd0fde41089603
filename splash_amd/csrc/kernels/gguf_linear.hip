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
// A wave's cursors into one column tile's record stream: its lane's 16 bytes of each 1024-byte
// part, and its column's scale fields. They advance one record per super-block.
template <uint32_t FMT> struct Cursor {
  const uint4 *mine = nullptr;
  const uint4 *column = nullptr;
  const uint16_t *d = nullptr;  // Q6_K only
  __device__ __forceinline__ void open(const uint8_t *record, uint32_t lane) {
    const uint4 *p = reinterpret_cast<const uint4 *>(record);
    mine = p + lane;
    if constexpr (FMT == GGUF_FMT_Q4K) {
      column = p + 128 + (lane & 15u);
    } else {
      column = p + 192 + (lane & 15u);
      d = reinterpret_cast<const uint16_t *>(record + GGUF_Q6K_D) + (lane & 15u);
    }
  }
  __device__ __forceinline__ void advance() {
    constexpr uint32_t kVectors = (FMT == GGUF_FMT_Q4K ? GGUF_Q4K_RECORD : GGUF_Q6K_RECORD) / 16u;
    mine += kVectors;
    column += kVectors;
    if constexpr (FMT == GGUF_FMT_Q6K) d += kVectors * 8u;
  }
};

template <uint32_t FMT> struct Record;
template <> struct Record<GGUF_FMT_Q4K> {
  uint4 n0, n1, meta;
  __device__ __forceinline__ void load(const Cursor<GGUF_FMT_Q4K> &at) {
    n0 = load_stream(at.mine);
    n1 = load_stream(at.mine + 64);
    meta = load_stream(at.column);
  }
};
template <> struct Record<GGUF_FMT_Q6K> {
  uint4 n0, n1, high, scales;
  uint32_t d;
  __device__ __forceinline__ void load(const Cursor<GGUF_FMT_Q6K> &at) {
    n0 = load_stream(at.mine);
    n1 = load_stream(at.mine + 64);
    high = load_stream(at.mine + 128);
    scales = load_stream(at.column);
    d = __builtin_nontemporal_load(at.d);
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
  Cursor<FMT> cursor;
  cursor.open(image + (size_t(tile) * blocks + b) * gguf_record_bytes(FMT), lane);
  rec.load(cursor);
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

// One record's contribution to a wave's sums. `a` and `sums` are the workgroup's staged
// activations of the record's super-block in LDS: a[t][g][lane] the MFMA operand of row tile t,
// group g; sums[t][j][lane] the row sums of the j-th K = 4 MFMA.
template <uint32_t FMT, int RT>
__device__ __forceinline__ void accumulate_record(const Record<FMT> &rec, const uint4 (*a)[8][64], const float (*sums)[4][64],
                                                  f32x4 (&acc)[RT], uint32_t lane, uint32_t kq, float keep) {
  uint4 ops[8];
  record_operands(rec, ops);
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  if constexpr (FMT == GGUF_FMT_Q4K) {
    Q4KScales sc = q4k_scales(rec.meta);
    sc.d *= keep;
    sc.dmin *= keep;
    float s[8];
#pragma unroll
    for (uint32_t g = 0; g < 8; ++g) s[g] = sc.d * byte_of(g < 4 ? sc.sc_lo : sc.sc_hi, g & 3u);
    // Constant terms of groups kq and 4 + kq: m - 128 s.
    const float s_lo = sc.d * byte_of(sc.sc_lo, kq), s_hi = sc.d * byte_of(sc.sc_hi, kq);
    const float c_lo = __fmaf_rn(-128.f, s_lo, -(sc.dmin * byte_of(sc.mn_lo, kq)));
    const float c_hi = __fmaf_rn(-128.f, s_hi, -(sc.dmin * byte_of(sc.mn_hi, kq)));
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[t][0][lane], c_lo, acc[t], 0, 0, 0);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[t][1][lane], c_hi, acc[t], 0, 0, 0);
    }
#pragma unroll
    for (uint32_t g = 0; g < 8; ++g) {
      const bf16x8 b = as_bf16x8(ops[g]);
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        const f32x4 dot = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a[t][g][lane]), b, zero, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[t][i] = __fmaf_rn(dot[i], s[g], acc[t][i]);
      }
    }
  } else {
    const float d = half_bits_to_float(rec.d) * keep;
    // Constant terms of 16-input blocks 4 j + kq: -160 d sc (operand 128 + q, value q - 32).
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
      const uint32_t word = j == 0 ? rec.scales.x : j == 1 ? rec.scales.y : j == 2 ? rec.scales.z : rec.scales.w;
      const float coef = -160.f * (d * float(int(int8_t((word >> (8u * kq)) & 0xFFu))));
#pragma unroll
      for (int t = 0; t < RT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[t][j][lane], coef, acc[t], 0, 0, 0);
    }
#pragma unroll
    for (uint32_t g = 0; g < 8; ++g) {
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        const uint4 av = a[t][g][lane];
#pragma unroll
        for (uint32_t h = 0; h < 2; ++h) {
          const float s = d * q6_scale(rec.scales, 2u * g + h);
          const uint2 bw = h ? make_uint2(ops[g].z, ops[g].w) : make_uint2(ops[g].x, ops[g].y);
          const uint2 aw = h ? make_uint2(av.z, av.w) : make_uint2(av.x, av.y);
          const f32x4 dot = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, aw),
                                                                      __builtin_bit_cast(s16x4, bw), zero, 0, 0, 0);
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
  // The workgroup's four waves walk one K range in step and own different column tiles; the
  // range's activations pass through LDS one super-block at a time (two buffers, one barrier per
  // super-block), each wave fetching a quarter of them, so a wave's vector-memory queue holds
  // almost only weights and the MFMA operands arrive on the LDS counter instead.
  __shared__ uint4 ldsA[2][RT][8][64];
  __shared__ float ldsSums[2][RT][4][64];
  __shared__ uint32_t arrived;

  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, c = lane & 15u, kq = lane >> 4;
  const uint32_t unit = blockIdx.x * 4u + wave;
  const uint32_t split = blockIdx.y;
  const uint32_t blocks = p.input_size / GGUF_BLOCK, G = p.input_size / 32u;
  const uint32_t tiles = gguf_row_tiles(p.rows);
  const uint8_t *const seg[3] = {seg0, seg1, seg2};
  const uint32_t ks = 0;

  // Every wave streams real records, so the main loop has no divergent control flow: a wave past
  // the dispatch's last unit, or a tile past its last tile, re-reads the first tile and stores nothing.
  TileRef tile[kUnitTiles];
  bool live[kUnitTiles];
  {
    const uint32_t mine = unit < p.units ? unit : 0u;
    if constexpr (EP == GGUF_EPILOGUE_GATE_UP) {
      tile[0] = {seg0 + size_t(mine) * blocks * kRecord, p.offset[0] + mine * GGUF_TILE_COLUMNS};
      tile[1] = {seg1 + size_t(mine) * blocks * kRecord, p.offset[0] + mine * GGUF_TILE_COLUMNS};
      live[0] = live[1] = unit < p.units;
    } else {
#pragma unroll
      for (int i = 0; i < kUnitTiles; ++i) {
        tile[i] = find_tile(mine * kUnitTiles + i, seg, p, kRecord);
        live[i] = unit < p.units && tile[i].image != nullptr;
        if (!tile[i].image) tile[i] = {seg0, p.offset[0]};
      }
    }
  }

  // The workgroup's super-blocks: part `split` of K.
  const uint32_t b0 = uint32_t(uint64_t(blocks) * split / p.splits), b1 = uint32_t(uint64_t(blocks) * (split + 1) / p.splits);

  f32x4 acc[kUnitTiles][RT];
#pragma unroll
  for (int i = 0; i < kUnitTiles; ++i)
#pragma unroll
    for (int t = 0; t < RT; ++t) acc[i][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  const uint4 *values = reinterpret_cast<const uint4 *>(table);
  const float *sumsBase = reinterpret_cast<const float *>(
      table + (FMT == GGUF_FMT_Q4K ? gguf_table_sums32_offset(p.input_size, tiles) : gguf_table_sums16_offset(p.input_size, tiles)));
  const uint32_t sumGroups = FMT == GGUF_FMT_Q4K ? G : 2u * G;  // row-sum entries per row tile

  {
    // A software pipeline of kStages super-blocks in registers: the loads of super-block
    // b + kStages - 1 are issued before the MFMAs of super-block b, so kStages - 1 super-blocks of
    // weights per wave stay in flight (loads return in issue order, so waiting for b's never
    // waits for a later one's). The loop body is one straight block: the range is walked in
    // rounds of kStages, loads past its end re-read its last super-block (the cursors stop
    // there) and the super-blocks past its end are multiplied by a zero scale.
    constexpr int kStages = RT > 1 ? 2 : FMT == GGUF_FMT_Q4K ? 4 : 3;
    constexpr uint32_t kSumFloats = RT * kSumsPerBlock * 64u;  // staged row sums per super-block
    constexpr int kSumShare = (kSumFloats + 255u) / 256u;
    struct Stage {
      Record<FMT> rec[kUnitTiles];
      uint4 a[2 * RT];       // this thread's share of the super-block's RT * 8 * 64 operand vectors
      float sum[kSumShare];  // and of its row sums
    };
    Stage stage[kStages];
    Cursor<FMT> cursor[kUnitTiles];
#pragma unroll
    for (int i = 0; i < kUnitTiles; ++i) cursor[i].open(tile[i].image + size_t(b0) * kRecord, lane);
    const uint4 *share[2 * RT];
#pragma unroll
    for (int j = 0; j < 2 * RT; ++j) {
      const uint32_t at = threadIdx.x + 256u * j, t = at / 512u, g = (at / 64u) % 8u, l = at % 64u;
      share[j] = values + (size_t(t) * G + 8u * b0 + g) * 64u + l;
    }
    // Threads past the staged sums repeat an earlier thread's (same value to the same slot).
    const float *sumShare[kSumShare];
    uint32_t sumSlot[kSumShare];
#pragma unroll
    for (int q = 0; q < kSumShare; ++q) {
      const uint32_t at = (threadIdx.x + 256u * q) % kSumFloats;
      const uint32_t t = at / (kSumsPerBlock * 64u), j = (at / 64u) % kSumsPerBlock, l = at % 64u;
      sumShare[q] = sumsBase + (size_t(t) * sumGroups + kSumsPerBlock * 4u * b0 + 4u * j + (l >> 4)) * 16u + (l & 15u);
      sumSlot[q] = (t * 4u + j) * 64u + l;
    }
    uint32_t issued = b0;  // the next super-block to issue; stops at b1 - 1
    auto issue = [&](Stage &st) {
#pragma unroll
      for (int j = 0; j < 2 * RT; ++j) st.a[j] = *share[j];
#pragma unroll
      for (int q = 0; q < kSumShare; ++q) st.sum[q] = *sumShare[q];
#pragma unroll
      for (int i = 0; i < kUnitTiles; ++i) st.rec[i].load(cursor[i]);
      if (issued + 1 < b1) {  // uniform: scalar branch over a few pointer bumps
        ++issued;
#pragma unroll
        for (int j = 0; j < 2 * RT; ++j) share[j] += 8u * 64u;
#pragma unroll
        for (int q = 0; q < kSumShare; ++q) sumShare[q] += kSumsPerBlock * 4u * 16u;
#pragma unroll
        for (int i = 0; i < kUnitTiles; ++i) cursor[i].advance();
      }
    };
#pragma unroll
    for (int s = 0; s < kStages - 1; ++s) issue(stage[s]);
    const uint32_t count = b1 - b0, rounds = (count + kStages - 1) / kStages;
    uint32_t now = 0;
    for (uint32_t round = 0; round < rounds; ++round) {
#pragma unroll
      for (int u = 0; u < kStages; ++u, ++now) {
        const uint32_t buffer = now & 1u;
#pragma unroll
        for (int j = 0; j < 2 * RT; ++j) (&ldsA[buffer][0][0][0])[threadIdx.x + 256u * j] = stage[u].a[j];
#pragma unroll
        for (int q = 0; q < kSumShare; ++q) (&ldsSums[buffer][0][0][0])[sumSlot[q]] = stage[u].sum[q];
        __syncthreads();
        issue(stage[(u + kStages - 1) % kStages]);
        const float keep = now < count ? 1.0f : 0.0f;
#pragma unroll
        for (int i = 0; i < kUnitTiles; ++i)
          accumulate_record<FMT, RT>(stage[u].rec[i], ldsA[buffer], ldsSums[buffer], acc[i], lane, kq, keep);
      }
    }
  }

  tile[0].image = live[0] ? tile[0].image : nullptr;
#pragma unroll
  for (int i = 1; i < kUnitTiles; ++i) tile[i].image = live[i] ? tile[i].image : nullptr;

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
            __hip_atomic_store(&partials[(size_t(split) * paddedRows + 16u * t + 4u * kq + v) * width + column], acc[i][t][v],
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    // The partials are written and read with agent-scope atomics, which go to the coherence
    // point instead of a compute die's own L2, so no cache write-back or invalidate is needed: the
    // workgroup only waits for its stores to complete before it counts itself in.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x == 0) arrived = __hip_atomic_fetch_add(&counters[blockIdx.x], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (arrived != p.splits - 1) return;
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
              sum += __hip_atomic_load(&partials[(size_t(s) * paddedRows + 16u * t + 4u * kq + v) * width + column],
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            acc[i][t][v] = sum;
          }
      }
    }
    if (threadIdx.x == 0) __hip_atomic_store(&counters[blockIdx.x], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
