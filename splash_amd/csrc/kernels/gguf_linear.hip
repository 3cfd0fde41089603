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
#include "abi/PagedAttention.h"

#include "abi/Gguf.h"
#include "abi/Moe.h"
#include "backend/KernelRegistry.hpp"
#include "kernels/gguf_device.hpp"

namespace splash::kernels {

#define GGUF_DECODE_UNIT_TILES 2

// ---------------------------------------------------------------------------------------------
// gguf_prepare_table: bf16 rows -> the activation table (abi/Gguf.h).
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(64) void gguf_prepare_table(const uint16_t *__restrict__ input, uint8_t *__restrict__ table,
                                                         GgufPrepareParams p) {
  const uint32_t g = blockIdx.x, lane = threadIdx.x, r = lane & 15u, kq = lane >> 4;
  const uint32_t G = p.input_size / 32u, row = 16u * blockIdx.y + r;
  // Row tile blockIdx.y is tile t of its piece's table, which holds `tiles` row tiles.
  const uint32_t piece = blockIdx.y / GGUF_PIECE_TILES, t = blockIdx.y % GGUF_PIECE_TILES;
  const uint32_t tiles = min(uint32_t(GGUF_PIECE_TILES), p.tiles - piece * GGUF_PIECE_TILES);
  table += piece * gguf_table_bytes(p.input_size, GGUF_PIECE_TILES);
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
    float *sums32 = reinterpret_cast<float *>(table + gguf_table_sums32_offset(p.input_size, tiles));
    float *sums16 = reinterpret_cast<float *>(table + gguf_table_sums16_offset(p.input_size, tiles));
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
  const uint16_t *d = nullptr;   // Q6_K only
  const uint2 *fifth = nullptr;  // Q5_K only
  const uint2 *meta8 = nullptr;  // IQ4_XS only: its column's eight bytes
  static constexpr uint32_t kColumnPart = FMT == GGUF_FMT_Q4K   ? 2048u
                                          : FMT == GGUF_FMT_Q6K ? GGUF_Q6K_SCALES
                                          : FMT == GGUF_FMT_Q5K ? GGUF_Q5K_META
                                          : FMT == GGUF_FMT_Q80 ? GGUF_Q80_SCALES
                                                                : GGUF_IQ4_SCALES;
  __device__ __forceinline__ void open(const uint8_t *record, uint32_t lane) {
    const uint4 *p = reinterpret_cast<const uint4 *>(record);
    mine = p + lane;
    column = p + kColumnPart / 16u + (lane & 15u);
    if constexpr (FMT == GGUF_FMT_Q6K) d = reinterpret_cast<const uint16_t *>(record + GGUF_Q6K_D) + (lane & 15u);
    if constexpr (FMT == GGUF_FMT_Q5K) fifth = reinterpret_cast<const uint2 *>(record + GGUF_Q5K_HIGH) + lane;
    if constexpr (FMT == GGUF_FMT_IQ4XS) meta8 = reinterpret_cast<const uint2 *>(record + GGUF_IQ4_SCALES) + (lane & 15u);
  }
  __device__ __forceinline__ void advance() {
    constexpr uint32_t kVectors = gguf_record_bytes(FMT) / 16u;
    mine += kVectors;
    column += kVectors;
    if constexpr (FMT == GGUF_FMT_Q6K) d += kVectors * 8u;
    if constexpr (FMT == GGUF_FMT_Q5K) fifth += kVectors * 2u;
    if constexpr (FMT == GGUF_FMT_IQ4XS) meta8 += kVectors * 2u;
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

template <> struct Record<GGUF_FMT_Q5K> {
  uint4 n0, n1, meta;
  uint2 fifth;
  __device__ __forceinline__ void load(const Cursor<GGUF_FMT_Q5K> &at) {
    n0 = load_stream(at.mine);
    n1 = load_stream(at.mine + 64);
    meta = load_stream(at.column);
    fifth = *at.fifth;
  }
};
template <> struct Record<GGUF_FMT_Q80> {
  uint4 v[4], scales;
  __device__ __forceinline__ void load(const Cursor<GGUF_FMT_Q80> &at) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = load_stream(at.mine + 64 * i);
    scales = load_stream(at.column);
  }
};

template <> struct Record<GGUF_FMT_IQ4XS> {
  uint4 n0, n1;
  uint2 meta;  // x: d | scales_h << 16; y: the low four bits of the eight groups' scales
  __device__ __forceinline__ void load(const Cursor<GGUF_FMT_IQ4XS> &at) {
    n0 = load_stream(at.mine);
    n1 = load_stream(at.mine + 64);
    meta = *at.meta8;
  }
};
template <> struct Record<GGUF_FMT_IQ4NL> {
  uint4 n0, n1, scales;
  __device__ __forceinline__ void load(const Cursor<GGUF_FMT_IQ4NL> &at) {
    n0 = load_stream(at.mine);
    n1 = load_stream(at.mine + 64);
    scales = load_stream(at.column);
  }
};

// The eight groups' operand registers of a record, group g's in ops[g].
template <uint32_t FMT>
__device__ __forceinline__ void iq4_record_operands(const Record<FMT> &r, uint4 ops[8]) {
  ops[0] = iq4_operands(r.n0.x);
  ops[1] = iq4_operands(r.n0.y);
  ops[2] = iq4_operands(r.n0.z);
  ops[3] = iq4_operands(r.n0.w);
  ops[4] = iq4_operands(r.n1.x);
  ops[5] = iq4_operands(r.n1.y);
  ops[6] = iq4_operands(r.n1.z);
  ops[7] = iq4_operands(r.n1.w);
}
__device__ __forceinline__ void record_operands(const Record<GGUF_FMT_IQ4XS> &r, uint4 ops[8]) { iq4_record_operands(r, ops); }
__device__ __forceinline__ void record_operands(const Record<GGUF_FMT_IQ4NL> &r, uint4 ops[8]) { iq4_record_operands(r, ops); }
// Group g's scale of an IQ4_XS record's column: d * (ls - 32), ls its six bits of scales_l and scales_h (exact).
__device__ __forceinline__ float iq4xs_scale(const uint2 &meta, uint32_t g) {
  const uint32_t ls = ((meta.y >> (4u * g)) & 15u) | (((meta.x >> (16u + 2u * g)) & 3u) << 4);
  return half_bits_to_float(meta.x & 0xFFFFu) * float(int(ls) - 32);
}
__device__ __forceinline__ void record_operands(const Record<GGUF_FMT_Q5K> &r, uint4 ops[8]) {
  ops[0] = q5_operands<false, 0>(r.n0.x, r.n0.y, r.fifth.x);
  ops[1] = q5_operands<true, 4>(r.n0.x, r.n0.y, r.fifth.x);
  ops[2] = q5_operands<false, 8>(r.n0.z, r.n0.w, r.fifth.x);
  ops[3] = q5_operands<true, 12>(r.n0.z, r.n0.w, r.fifth.x);
  ops[4] = q5_operands<false, 0>(r.n1.x, r.n1.y, r.fifth.y);
  ops[5] = q5_operands<true, 4>(r.n1.x, r.n1.y, r.fifth.y);
  ops[6] = q5_operands<false, 8>(r.n1.z, r.n1.w, r.fifth.y);
  ops[7] = q5_operands<true, 12>(r.n1.z, r.n1.w, r.fifth.y);
}
__device__ __forceinline__ void record_operands(const Record<GGUF_FMT_Q80> &r, uint4 ops[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    ops[2 * i] = q8_operands(r.v[i].x, r.v[i].y);
    ops[2 * i + 1] = q8_operands(r.v[i].z, r.v[i].w);
  }
}
// Group g's fp16 scale of a Q8_0 record's column.
__device__ __forceinline__ float q8_scale(const uint4 &scales, uint32_t g) {
  const uint32_t word = g < 2 ? scales.x : g < 4 ? scales.y : g < 6 ? scales.z : scales.w;
  return half_bits_to_float((word >> (16u * (g & 1u))) & 0xFFFFu);
}
// Group g's scale of a record of one of the formats whose groups carry one scale and no minimum.
__device__ __forceinline__ float group_scale(const Record<GGUF_FMT_Q80> &r, uint32_t g) { return q8_scale(r.scales, g); }
__device__ __forceinline__ float group_scale(const Record<GGUF_FMT_IQ4NL> &r, uint32_t g) { return q8_scale(r.scales, g); }
__device__ __forceinline__ float group_scale(const Record<GGUF_FMT_IQ4XS> &r, uint32_t g) { return iq4xs_scale(r.meta, g); }
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
  if constexpr (FMT == GGUF_FMT_Q80 || FMT == GGUF_FMT_IQ4XS || FMT == GGUF_FMT_IQ4NL) {
#pragma unroll
    for (uint32_t g = 0; g < 8; ++g) {
      const float d = group_scale(rec, g);
      const uint32_t regs[4] = {ops[g].x, ops[g].y, ops[g].z, ops[g].w};
#pragma unroll
      for (uint32_t e = 0; e < 8; ++e)
        row[32u * g + gguf_operand_input(kq, e)] = d * (bf16_bits_to_float((regs[e >> 1] >> (16u * (e & 1u))) & 0xFFFFu) - 128.f);  // exact
    }
  } else if constexpr (FMT == GGUF_FMT_Q4K || FMT == GGUF_FMT_Q5K) {
    const Q4KScales sc = q4k_scales(rec.meta);
#pragma unroll
    for (uint32_t g = 0; g < 8; ++g) {
      const float s = sc.d * byte_of(g < 4 ? sc.sc_lo : sc.sc_hi, g & 3u);
      const float m = -(sc.dmin * byte_of(g < 4 ? sc.mn_lo : sc.mn_hi, g & 3u));
      const uint32_t regs[4] = {ops[g].x, ops[g].y, ops[g].z, ops[g].w};
#pragma unroll
      for (uint32_t e = 0; e < 8; ++e) {
        const float code = float(operand_code(regs[e >> 1], e & 1u) & (FMT == GGUF_FMT_Q5K ? 0x1Fu : 0xFu));
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
SP_REGISTER_KERNEL("gguf_dequant_q5k", &gguf_dequant<GGUF_FMT_Q5K>);
SP_REGISTER_KERNEL("gguf_dequant_q80", &gguf_dequant<GGUF_FMT_Q80>);
SP_REGISTER_KERNEL("gguf_dequant_iq4xs", &gguf_dequant<GGUF_FMT_IQ4XS>);
SP_REGISTER_KERNEL("gguf_dequant_iq4nl", &gguf_dequant<GGUF_FMT_IQ4NL>);

// ---------------------------------------------------------------------------------------------
// The decode projection.
// ---------------------------------------------------------------------------------------------
// Streams are read through buffer resources: a load past the end of its range returns zeros and
// moves no memory, so the software pipeline below needs no branch around a load and no
// special case at the end of a range, and its address arithmetic is one 32-bit add per stream.
using Resource = __amdgpu_buffer_rsrc_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
__device__ __forceinline__ Resource make_resource(const void *base, uint32_t bytes) {
  // The base must be wave-uniform (it lives in scalar registers).
  const uint64_t v = reinterpret_cast<uint64_t>(base);
  // readfirstlane returns a signed int: widen each half as unsigned.
  const uint32_t hi = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(v >> 32))));
  const uint32_t lo = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(v))));
  const uint64_t u = (uint64_t(hi) << 32) | uint64_t(lo);
  return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void *>(u), 0, __builtin_amdgcn_readfirstlane(int(bytes)), 0x00020000);
}
constexpr int kStreamOnce = 2;  // non-temporal: weights are read once
template <int Aux> __device__ __forceinline__ uint4 load128(Resource r, uint32_t offset) {
  const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, int(offset), 0, Aux);
  return make_uint4(v.x, v.y, v.z, v.w);
}
// `mine` is the lane's 16 bytes of the record's first 1024-byte part, `column` its column's scale
// field, both as byte offsets into the resource.
__device__ __forceinline__ void load_record(Record<GGUF_FMT_Q4K> &rec, Resource r, uint32_t mine, uint32_t column) {
  rec.n0 = load128<kStreamOnce>(r, mine);
  rec.n1 = load128<kStreamOnce>(r, mine + 1024u);
  rec.meta = load128<kStreamOnce>(r, column);
}
__device__ __forceinline__ void load_record(Record<GGUF_FMT_Q6K> &rec, Resource r, uint32_t mine, uint32_t column) {
  rec.n0 = load128<kStreamOnce>(r, mine);
  rec.n1 = load128<kStreamOnce>(r, mine + 1024u);
  rec.high = load128<kStreamOnce>(r, mine + 2048u);
  rec.scales = load128<kStreamOnce>(r, column);
  // The lane's 16 l and the column's 16 c locate the record and c: d sits at record + 3328 + 2 c.
  const uint32_t lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  rec.d = __builtin_amdgcn_raw_buffer_load_b16(r, int(mine - 16u * lane + GGUF_Q6K_D + 2u * (lane & 15u)), 0, kStreamOnce);
}

__device__ __forceinline__ void load_record(Record<GGUF_FMT_Q5K> &rec, Resource r, uint32_t mine, uint32_t column) {
  rec.n0 = load128<kStreamOnce>(r, mine);
  rec.n1 = load128<kStreamOnce>(r, mine + 1024u);
  rec.meta = load128<kStreamOnce>(r, column);
  // The lane's 8 bytes of fifth bits sit at record + 2048 + 8 l; `mine` is record + 16 l.
  const uint32_t lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  const u32x2 fifth = __builtin_amdgcn_raw_buffer_load_b64(r, int(mine - 8u * lane + GGUF_Q5K_HIGH), 0, kStreamOnce);
  rec.fifth = make_uint2(fifth.x, fifth.y);
}
__device__ __forceinline__ void load_record(Record<GGUF_FMT_Q80> &rec, Resource r, uint32_t mine, uint32_t column) {
#pragma unroll
  for (uint32_t i = 0; i < 4; ++i) rec.v[i] = load128<kStreamOnce>(r, mine + 1024u * i);
  rec.scales = load128<kStreamOnce>(r, column);
}

__device__ __forceinline__ void load_record(Record<GGUF_FMT_IQ4XS> &rec, Resource r, uint32_t mine, uint32_t) {
  rec.n0 = load128<kStreamOnce>(r, mine);
  rec.n1 = load128<kStreamOnce>(r, mine + 1024u);
  // The column's 8 bytes sit at record + 2048 + 8 c; `mine` is record + 16 l.
  const uint32_t lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  const u32x2 meta = __builtin_amdgcn_raw_buffer_load_b64(r, int(mine - 16u * lane + GGUF_IQ4_SCALES + 8u * (lane & 15u)), 0, kStreamOnce);
  rec.meta = make_uint2(meta.x, meta.y);
}
__device__ __forceinline__ void load_record(Record<GGUF_FMT_IQ4NL> &rec, Resource r, uint32_t mine, uint32_t column) {
  rec.n0 = load128<kStreamOnce>(r, mine);
  rec.n1 = load128<kStreamOnce>(r, mine + 1024u);
  rec.scales = load128<kStreamOnce>(r, column);
}

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
// acc[t] = fma(dot(step, t), scale(step), acc[t]) over a record's `Steps` steps in order, every row tile. A step's
// products are issued before the multiply-adds of the step before it, so that those run while the matrix cores work
// (each element's multiply-adds keep their order: the sums are the same).
template <int RT, uint32_t Steps, class Dot, class Scale>
__device__ __forceinline__ void scaled_groups(f32x4 (&acc)[RT], Dot dot, Scale scale) {
  // (not the two-tile Q6_K kernel, whose sixteen steps of two products would cost it a wave a SIMD in registers)
  if constexpr (!(RT == 2 && Steps == 16)) {
    f32x4 held[2][RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) held[0][t] = dot(0u, t);
#pragma unroll
    for (uint32_t j = 1; j <= Steps; ++j) {
      if (j < Steps) {
#pragma unroll
        for (int t = 0; t < RT; ++t) held[j & 1u][t] = dot(j, t);
      }
      const float s = scale(j - 1u);
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[t][i] = __fmaf_rn(held[(j - 1u) & 1u][t][i], s, acc[t][i]);
    }
  } else {
#pragma unroll
    for (uint32_t j = 0; j < Steps; ++j) {
      const float s = scale(j);
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        const f32x4 product = dot(j, t);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[t][i] = __fmaf_rn(product[i], s, acc[t][i]);
      }
    }
  }
}

template <uint32_t FMT, int RT>
__device__ __forceinline__ void accumulate_record(const Record<FMT> &rec, const uint4 (*a)[8][64], const float (*sums)[4][64],
                                                  f32x4 (&acc)[RT], uint32_t lane, uint32_t kq) {
  uint4 ops[8];
  record_operands(rec, ops);
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  if constexpr (FMT == GGUF_FMT_Q80 || FMT == GGUF_FMT_IQ4XS || FMT == GGUF_FMT_IQ4NL) {
    // One scale a group; the operands' 128 leaves through the row sums: -128 s of groups kq and 4 + kq.
    float s[8];
#pragma unroll
    for (uint32_t g = 0; g < 8; ++g) s[g] = group_scale(rec, g);
    float c_lo, c_hi;
    if constexpr (FMT == GGUF_FMT_IQ4XS) {
      c_lo = -128.f * iq4xs_scale(rec.meta, kq);
      c_hi = -128.f * iq4xs_scale(rec.meta, 4u + kq);
    } else {
      const uint32_t lowWord = kq == 0 ? rec.scales.x : kq == 1 ? rec.scales.x >> 16 : kq == 2 ? rec.scales.y : rec.scales.y >> 16;
      const uint32_t highWord = kq == 0 ? rec.scales.z : kq == 1 ? rec.scales.z >> 16 : kq == 2 ? rec.scales.w : rec.scales.w >> 16;
      c_lo = -128.f * half_bits_to_float(lowWord & 0xFFFFu);
      c_hi = -128.f * half_bits_to_float(highWord & 0xFFFFu);
    }
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[t][0][lane], c_lo, acc[t], 0, 0, 0);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[t][1][lane], c_hi, acc[t], 0, 0, 0);
    }
    scaled_groups<RT, 8>(acc, [&](uint32_t g, int t) {
      return __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a[t][g][lane]), as_bf16x8(ops[g]), zero, 0, 0, 0);
    }, [&](uint32_t g) { return s[g]; });
  } else if constexpr (FMT == GGUF_FMT_Q4K || FMT == GGUF_FMT_Q5K) {
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
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[t][0][lane], c_lo, acc[t], 0, 0, 0);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[t][1][lane], c_hi, acc[t], 0, 0, 0);
    }
    scaled_groups<RT, 8>(acc, [&](uint32_t g, int t) {
      return __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a[t][g][lane]), as_bf16x8(ops[g]), zero, 0, 0, 0);
    }, [&](uint32_t g) { return s[g]; });
  } else {
    const float d = half_bits_to_float(rec.d);
    // Constant terms of 16-input blocks 4 j + kq: -160 d sc (operand 128 + q, value q - 32).
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
      const uint32_t word = j == 0 ? rec.scales.x : j == 1 ? rec.scales.y : j == 2 ? rec.scales.z : rec.scales.w;
      const float coef = -160.f * (d * float(int(int8_t((word >> (8u * kq)) & 0xFFu))));
#pragma unroll
      for (int t = 0; t < RT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[t][j][lane], coef, acc[t], 0, 0, 0);
    }
    // a step is half a group: 16 inputs under one scale
    scaled_groups<RT, 16>(acc, [&](uint32_t j, int t) {
      const uint32_t g = j >> 1;
      const uint4 av = a[t][g][lane];
      const uint2 bw = j & 1u ? make_uint2(ops[g].z, ops[g].w) : make_uint2(ops[g].x, ops[g].y);
      const uint2 aw = j & 1u ? make_uint2(av.z, av.w) : make_uint2(av.x, av.y);
      return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, aw), __builtin_bit_cast(s16x4, bw), zero, 0, 0, 0);
    }, [&](uint32_t j) { return d * q6_scale(rec.scales, j); });
  }
}

// The staged rule (the reference's staged tile, kernels/common/gguf_staged.h:12-66: every weight decoded with fp32 group
// coefficients and rounded once to half, products with the bf16 inputs accumulated in fp32): a group's eight values of
// this lane as halves, each split into the bf16 that holds its leading eight significant bits and the bf16 that holds
// the rest (a half has eleven), so that two bf16 MFMAs multiply the inputs by the half exactly; the constant terms ride
// in the values, so the row sums stay unread.
__device__ __forceinline__ void staged_operands(const float (&value)[8], bf16x8 &high, bf16x8 &low) {
  uint32_t highWords[4], lowWords[4];
#pragma unroll
  for (uint32_t e = 0; e < 8; e += 2) {
    uint32_t h[2], l[2];
#pragma unroll
    for (uint32_t i = 0; i < 2; ++i) {
      const float rounded = float(_Float16(value[e + i]));                    // the staged tile's half
      const uint32_t bits = __float_as_uint(rounded), lead = bits & 0xFFFF0000u;  // a bf16: sign, exponent, seven fraction bits
      h[i] = lead >> 16;
      l[i] = __float_as_uint(rounded - __uint_as_float(lead)) >> 16;           // at most three significant bits: a bf16 holds them
    }
    highWords[e / 2] = h[0] | (h[1] << 16);
    lowWords[e / 2] = l[0] | (l[1] << 16);
  }
  high = as_bf16x8(make_uint4(highWords[0], highWords[1], highWords[2], highWords[3]));
  low = as_bf16x8(make_uint4(lowWords[0], lowWords[1], lowWords[2], lowWords[3]));
}
// A record's coefficients of the staged rule and a group's two operands.
template <uint32_t FMT> struct StagedCoefficients {
  Q4KScales sc{};
  float d6 = 0.f;
  __device__ __forceinline__ explicit StagedCoefficients(const Record<FMT> &rec) {
    if constexpr (FMT == GGUF_FMT_Q4K || FMT == GGUF_FMT_Q5K) sc = q4k_scales(rec.meta);
    if constexpr (FMT == GGUF_FMT_Q6K) d6 = half_bits_to_float(rec.d);
  }
};
// A group's eight values of this lane in fp32, element e the lane's input gguf_operand_input(kq, e).
template <uint32_t FMT>
__device__ __forceinline__ void staged_values(const Record<FMT> &rec, const StagedCoefficients<FMT> &k, const uint4 &operand, uint32_t g,
                                              float (&value)[8]) {
  const uint32_t regs[4] = {operand.x, operand.y, operand.z, operand.w};
  // the fp32 values of gguf_dequant, each exact or rounded once
  if constexpr (FMT == GGUF_FMT_Q80 || FMT == GGUF_FMT_IQ4XS || FMT == GGUF_FMT_IQ4NL) {
    const float d = group_scale(rec, g);
#pragma unroll
    for (uint32_t e = 0; e < 8; ++e) value[e] = d * (bf16_bits_to_float((regs[e >> 1] >> (16u * (e & 1u))) & 0xFFFFu) - 128.f);
  } else if constexpr (FMT == GGUF_FMT_Q4K || FMT == GGUF_FMT_Q5K) {
    const float s = k.sc.d * byte_of(g < 4 ? k.sc.sc_lo : k.sc.sc_hi, g & 3u);
    const float m = -(k.sc.dmin * byte_of(g < 4 ? k.sc.mn_lo : k.sc.mn_hi, g & 3u));
#pragma unroll
    for (uint32_t e = 0; e < 8; ++e)
      value[e] = __fmaf_rn(s, float(operand_code(regs[e >> 1], e & 1u) & (FMT == GGUF_FMT_Q5K ? 0x1Fu : 0xFu)), m);
  } else {
#pragma unroll
    for (uint32_t e = 0; e < 8; ++e)
      value[e] = (k.d6 * q6_scale(rec.scales, 2u * g + (e >> 2))) * float(int(operand_code(regs[e >> 1], e & 1u) & 0x3Fu) - 32);
  }
}
template <uint32_t FMT>
__device__ __forceinline__ void staged_group(const Record<FMT> &rec, const StagedCoefficients<FMT> &k, const uint4 &operand, uint32_t g,
                                             bf16x8 &high, bf16x8 &low) {
  float value[8];
  staged_values(rec, k, operand, g, value);
  staged_operands(value, high, low);
}
template <uint32_t FMT, int RT>
__device__ __forceinline__ void accumulate_record_staged(const Record<FMT> &rec, const uint4 (*a)[8][64], f32x4 (&acc)[RT], uint32_t lane,
                                                         uint32_t kq) {
  uint4 ops[8];
  record_operands(rec, ops);
  const StagedCoefficients<FMT> k(rec);
#pragma unroll
  for (uint32_t g = 0; g < 8; ++g) {
    bf16x8 high, low;
    staged_group(rec, k, ops[g], g, high, low);
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const bf16x8 rows = as_bf16x8(a[t][g][lane]);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rows, high, acc[t], 0, 0, 0);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rows, low, acc[t], 0, 0, 0);
    }
  }
  (void)kq;
}

// Work split: a wave owns one column tile over the workgroup's K range; the four waves of a
// workgroup walk that range in step and share its activations through LDS. Unit u of a dispatch
// is tile u of its concatenated segments; of a gate/up pair, unit 2 j is gate tile j and unit
// 2 j + 1 up tile j, so the two halves of a pair sit in neighbouring waves of one workgroup.
// `item` is the workgroup's place in the dispatch (blockIdx.x of gguf_decode).
// A workgroup's LDS, which the kernel declares once whatever formats its workgroups decode.
// The four-tile kernels keep ONE buffer of a super-block's activations (two barriers a super-block instead of one): at
// 32 KiB instead of 64 a compute unit holds three of their workgroups, not two, which their waits on LDS and on the
// weight stream need more than they need the barrier. `spare` extends the buffer for the epilogues that lay rows out in it.
template <int RT> struct DecodeShared {
  static constexpr int kBuffers = RT > 2 ? 1 : 2;
  uint4 a[kBuffers][RT][8][64];
  uint4 spare[RT > 2 ? 512 : 1];
  float sums[kBuffers][RT][4][64];
  uint32_t arrived;
  float scaleParts[256 * RT], rowScale[16 * RT];  // of a table with a deferred scale
};

// A projection's place in a chain of projections that share one dispatch (gguf_decode_chain): link i + 1 reads what link
// i's epilogues wrote, so its workgroups, which the device starts after every workgroup of link i, fetch their first
// weights, which depend on nothing, and then wait for link i's count of finished workgroups. Results that a later link
// reads leave through agent-scope stores, which go to the memory side of the compute dies' caches, and are counted in
// only once those stores have completed; the reader finds no older copy of them in its own die's cache because nothing
// of the dispatch read those addresses before (every link has tables, partials and counters of its own) and every
// cache line it reads through the cache had a single writer.
struct ChainPosition {
  // The link before's go flag this workgroup polls (one of GGUF_CHAIN_FLAGS words in cache lines of their own, so that the
  // device's waiting workgroups do not all ask one memory channel for one word); null for the first link.
  uint32_t *wait;
  uint32_t *done;       // this link's count, of doneTarget workgroups
  uint32_t doneTarget;
  uint32_t *flags;      // this link's go flags, which the workgroup that completes the count sets; null for the last link
  uint32_t *flagsBefore;  // the link before's, which that workgroup clears: every workgroup of this link has passed them
  uint32_t spinLimit;   // polls a workgroup waits before it gives up and reports through *status
  uint32_t *status;
};
template <bool Coherent, class T> __device__ __forceinline__ void store_result(T *at, T value) {
  if constexpr (Coherent) __hip_atomic_store(at, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else *at = value;
}
template <bool Coherent, class T> __device__ __forceinline__ T load_result(const T *at) {
  if constexpr (Coherent) return __hip_atomic_load(at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else return *at;
}
// The wait of a link's workgroup: one thread polls, with a bound, so that every wave ends whatever the count does.
__device__ __forceinline__ void chain_wait(const ChainPosition &chain) {
  if (chain.wait) {
    if (threadIdx.x == 0) {
      uint32_t polls = 0;
      while (__hip_atomic_load(chain.wait, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u) {
        if (++polls > chain.spinLimit) {
          __hip_atomic_store(chain.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        __builtin_amdgcn_s_sleep(8);
      }
    }
    __syncthreads();
  }
  // nothing that reads the link before's results moves above the wait
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  __builtin_amdgcn_sched_barrier(0);
}

// The head norms, RoPE and cache store of attention_q8_qkv (kernels/paged_attention.hip; the reference's
// attention_qkv_prepare.h:59-66, attention_store.h:52-85) as the epilogue of the fused q|k|v projection
// (GGUF_EPILOGUE_QKV_PREPARE): what that kernel binds and its parameters.
struct QkvPrepare {
  const uint16_t *queryNorm, *keyNorm;
  const float *ropeCos, *ropeSin;
  _Float16 *queries;
  float *querySums;
  const uint64_t *pageTable;
  uint8_t *pool;
  const AttentionParams *attention;
};
// One head's rows, a wave a row at a time, four rows a wave of each 16: `tile` holds the head's columns of every packed
// row as the projection's bf16 results (the values attention_q8_qkv reads back from the packed rows), lane l of a wave
// elements l and l + 64 of its row. Every sum and maximum is taken as attention_q8_qkv's 64-lane waves take them (a
// butterfly over elements 0..63, one over 64..127, then the two added in that order), so the staged queries, their sums,
// the cached codes and scales are that kernel's bit for bit.
// What a row needs from memory does not depend on the projection's sums -- its sequence, its RoPE angles, its page --
// so a wave fetches that of its four rows ahead (QkvRowsAhead), before the sums' own loads, and the epilogue waits
// for one round trip instead of one a row.
struct QkvRowAhead {
  uint32_t z, row, token;   // the sequence (sequences: the packed row is in no block), the row of its block, its slot in the page
  float cosine[2], sine[2];
  uint64_t page;            // the physical page of the row's slot
};
struct QkvHead {
  bool query, key;
  uint32_t index, group;    // the head among its kind; query heads a KV head
  uint32_t weight[2];       // the head norm's weights of this lane's elements, as loaded (converted where they are used, so
                            // that nothing waits for them before the other loads have left)
};
__device__ __forceinline__ QkvHead qkv_head(uint32_t head, const QkvPrepare &q) {
  const AttentionParams &a = *q.attention;
  const uint32_t lane = threadIdx.x & 63u, halves = a.head_dim / 64u;
  QkvHead h;
  h.query = head < a.q_heads;
  h.key = !h.query && head < a.q_heads + a.kv_heads;
  h.index = h.query ? head : h.key ? head - a.q_heads : head - a.q_heads - a.kv_heads;
  h.group = a.q_heads / a.kv_heads;
  h.weight[0] = h.weight[1] = 0;
  if (a.normalize && (h.query || h.key))
    _Pragma("unroll") for (uint32_t e = 0; e < 2u; ++e) if (e < halves) h.weight[e] = (h.query ? q.queryNorm : q.keyNorm)[lane + 64u * e];
  return h;
}
__device__ __forceinline__ void qkv_rows_ahead(QkvRowAhead (&ahead)[4], const QkvHead &h, uint32_t first, uint32_t rows, const QkvPrepare &q) {
  const AttentionParams &a = *q.attention;
  const uint32_t lane = threadIdx.x & 63u, halves = a.head_dim / 64u;
  // a wave's rows are the same in every lane: the search of their sequences runs on the scalar unit
  const uint32_t wave = uint32_t(__builtin_amdgcn_readfirstlane(int(threadIdx.x >> 6)));
  uint32_t entry[4] = {0, 0, 0, 0};
#pragma unroll
  for (uint32_t i = 0; i < 4; ++i) ahead[i].z = a.sequences;
  for (uint32_t s = 0; s < a.sequences; ++s) {
    const AttentionSequence seq = a.sequence[s];
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
      const uint32_t packed = first + wave + 4u * i;
      if (packed < rows && packed - seq.first_row < seq.rows) {
        const uint32_t slot = seq.committed + (packed - seq.first_row);
        ahead[i].z = s;
        ahead[i].row = packed - seq.first_row;
        ahead[i].token = slot % ATTENTION_PAGE_TOKENS;
        entry[i] = seq.table_first + slot / ATTENTION_PAGE_TOKENS;
      }
    }
  }
#pragma unroll
  for (uint32_t i = 0; i < 4; ++i) {
    QkvRowAhead &r = ahead[i];
    if (r.z == a.sequences) continue;
    const uint32_t packed = first + wave + 4u * i;
    if (a.rotary_pairs && (h.query || h.key))
      _Pragma("unroll") for (uint32_t e = 0; e < 2u; ++e) if (e < halves) {
        const uint32_t at = lane + 64u * e;
        if (at < 2u * a.rotary_pairs) {
          const uint32_t pair = at < a.rotary_pairs ? at : at - a.rotary_pairs;
          r.cosine[e] = q.ropeCos[size_t(packed) * a.rotary_pairs + pair];
          r.sine[e] = q.ropeSin[size_t(packed) * a.rotary_pairs + pair];
        }
      }
    if (!h.query) r.page = q.pageTable[entry[i]];
  }
}
// A wave's four rows move through the stages together: the reductions of different rows are independent chains the
// hardware overlaps, and no row waits for the stores of the one before it.
__device__ __forceinline__ void qkv_prepare_rows(const float (*tile)[128], float (*staged)[4][128], const QkvRowAhead (&ahead)[4],
                                                 const QkvHead &head, uint32_t first, const QkvPrepare &q) {
  const AttentionParams &a = *q.attention;
  const uint32_t lane = threadIdx.x & 63u, wave = uint32_t(__builtin_amdgcn_readfirstlane(int(threadIdx.x >> 6)));
  const uint32_t D = a.head_dim, halves = D / 64u;
  const bool query = head.query, key = head.key, two = halves == 2u;
  const uint32_t index = head.index, group = head.group;
  // the weights' bits become floats here and no earlier: the conversion placed at their load would wait for it there
  uint32_t weightBits[2] = {head.weight[0], head.weight[1]};
  asm volatile("" : "+v"(weightBits[0]), "+v"(weightBits[1]));
  const float weight[2] = {bf16_bits_to_float(weightBits[0]), bf16_bits_to_float(weightBits[1])};
  bool valid[4];
  float result[4][2];
#pragma unroll
  for (uint32_t i = 0; i < 4; ++i) {
    valid[i] = ahead[i].z != a.sequences;
    const uint32_t packed = first + wave + 4u * i;
    result[i][0] = valid[i] ? tile[packed][lane] : 0.f;
    result[i][1] = valid[i] && two ? tile[packed][lane + 64u] : 0.f;
  }
  if (a.normalize && (query || key)) {
    // attention_qkv_prepare.h:59-66: inv = rsqrt(sum x^2 / D + 1e-6); n = bf16(x inv w)
    float total[4], high[4];
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) total[i] = wave_sum(result[i][0] * result[i][0]);
    if (two) {
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) high[i] = wave_sum(result[i][1] * result[i][1]);
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) total[i] += high[i];
    }
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
      const float inverse = 1.0f / sqrtf(total[i] / float(D) + 1e-6f);
      result[i][0] = round_bf16(result[i][0] * inverse * weight[0]);
      if (two) result[i][1] = round_bf16(result[i][1] * inverse * weight[1]);
    }
  }
  if (a.rotary_pairs && (query || key)) {
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
      staged[wave][i][lane] = result[i][0];
      if (two) staged[wave][i][lane + 64u] = result[i][1];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i)
      _Pragma("unroll") for (uint32_t h = 0; h < 2u; ++h) if (h < halves) {
        const uint32_t at = lane + 64u * h;
        if (valid[i] && at < 2u * a.rotary_pairs) {
          const uint32_t pair = at < a.rotary_pairs ? at : at - a.rotary_pairs;
          const float low = staged[wave][i][pair], other = staged[wave][i][pair + a.rotary_pairs];
          const float cosine = ahead[i].cosine[h], sine = ahead[i].sine[h];
          result[i][h] = at < a.rotary_pairs ? round_bf16(low * cosine - other * sine) : round_bf16(other * cosine + low * sine);
        }
      }
    __builtin_amdgcn_wave_barrier();
  }
  if (query) {
    _Float16 half[4][2];
    float sum[4], high[4];
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
      half[i][0] = _Float16(result[i][0]);
      half[i][1] = _Float16(result[i][1]);
      sum[i] = wave_sum(float(half[i][0]));
    }
    if (two) {
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) high[i] = wave_sum(float(half[i][1]));
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) sum[i] += high[i];
    }
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
      if (!valid[i]) continue;
      const size_t at = (size_t(ahead[i].z) * a.kv_heads * group + index) * 16u + ahead[i].row;
      q.queries[at * D + lane] = half[i][0];
      if (two) q.queries[at * D + lane + 64u] = half[i][1];
      if (lane == 0) q.querySums[at] = sum[i];
    }
    return;
  }
  // attention_store.h:52-85: scale = max / 127, code = clamp(rint(v 127 / max)); the scale is stored fp16.
  float largest[4];
#pragma unroll
  for (uint32_t i = 0; i < 4; ++i) largest[i] = wave_max(fmaxf(fabsf(result[i][0]), fabsf(result[i][1])));
#pragma unroll
  for (uint32_t i = 0; i < 4; ++i) {
    if (!valid[i]) continue;
    const QkvRowAhead &r = ahead[i];
    uint8_t *page = q.pool + r.page * a.page_bytes;
    _Pragma("unroll") for (uint32_t h = 0; h < 2u; ++h) if (h < halves) {
      int code = 0;
      if (largest[i] != 0.0f) {
        code = int(rintf(result[i][h] * 127.0f / largest[i]));
        code = code < -127 ? -127 : code > 127 ? 127 : code;
      }
      const uint32_t dim = lane + 64u * h;
      if (key) reinterpret_cast<int8_t *>(page)[attention_key_index(index, r.token, dim, D)] = int8_t(code);
      else reinterpret_cast<int8_t *>(page + attention_page_values_offset(a.kv_heads, D))[attention_value_index(index, r.token, dim, D)] = int8_t(code);
    }
    if (lane == 0) {
      uint16_t *scales = reinterpret_cast<uint16_t *>(page + (key ? attention_page_key_scales_offset(a.kv_heads, D) : attention_page_value_scales_offset(a.kv_heads, D)));
      scales[attention_scale_index(index, r.token)] = uint16_t(float_to_half_bits(largest[i] == 0.0f ? 0.0f : largest[i] / 127.0f));
    }
  }
}
// the staged rows past a sequence's block are zero (the attention kernel reads 16 rows a head)
__device__ __forceinline__ void qkv_clear_rows(const QkvHead &head, const QkvPrepare &q) {
  const AttentionParams &a = *q.attention;
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, D = a.head_dim, halves = D / 64u;
  if (!head.query) return;
  for (uint32_t z = 0; z < a.sequences; ++z)
    for (uint32_t row = a.sequence[z].rows + wave; row < 16u; row += 4u) {
      const size_t at = (size_t(z) * a.kv_heads * head.group + head.index) * 16u + row;
      _Pragma("unroll") for (uint32_t h = 0; h < 2u; ++h) if (h < halves) q.queries[at * D + lane + 64u * h] = _Float16(0.f);
      if (lane == 0) q.querySums[at] = 0.f;
    }
}

template <uint32_t FMT, int RT, uint32_t EP, bool Chain = false, bool Staged = false>
__device__ __forceinline__ void decode_workgroup(DecodeShared<RT> &shared, const uint8_t *__restrict__ seg0,
                                                 const uint8_t *__restrict__ seg1, const uint8_t *__restrict__ seg2,
                                                 const uint8_t *__restrict__ table, void *__restrict__ out,
                                                 const uint16_t *__restrict__ residual, float *__restrict__ partials,
                                                 uint32_t *__restrict__ counters, const GgufDecodeParams &p, const uint32_t item,
                                                 const ChainPosition &chain = ChainPosition{}, const QkvPrepare *prepare = nullptr) {
  // A chained link reads only what has one writer a cache line: a group's values, a workgroup's 16-input sums, a squares
  // entry. The 32-input sums have two (a gate/up workgroup writes 64 bytes of them), so a chained link adds the two
  // 16-input sums they are the sum of, the same fp32 addition their writer made.
  constexpr bool kPairSums = Chain && FMT != GGUF_FMT_Q6K;
  constexpr uint32_t kRecord = gguf_record_bytes(FMT);
  constexpr bool kTable = EP == GGUF_EPILOGUE_GATE_UP_TABLE, kGateUp = EP == GGUF_EPILOGUE_GATE_UP || kTable;
  constexpr uint32_t kColumnPart = Cursor<FMT>::kColumnPart;
  constexpr bool kSums32 = FMT != GGUF_FMT_Q6K;                // the constant term rides on 32-input sums (Q6_K: 16)
  constexpr uint32_t kSumsPerBlock = kSums32 ? 2 : 4;          // K = 4 MFMAs of row sums per super-block
  // The range's activations pass through LDS one super-block at a time (two buffers, one barrier
  // per super-block), each wave fetching a quarter of them, so a wave's vector-memory queue holds
  // almost only weights and the MFMA operands arrive on the LDS counter instead.
  auto &ldsA = shared.a;
  auto &ldsSums = shared.sums;
  uint32_t &arrived = shared.arrived;
  auto &scaleParts = shared.scaleParts;
  auto &rowScale = shared.rowScale;

  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, c = lane & 15u, kq = lane >> 4;
  // Workgroup items: the whole groups first, then the partitioned ones part by part.
  uint32_t group = item, split = 0, splits = 1;
  if (item >= p.whole_groups && p.splits > 1) {
    const uint32_t past = item - p.whole_groups;
    group = p.whole_groups + uint32_t(__builtin_amdgcn_readfirstlane(int(past / p.splits)));
    split = uint32_t(__builtin_amdgcn_readfirstlane(int(past % p.splits)));
    splits = p.splits;
  }
  const uint32_t unit = group * 4u + wave;
  const uint32_t blocks = p.input_size / GGUF_BLOCK, G = p.input_size / 32u;
  const uint32_t tiles = gguf_row_tiles(p.rows);
  const bool live = unit < p.units;

  TileRef tile{nullptr, 0};
  if (live) {
    if constexpr (kGateUp) {
      tile = {(unit & 1u ? seg1 : seg0) + size_t(unit >> 1) * blocks * kRecord, p.offset[0] + (unit >> 1) * GGUF_TILE_COLUMNS};
    } else if constexpr (EP == GGUF_EPILOGUE_RESIDUAL_NORM) {
      // one segment: the other two slots bind the norm's weights and the next projection's table
      tile = {seg0 + size_t(unit) * blocks * kRecord, p.offset[0] + unit * GGUF_TILE_COLUMNS};
    } else {
      const uint8_t *const seg[3] = {seg0, seg1, seg2};
      tile = find_tile(unit, seg, p, kRecord);
    }
  }

  // The workgroup's super-blocks: part `split` of K.
  // (blocks <= 2^16 and splits <= 16, so the products fit 32 bits; the quotients are wave-uniform.)
  const uint32_t b0 = uint32_t(__builtin_amdgcn_readfirstlane(int(blocks * split / splits)));
  const uint32_t b1 = uint32_t(__builtin_amdgcn_readfirstlane(int(blocks * (split + 1u) / splits)));
  const uint32_t count = b1 - b0;

  f32x4 acc[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  {
    // A software pipeline of kStages super-blocks in registers: the loads of super-block
    // b + kStages - 1 are issued before the MFMAs of super-block b, so kStages - 1 super-blocks of
    // weights per wave stay in flight (loads return in issue order, so waiting for b's never
    // waits for a later one's). Loads past the range return zeros without touching memory.
    constexpr int kStages = RT > 2 ? 2 : 3;
    constexpr uint32_t kSumFloats = RT * kSumsPerBlock * 64u;  // staged row sums per super-block
    constexpr int kSumShare = (kSumFloats + 255u) / 256u;
    struct Stage {
      Record<FMT> rec;
      uint4 a[2 * RT];       // this thread's share of the super-block's RT * 8 * 64 operand vectors
      float sum[kSumShare];  // and of its row sums
      float second[kPairSums ? kSumShare : 1];  // a chained link: the other 16-input half of a 32-input sum
    };
    Stage stage[kStages];
    // A wave without a tile reads an empty range.
    const Resource weights = make_resource(tile.image ? tile.image + size_t(b0) * kRecord : seg0, tile.image ? count * kRecord : 0u);
    uint32_t mine = 16u * lane, column = kColumnPart + 16u * c;
    // The table's values of row tile t, super-blocks b0..b1: one resource per row tile.
    Resource values[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t)  // a row tile past the table's reads as zeros
      values[t] = make_resource(table + (size_t(uint32_t(t) < tiles ? t : 0) * G + 8u * b0) * 1024u, uint32_t(t) < tiles ? count * 8192u : 0u);
    uint32_t share[2];  // vector j of a row tile's super-block: byte offset of this thread's
#pragma unroll
    for (int j = 0; j < 2; ++j) share[j] = (threadIdx.x + 256u * j) * 16u;
    const uint32_t sumsAt = kSums32 && !kPairSums ? gguf_table_sums32_offset(p.input_size, tiles) : gguf_table_sums16_offset(p.input_size, tiles);
    const uint32_t sumGroups = kSums32 ? G : 2u * G;  // row-sum entries per row tile
    const Resource sums = make_resource(table + sumsAt, tiles * (kPairSums ? 2u * G : sumGroups) * 64u);
    // Threads past the staged sums repeat an earlier thread's (same value to the same slot).
    uint32_t sumShare[kSumShare], sumSlot[kSumShare];
#pragma unroll
    for (int q = 0; q < kSumShare; ++q) {
      const uint32_t at = (threadIdx.x + 256u * q) % kSumFloats;
      const uint32_t t = at / (kSumsPerBlock * 64u), j = (at / 64u) % kSumsPerBlock, l = at % 64u;
      sumShare[q] = ((t * sumGroups + kSumsPerBlock * 4u * b0 + 4u * j + (l >> 4)) * 16u * (kPairSums ? 2u : 1u) + (l & 15u)) * 4u;
      sumSlot[q] = (t * 4u + j) * 64u + l;
    }
    auto issueTable = [&](Stage &st) {
#pragma unroll
      for (int j = 0; j < 2 * RT; ++j) st.a[j] = load128<0>(values[j / 2], share[j % 2]);
#pragma unroll
      for (int q = 0; q < kSumShare; ++q)
        st.sum[q] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(sums, int(sumShare[q]), 0, 0));
      if constexpr (kPairSums) {
#pragma unroll
        for (int q = 0; q < kSumShare; ++q)
          st.second[q] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(sums, int(sumShare[q] + 64u), 0, 0));
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) share[j] += 8192u;
      // Sums past the range are the next range's or, past the table, zeros: staged and never used.
#pragma unroll
      for (int q = 0; q < kSumShare; ++q) sumShare[q] += kSumsPerBlock * 4u * 16u * 4u * (kPairSums ? 2u : 1u);
    };
    auto issueWeights = [&](Stage &st) {
      load_record(st.rec, weights, mine, column);
      mine += kRecord;
      column += kRecord;
    };
    auto issue = [&](Stage &st) {
      issueTable(st);
      issueWeights(st);
    };
    // Every row's inverse RMS from the squares the table's writer left, one entry a 64-column group:
    // part q of 16 adds entries q, q + 16, ... in order, then the 16 parts are added in order -- the same
    // sums whatever the kernel's row tiles, so a row's result does not depend on the block's height. A
    // thread takes RT parts of its row. The loads go out before the first weights', so the wait for
    // them leaves those in flight.
    constexpr uint32_t kRows = 16u * RT, kParts = 16u, kThreadParts = 256u / kRows;
    // Eight entries of a part are loaded together and added in their order afterwards, so a part costs one round trip
    // to the cache, not one an entry; the first eight go out before the first weights and are added once those are
    // on their way. The squares are read through a resource of their own: an entry past the table's, a row past its
    // rows and every entry of a table without a deferred scale read as zero without touching memory (a squares entry
    // is a sum of squares: adding 0 changes nothing).
    constexpr uint32_t kChunk = 8u;
    float squareSum[RT], loaded[RT][kChunk];
#pragma unroll
    for (int i = 0; i < RT; ++i) squareSum[i] = 0.f;
    const uint32_t squareRow = threadIdx.x % kRows, squareEntries = p.input_size / 64u, squareStride = gguf_squares_stride(tiles) * 4u;
    const Resource squares = make_resource(table + gguf_table_squares_offset(p.input_size, tiles),
                                           p.deferred_scale && squareRow < 16u * tiles ? squareEntries * squareStride : 0u);
    auto loadSquares = [&](int i, uint32_t base) {
#pragma unroll
      for (uint32_t e = 0; e < kChunk; ++e)
        loaded[i][e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(squares, int((base + kParts * e) * squareStride + squareRow * 4u), 0, 0));
    };
    auto addSquares = [&](int i) {
#pragma unroll
      for (uint32_t e = 0; e < kChunk; ++e) squareSum[i] += loaded[i][e];
    };
    if constexpr (Chain) {
      // The first stages' weights go out, then the wait for the link before, then what that link wrote.
#pragma unroll
      for (int s = 0; s < kStages - 1; ++s) {
        issueWeights(stage[s]);
        __builtin_amdgcn_sched_barrier(0);
      }
      chain_wait(chain);
#pragma unroll
      for (int i = 0; i < RT; ++i) loadSquares(i, threadIdx.x / kRows + kThreadParts * i);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < kStages - 1; ++s) {
        issueTable(stage[s]);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
#pragma unroll
      for (int i = 0; i < RT; ++i) loadSquares(i, threadIdx.x / kRows + kThreadParts * i);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < kStages - 1; ++s) {
        issue(stage[s]);
        // Keep the stages' loads in issue order: the loop's counted waits assume it on entry too.
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int i = 0; i < RT; ++i) {
      addSquares(i);
      // a wider table: the part's further entries, eight at a time (these waits do reach the weights')
      if (p.deferred_scale)
        for (uint32_t base = threadIdx.x / kRows + kThreadParts * i + kParts * kChunk; base < squareEntries; base += kParts * kChunk) {
          loadSquares(i, base);
          addSquares(i);
        }
    }
    if (p.deferred_scale) {
#pragma unroll
      for (int i = 0; i < RT; ++i) scaleParts[256u * i + threadIdx.x] = squareSum[i];   // part (threadIdx.x / kRows + kThreadParts i) of row threadIdx.x % kRows
      __syncthreads();
      if (threadIdx.x < kRows) {
        float total = 0.f;
        for (uint32_t q = 0; q < kParts; ++q) total += scaleParts[q * kRows + threadIdx.x];
        rowScale[threadIdx.x] = 1.0f / sqrtf(total / float(p.input_size) + 1e-6f);
      }
      __syncthreads();
    }
    const uint32_t rounds = (count + kStages - 1) / kStages;
    uint32_t now = 0;
    for (uint32_t round = 0; round < rounds; ++round) {
#pragma unroll
      for (int u = 0; u < kStages; ++u, ++now) {
        const uint32_t buffer = DecodeShared<RT>::kBuffers == 2 ? (now & 1u) : 0u;
#pragma unroll
        for (int j = 0; j < 2 * RT; ++j) (&ldsA[buffer][0][0][0])[threadIdx.x + 256u * j] = stage[u].a[j];
#pragma unroll
        for (int q = 0; q < kSumShare; ++q)
          (&ldsSums[buffer][0][0][0])[sumSlot[q]] = kPairSums ? stage[u].sum[q] + stage[u].second[q] : stage[u].sum[q];
        __syncthreads();
        issue(stage[(u + kStages - 1) % kStages]);
        if (now < count) {
          if constexpr (Staged) accumulate_record_staged<FMT, RT>(stage[u].rec, ldsA[buffer], acc, lane, kq);
          else accumulate_record<FMT, RT>(stage[u].rec, ldsA[buffer], ldsSums[buffer], acc, lane, kq);
        }
        if constexpr (DecodeShared<RT>::kBuffers == 1) __syncthreads();   // every wave has read the buffer before the next super-block lands in it
      }
    }
  }

  // The sum of a unit's parts in part order; the loads of a round are in flight together (the loop's staging registers
  // are free by now), so the sum costs one or two round trips to the coherence point whatever the parts.
  auto orderedSum = [&](const float *from, size_t stride, uint32_t parts) {
    constexpr uint32_t kRound = RT == 1 ? 16u : RT == 2 ? 8u : 4u;
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[t][v] = 0.f;
    for (uint32_t s0 = 0; s0 < parts; s0 += kRound) {
      float part[kRound][RT][4];
#pragma unroll
      for (uint32_t s = 0; s < kRound; ++s) {
        if (s0 + s < parts) {
#pragma unroll
          for (int t = 0; t < RT; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v)
              part[s][t][v] = __hip_atomic_load(from + size_t(s0 + s) * stride + (t * 4 + v) * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
#pragma unroll
          for (int t = 0; t < RT; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) part[s][t][v] = 0.f;
        }
      }
#pragma unroll
      for (uint32_t s = 0; s < kRound; ++s)
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
          for (int v = 0; v < 4; ++v) acc[t][v] += s0 + s < parts ? part[s][t][v] : 0.f;
    }
  };
  // Element (t, v) of this lane is row 16 t + 4 kq + v, column tile.column + c.
  if constexpr (EP == GGUF_EPILOGUE_QKV_PREPARE) {
    // A head's columns lie in one or two workgroups (64 columns each) times `splits` parts of K: every one of them leaves
    // its sums as partials and counts itself in on the head's counter, and the last to arrive sums each column tile's
    // parts in part order (the sums of the plain projection), writes the packed rows and runs the head's norms, RoPE
    // and cache store on them.
    const AttentionParams &a = *prepare->attention;
    const uint32_t halves = a.head_dim / 64u, headOf = group / halves;
    const size_t stride = size_t((p.units + 3u) / 4u) * 4u * RT * 256u;
    float *mineAt = partials + (size_t(unit) * RT * 4u) * 64u + lane;
    if (live) {
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v)
          __hip_atomic_store(mineAt + size_t(split) * stride + (t * 4 + v) * 64, acc[t][v], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x == 0) arrived = __hip_atomic_fetch_add(counters + headOf, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (arrived != halves * splits - 1u) return;
    if (threadIdx.x == 0) __hip_atomic_store(counters + headOf, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // the staging buffers are free: the head's rows as floats, then a row a wave for the RoPE exchange
    float (*headRows)[128] = reinterpret_cast<float (*)[128]>(&ldsA[0][0][0][0]);
    float (*waveRows)[4][128] = reinterpret_cast<float (*)[4][128]>(reinterpret_cast<char *>(&ldsA[0][0][0][0]) + 16u * RT * 128u * 4u);
    static_assert(sizeof(shared.a) + (RT > 2 ? sizeof(shared.spare) : 0u) >= 16u * RT * 128u * 4u + 4u * 4u * 128u * 4u,
                  "the staging buffers hold a head's rows and a wave's four");
    const uint8_t *const seg[3] = {seg0, seg1, seg2};
    const uint32_t firstColumn = uint32_t(__builtin_amdgcn_readfirstlane(int(find_tile(headOf * halves * 4u, seg, p, kRecord).column)));
    const uint32_t rows = min(p.rows, 16u * RT);
    // what the first rows need from memory, in flight with the sums' own loads
    const QkvHead head = qkv_head(firstColumn / a.head_dim, *prepare);
    QkvRowAhead ahead[4];
    qkv_rows_ahead(ahead, head, 0u, rows, *prepare);
    // A head of two halves at one row tile and up to eight parts: both halves' parts in flight together.
    constexpr uint32_t kBoth = RT == 1 ? 8u : 0u;
    float sums[2][RT][4];
    if (kBoth && halves == 2u && splits <= kBoth) {
      float part[2][kBoth ? kBoth : 1u][4];
#pragma unroll
      for (uint32_t half = 0; half < 2u; ++half) {
        const float *from = partials + (size_t((headOf * 2u + half) * 4u + wave) * RT * 4u) * 64u + lane;
#pragma unroll
        for (uint32_t s = 0; s < kBoth; ++s)
#pragma unroll
          for (int v = 0; v < 4; ++v)
            part[half][s][v] = s < splits ? __hip_atomic_load(from + size_t(s) * stride + v * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.f;
      }
#pragma unroll
      for (uint32_t half = 0; half < 2u; ++half)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          float total = 0.f;
#pragma unroll
          for (uint32_t s = 0; s < kBoth; ++s) total += s < splits ? part[half][s][v] : 0.f;
          sums[half][0][v] = total;
        }
    } else {
#pragma unroll
      for (uint32_t half = 0; half < 2u; ++half) {
        if (half >= halves) break;
        orderedSum(partials + (size_t((headOf * halves + half) * 4u + wave) * RT * 4u) * 64u + lane, stride, splits);
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
          for (int v = 0; v < 4; ++v) sums[half][t][v] = acc[t][v];
      }
    }
#pragma unroll
    for (uint32_t half = 0; half < 2u; ++half) {
      if (half >= halves) break;
      const uint32_t column = find_tile((headOf * halves + half) * 4u + wave, seg, p, kRecord).column;
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const uint32_t row = 16u * t + 4u * kq + v;
          if (row >= p.rows) continue;
          const float sum = p.deferred_scale ? sums[half][t][v] * rowScale[row] : sums[half][t][v];
          const uint32_t bits = float_to_bf16_bits(sum);
          static_cast<uint16_t *>(out)[size_t(row) * p.out_stride + column + c] = uint16_t(bits);
          headRows[row][half * 64u + 16u * wave + c] = bf16_bits_to_float(bits);
        }
    }
    __syncthreads();
    for (uint32_t first = 0; first < rows; first += 16u) {
      if (first) qkv_rows_ahead(ahead, head, first, rows, *prepare);
      // everything fetched ahead has arrived before the first store leaves: no later wait counts stores
      __builtin_amdgcn_s_waitcnt(0);
      qkv_prepare_rows(headRows, waveRows, ahead, head, first, *prepare);
    }
    qkv_clear_rows(head, *prepare);
    return;
  }
  if (splits > 1) {
    // Partials [split][partitioned unit][t][v][lane]: whole-wave contiguous stores and loads.
    const uint32_t partitioned = (p.units + 3u) / 4u - p.whole_groups;  // workgroups
    const size_t stride = size_t(partitioned) * 4u * RT * 256u;
    float *mineAt = partials + (size_t(unit - 4u * p.whole_groups) * RT * 4u) * 64u + lane;
    uint32_t *counter = counters + (group - p.whole_groups);
    if (live) {
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v)
          __hip_atomic_store(mineAt + size_t(split) * stride + (t * 4 + v) * 64, acc[t][v], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // The partials are written and read with agent-scope atomics, which go to the coherence
    // point instead of a compute die's own L2, so no cache write-back or invalidate is needed: the
    // workgroup only waits for its stores to complete before it counts itself in.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x == 0) arrived = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (arrived != splits - 1) return;
    orderedSum(mineAt, stride, splits);
    if (threadIdx.x == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (p.deferred_scale) {
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[t][v] *= rowScale[16u * t + 4u * kq + v];
  }

  if constexpr (kGateUp) {
    // The up wave hands its sums to the gate wave beside it through LDS (the staging buffers are free).
    float *exchange = reinterpret_cast<float *>(&ldsA[0][0][0][0]);
    __syncthreads();
    if (wave & 1u) {
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) exchange[((wave >> 1) * RT * 4u + t * 4 + v) * 64u + lane] = acc[t][v];
    }
    __syncthreads();
    // With the table epilogue the workgroup's 32 columns, one group of the next projection's
    // inputs, also leave as that projection's activation table (abi/Gguf.h), as gguf_prepare_table
    // would write them: tileOut[half][row tile][row][column] collects the bf16 results.
    uint16_t *tileOut = reinterpret_cast<uint16_t *>(exchange + 2u * RT * 256u);
    float *halfSums = reinterpret_cast<float *>(tileOut + 2u * RT * 256u);
    const uint32_t half = wave >> 1;
    if (!(wave & 1u)) {
      uint16_t *o = static_cast<uint16_t *>(out);
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const uint32_t row = 16u * t + 4u * kq + v;
          uint32_t bits = 0;
          if (live && row < p.rows) {
            const float gate = round_bf16(acc[t][v]), up = round_bf16(exchange[(half * RT * 4u + t * 4 + v) * 64u + lane]);
            bits = float_to_bf16_bits(up * silu(gate));
            o[size_t(row) * p.out_stride + tile.column + c] = uint16_t(bits);
          }
          if constexpr (kTable) tileOut[((half * RT + t) * 16u + 4u * kq + v) * 16u + c] = uint16_t(bits);
        }
    }
    if constexpr (kTable) {
      __syncthreads();
      uint8_t *next = reinterpret_cast<uint8_t *>(const_cast<uint16_t *>(residual));
      const uint32_t G2 = p.out_stride / 32u, g = group;
      uint64_t *values = reinterpret_cast<uint64_t *>(next);
      float *sums32 = reinterpret_cast<float *>(next + gguf_table_sums32_offset(p.out_stride, tiles));
      float *sums16 = reinterpret_cast<float *>(next + gguf_table_sums16_offset(p.out_stride, tiles));
      // Piece (t, half, kq, r): inputs 16 half + 4 kq .. + 3 of row 16 t + r; a wave holds one (t, half).
      for (uint32_t piece = threadIdx.x; piece < 2u * RT * 64u; piece += 256u) {
        const uint32_t r = piece & 15u, q4 = (piece >> 4) & 3u, h2 = (piece >> 6) & 1u, t2 = piece >> 7;
        if (t2 >= tiles) continue;  // a whole wave: the kernel's row tiles past the table's
        const uint2 raw = *reinterpret_cast<const uint2 *>(&tileOut[((h2 * RT + t2) * 16u + r) * 16u + 4u * q4]);
        const uint32_t x0 = raw.x & 0xFFFFu, x1 = raw.x >> 16, x2 = raw.y & 0xFFFFu, x3 = raw.y >> 16;
        store_result<Chain>(&values[((size_t(t2) * G2 + g) * 64u + q4 * 16u + r) * 2u + h2],
                            uint64_t(x0 | (x2 << 16)) | uint64_t(x1 | (x3 << 16)) << 32);
        const float run = (bf16_bits_to_float(x0) + bf16_bits_to_float(x1)) + (bf16_bits_to_float(x2) + bf16_bits_to_float(x3));
        const float r0 = __shfl(run, int(r), 64), r1 = __shfl(run, int(r) + 16, 64), r2 = __shfl(run, int(r) + 32, 64),
                    r3 = __shfl(run, int(r) + 48, 64);
        const float sum = ((r0 + r1) + r2) + r3;
        if (q4 == 0) {
          store_result<Chain>(&sums16[(size_t(t2) * 2u * G2 + 2u * g + h2) * 16u + r], sum);
          halfSums[(t2 * 2u + h2) * 16u + r] = sum;
        }
      }
      __syncthreads();
      if (threadIdx.x < tiles * 16u) {
        const uint32_t t2 = threadIdx.x >> 4, r = threadIdx.x & 15u;
        store_result<Chain>(&sums32[(size_t(t2) * G2 + g) * 16u + r], halfSums[(t2 * 2u) * 16u + r] + halfSums[(t2 * 2u + 1u) * 16u + r]);
      }
    }
  } else if constexpr (EP == GGUF_EPILOGUE_RESIDUAL_NORM) {
    // The residual rows leave as they do without the norm. Their table holds bf16(row * weight):
    // the inverse RMS is left to the projection that reads it, from the sums of squares written here.
    constexpr uint32_t kRows = 16u * RT;
    const uint16_t *normWeight = reinterpret_cast<const uint16_t *>(seg1);
    uint8_t *next = const_cast<uint8_t *>(seg2);
    const bool owns = live && tile.image;
    const float weight = owns ? bf16_bits_to_float(normWeight[tile.column + c]) : 0.f;
    // The staging buffers are free once every wave has left the loop.
    __syncthreads();
    float *waveSquares = reinterpret_cast<float *>(&ldsA[0][0][0][0]);          // [wave][row]
    uint16_t *tileOut = reinterpret_cast<uint16_t *>(waveSquares + 4u * kRows);  // [wave][row tile][row][column]
    float *halfSums = reinterpret_cast<float *>(tileOut + 4u * RT * 256u);       // [row tile][wave][row]
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const uint32_t row = 16u * t + 4u * kq + v;
        float hidden = 0.f;
        uint32_t scaled = 0;
        if (owns && row < p.rows) {
          const size_t at = size_t(row) * p.out_stride + tile.column + c;
          const uint32_t bits = float_to_bf16_bits(acc[t][v] + bf16_bits_to_float(load_result<Chain>(&residual[at])));
          store_result<Chain>(&static_cast<uint16_t *>(out)[at], uint16_t(bits));
          hidden = bf16_bits_to_float(bits);
          scaled = float_to_bf16_bits(hidden * weight);
        }
        tileOut[((wave * RT + t) * 16u + 4u * kq + v) * 16u + c] = uint16_t(scaled);
        // the row's squares over the wave's 16 columns: the 16 lanes of one k quarter, by butterfly
        float sq = hidden * hidden;
#pragma unroll
        for (int o = 1; o < 16; o <<= 1) sq += __shfl_xor(sq, o, 64);
        if (c == 0) waveSquares[wave * kRows + row] = sq;
      }
    __syncthreads();
    if (threadIdx.x < 16u * tiles) {
      const float *w = waveSquares + threadIdx.x;
      float *squares = reinterpret_cast<float *>(next + gguf_table_squares_offset(p.out_stride, tiles));
      store_result<Chain>(&squares[size_t(group) * gguf_squares_stride(tiles) + threadIdx.x], ((w[0] + w[kRows]) + w[2u * kRows]) + w[3u * kRows]);
    }
    // The workgroup's 64 columns: two groups of the next projection's inputs.
    const uint32_t G2 = p.out_stride / 32u;
    uint64_t *values = reinterpret_cast<uint64_t *>(next);
    float *sums32 = reinterpret_cast<float *>(next + gguf_table_sums32_offset(p.out_stride, tiles));
    float *sums16 = reinterpret_cast<float *>(next + gguf_table_sums16_offset(p.out_stride, tiles));
    // Piece (t, w, kq, r): inputs 16 (w % 2) + 4 kq .. + 3 of group 2 group + w / 2, row 16 t + r.
    for (uint32_t piece = threadIdx.x; piece < 4u * RT * 64u; piece += 256u) {
      const uint32_t r = piece & 15u, q4 = (piece >> 4) & 3u, w2 = (piece >> 6) & 3u, t2 = piece >> 8;
      if (t2 >= tiles) continue;  // a whole wave: the kernel's row tiles past the table's
      const uint32_t g2 = 2u * group + (w2 >> 1), h2 = w2 & 1u;
      const uint2 raw = *reinterpret_cast<const uint2 *>(&tileOut[((w2 * RT + t2) * 16u + r) * 16u + 4u * q4]);
      const uint32_t x0 = raw.x & 0xFFFFu, x1 = raw.x >> 16, x2 = raw.y & 0xFFFFu, x3 = raw.y >> 16;
      store_result<Chain>(&values[((size_t(t2) * G2 + g2) * 64u + q4 * 16u + r) * 2u + h2],
                          uint64_t(x0 | (x2 << 16)) | uint64_t(x1 | (x3 << 16)) << 32);
      const float run = (bf16_bits_to_float(x0) + bf16_bits_to_float(x1)) + (bf16_bits_to_float(x2) + bf16_bits_to_float(x3));
      const float r0 = __shfl(run, int(r), 64), r1 = __shfl(run, int(r) + 16, 64), r2 = __shfl(run, int(r) + 32, 64),
                  r3 = __shfl(run, int(r) + 48, 64);
      const float sum = ((r0 + r1) + r2) + r3;
      if (q4 == 0) {
        store_result<Chain>(&sums16[(size_t(t2) * 2u * G2 + 2u * g2 + h2) * 16u + r], sum);
        halfSums[(t2 * 4u + w2) * 16u + r] = sum;
      }
    }
    __syncthreads();
    if (threadIdx.x < tiles * 32u) {
      const uint32_t t2 = threadIdx.x >> 5, pair = (threadIdx.x >> 4) & 1u, r = threadIdx.x & 15u;
      store_result<Chain>(&sums32[(size_t(t2) * G2 + 2u * group + pair) * 16u + r],
                          halfSums[(t2 * 4u + 2u * pair) * 16u + r] + halfSums[(t2 * 4u + 2u * pair + 1u) * 16u + r]);
    }
  } else {
    if (live && tile.image) {
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const uint32_t row = 16u * t + 4u * kq + v;
          if (row >= p.rows) continue;
          const size_t at = size_t(row) * p.out_stride + tile.column + c;
          if constexpr (EP == GGUF_EPILOGUE_PLAIN_F32) static_cast<float *>(out)[at] = acc[t][v];
          else if constexpr (EP == GGUF_EPILOGUE_RESIDUAL)
            store_result<Chain>(&static_cast<uint16_t *>(out)[at],
                                uint16_t(float_to_bf16_bits(acc[t][v] + bf16_bits_to_float(load_result<Chain>(&residual[at])))));
          else static_cast<uint16_t *>(out)[at] = uint16_t(float_to_bf16_bits(acc[t][v]));
        }
    }
  }
  if constexpr (Chain) {
    // The workgroup's results are out (its stores have completed) before it counts itself in; the one that completes
    // the count clears the count it waited for, which every workgroup of this link has passed by then.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x < 64u) {
      uint32_t before = 0;
      if (threadIdx.x == 0) before = __hip_atomic_fetch_add(chain.done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      before = uint32_t(__builtin_amdgcn_readfirstlane(int(before)));
      if (before + 1u == chain.doneTarget) {
        // the link is complete: its count returns to zero (nobody reads it), the next link's workgroups may go, and the
        // flags this link's workgroups waited for are cleared for the next dispatch; a lane a flag
        static_assert(GGUF_CHAIN_FLAGS == 64u, "one wave sets a link's flags");
        if (threadIdx.x == 0) __hip_atomic_store(chain.done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (chain.flags) __hip_atomic_store(chain.flags + threadIdx.x * GGUF_CHAIN_FLAG_STRIDE, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (chain.flagsBefore)
          __hip_atomic_store(chain.flagsBefore + threadIdx.x * GGUF_CHAIN_FLAG_STRIDE, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
}

template <uint32_t FMT, int RT, uint32_t EP, bool Staged = false>
__global__ __launch_bounds__(256, RT > 2 ? 3 : 1) void gguf_decode(const uint8_t *__restrict__ seg0, const uint8_t *__restrict__ seg1,
                                                   const uint8_t *__restrict__ seg2, const uint8_t *__restrict__ table,
                                                   void *__restrict__ out, const uint16_t *__restrict__ residual,
                                                   float *__restrict__ partials, uint32_t *__restrict__ counters,
                                                   GgufDecodeParams p) {
  // Piece blockIdx.y: rows 64 y .. of the dispatch's, with its own table, rows, partials and counters.
  if (const uint32_t piece = blockIdx.y) {
    const uint32_t first = piece * GGUF_MAXIMUM_ROWS, partitioned = (p.units + 3u) / 4u - p.whole_groups;
    const size_t rowBytes = size_t(p.out_stride) * (EP == GGUF_EPILOGUE_PLAIN_F32 ? 4u : 2u);
    table += piece * gguf_table_bytes(p.input_size, GGUF_PIECE_TILES);
    out = static_cast<uint8_t *>(out) + first * rowBytes;
    if constexpr (EP == GGUF_EPILOGUE_GATE_UP_TABLE)
      residual = reinterpret_cast<const uint16_t *>(reinterpret_cast<const uint8_t *>(residual) + piece * gguf_table_bytes(p.out_stride, GGUF_PIECE_TILES));
    else residual += size_t(first) * p.out_stride;
    if constexpr (EP == GGUF_EPILOGUE_RESIDUAL_NORM) seg2 += piece * gguf_table_bytes(p.out_stride, GGUF_PIECE_TILES);
    partials += size_t(piece) * p.splits * partitioned * 4u * RT * 256u;
    counters += piece * partitioned;
    p.rows -= first;
  }
  p.rows = min(p.rows, uint32_t(GGUF_MAXIMUM_ROWS));
  __shared__ DecodeShared<RT> shared;
  decode_workgroup<FMT, RT, EP, false, Staged>(shared, seg0, seg1, seg2, table, out, residual, partials, counters, p, blockIdx.x);
}

// Segments of different formats in one dispatch (the reference's fused projection takes a format per segment,
// gguf_linear.metal:237-261): p.formats names each segment's. Segments hold whole workgroups (multiples of 64
// columns), every workgroup takes one of p.splits parts of K (whole_groups 0), and a workgroup runs its segment's
// format as a projection of that segment alone, its partials and counters after those of the segments before it.
template <int RT>
__global__ __launch_bounds__(256) void gguf_decode_mixed(const uint8_t *__restrict__ seg0, const uint8_t *__restrict__ seg1,
                                                         const uint8_t *__restrict__ seg2, const uint8_t *__restrict__ table,
                                                         void *__restrict__ out, const uint16_t *__restrict__ residual,
                                                         float *__restrict__ partials, uint32_t *__restrict__ counters,
                                                         GgufDecodeParams p) {
  constexpr uint32_t kGroupFloats = 4u * RT * 256u;  // a workgroup's partials of one part
  const uint32_t groups = p.units / 4u;
  if (const uint32_t piece = blockIdx.y) {
    const uint32_t first = piece * GGUF_MAXIMUM_ROWS;
    table += piece * gguf_table_bytes(p.input_size, GGUF_PIECE_TILES);
    out = static_cast<uint8_t *>(out) + size_t(first) * p.out_stride * 2u;
    partials += size_t(piece) * p.splits * groups * kGroupFloats;
    counters += piece * groups;
    p.rows -= first;
  }
  p.rows = min(p.rows, uint32_t(GGUF_MAXIMUM_ROWS));
  const uint32_t group = blockIdx.x / p.splits, split = blockIdx.x % p.splits;
  uint32_t segment = 0, before = 0;
#pragma unroll
  for (uint32_t s = 0; s < 2u; ++s)
    if (segment == s && group >= before + p.cols[s] / 64u) {
      before += p.cols[s] / 64u;
      segment = s + 1u;
    }
  const uint8_t *image = segment == 0 ? seg0 : segment == 1 ? seg1 : seg2;
  auto of = [&](const uint32_t (&field)[3]) { return segment == 0 ? field[0] : segment == 1 ? field[1] : field[2]; };
  const uint32_t format = of(p.formats);
  GgufDecodeParams mine = p;
  mine.cols[0] = of(p.cols);
  mine.cols[1] = mine.cols[2] = 0;
  mine.offset[0] = of(p.offset);
  mine.units = mine.cols[0] / GGUF_TILE_COLUMNS;
  mine.whole_groups = 0;
  partials += size_t(before) * p.splits * kGroupFloats;
  counters += before;
  const uint32_t item = (group - before) * p.splits + split;
  __shared__ DecodeShared<RT> shared;
  switch (format) {
  case GGUF_FMT_Q4K:
    decode_workgroup<GGUF_FMT_Q4K, RT, GGUF_EPILOGUE_PLAIN>(shared, image, image, image, table, out, residual, partials, counters, mine, item);
    break;
  case GGUF_FMT_Q5K:
    decode_workgroup<GGUF_FMT_Q5K, RT, GGUF_EPILOGUE_PLAIN>(shared, image, image, image, table, out, residual, partials, counters, mine, item);
    break;
  case GGUF_FMT_Q6K:
    decode_workgroup<GGUF_FMT_Q6K, RT, GGUF_EPILOGUE_PLAIN>(shared, image, image, image, table, out, residual, partials, counters, mine, item);
    break;
  case GGUF_FMT_Q80:
    decode_workgroup<GGUF_FMT_Q80, RT, GGUF_EPILOGUE_PLAIN>(shared, image, image, image, table, out, residual, partials, counters, mine, item);
    break;
  case GGUF_FMT_IQ4XS:
    decode_workgroup<GGUF_FMT_IQ4XS, RT, GGUF_EPILOGUE_PLAIN>(shared, image, image, image, table, out, residual, partials, counters, mine, item);
    break;
  case GGUF_FMT_IQ4NL:
    decode_workgroup<GGUF_FMT_IQ4NL, RT, GGUF_EPILOGUE_PLAIN>(shared, image, image, image, table, out, residual, partials, counters, mine, item);
    break;
  default: break;
  }
}
SP_REGISTER_KERNEL("gguf_decode_mixed_m16_a", &gguf_decode_mixed<1>);
SP_REGISTER_KERNEL("gguf_decode_mixed_m32_a", &gguf_decode_mixed<2>);
SP_REGISTER_KERNEL("gguf_decode_mixed_m64_a", &gguf_decode_mixed<4>);

// The fused q|k|v projection that also prepares the attention block (GGUF_EPILOGUE_QKV_PREPARE): one format, or a format
// a segment as gguf_decode_mixed. Rows of one piece (up to 64).
#define SP_QKV_PARAMETERS                                                                                                        \
  const uint8_t *__restrict__ seg0, const uint8_t *__restrict__ seg1, const uint8_t *__restrict__ seg2,                          \
      const uint8_t *__restrict__ table, void *__restrict__ out, float *__restrict__ partials, uint32_t *__restrict__ counters,  \
      const uint16_t *__restrict__ query_norm, const uint16_t *__restrict__ key_norm, const float *__restrict__ rope_cos,       \
      const float *__restrict__ rope_sin, _Float16 *__restrict__ queries, float *__restrict__ query_sums,                       \
      const uint64_t *__restrict__ page_table, uint8_t *__restrict__ pool, GgufQkvParams qp
template <uint32_t FMT, int RT> __global__ __launch_bounds__(256) void gguf_decode_qkv(SP_QKV_PARAMETERS) {
  GgufDecodeParams p = qp.decode;
  p.rows = min(p.rows, uint32_t(GGUF_MAXIMUM_ROWS));
  const QkvPrepare prepare{query_norm, key_norm, rope_cos, rope_sin, queries, query_sums, page_table, pool, &qp.attention};
  __shared__ DecodeShared<RT> shared;
  decode_workgroup<FMT, RT, GGUF_EPILOGUE_QKV_PREPARE>(shared, seg0, seg1, seg2, table, out, nullptr, partials, counters, p, blockIdx.x,
                                                       ChainPosition{}, &prepare);
}
template <int RT> __global__ __launch_bounds__(256) void gguf_decode_qkv_mixed(SP_QKV_PARAMETERS) {
  constexpr uint32_t kGroupFloats = 4u * RT * 256u;
  GgufDecodeParams p = qp.decode;
  p.rows = min(p.rows, uint32_t(GGUF_MAXIMUM_ROWS));
  const QkvPrepare prepare{query_norm, key_norm, rope_cos, rope_sin, queries, query_sums, page_table, pool, &qp.attention};
  const uint32_t group = blockIdx.x / p.splits, split = blockIdx.x % p.splits;
  uint32_t segment = 0, before = 0;
#pragma unroll
  for (uint32_t s = 0; s < 2u; ++s)
    if (segment == s && group >= before + p.cols[s] / 64u) {
      before += p.cols[s] / 64u;
      segment = s + 1u;
    }
  const uint8_t *image = segment == 0 ? seg0 : segment == 1 ? seg1 : seg2;
  auto of = [&](const uint32_t (&field)[3]) { return segment == 0 ? field[0] : segment == 1 ? field[1] : field[2]; };
  const uint32_t format = of(p.formats);
  GgufDecodeParams mine = p;
  mine.cols[0] = of(p.cols);
  mine.cols[1] = mine.cols[2] = 0;
  mine.offset[0] = of(p.offset);
  mine.units = mine.cols[0] / GGUF_TILE_COLUMNS;
  mine.whole_groups = 0;
  partials += size_t(before) * p.splits * kGroupFloats;
  counters += before;
  const uint32_t item = (group - before) * p.splits + split;
  __shared__ DecodeShared<RT> shared;
#define SP_QKV_FORMAT(F)                                                                                                          \
  case F:                                                                                                                         \
    decode_workgroup<F, RT, GGUF_EPILOGUE_QKV_PREPARE>(shared, image, image, image, table, out, nullptr, partials, counters, mine, item, \
                                                       ChainPosition{}, &prepare);                                                \
    break
  switch (format) {
    SP_QKV_FORMAT(GGUF_FMT_Q4K);
    SP_QKV_FORMAT(GGUF_FMT_Q5K);
    SP_QKV_FORMAT(GGUF_FMT_Q6K);
    SP_QKV_FORMAT(GGUF_FMT_Q80);
    SP_QKV_FORMAT(GGUF_FMT_IQ4XS);
    SP_QKV_FORMAT(GGUF_FMT_IQ4NL);
  default: break;
  }
#undef SP_QKV_FORMAT
}
#undef SP_QKV_PARAMETERS
SP_REGISTER_KERNEL("gguf_decode_qkv_mixed_m16", &gguf_decode_qkv_mixed<1>);
SP_REGISTER_KERNEL("gguf_decode_qkv_mixed_m32", &gguf_decode_qkv_mixed<2>);
SP_REGISTER_KERNEL("gguf_decode_qkv_mixed_m64", &gguf_decode_qkv_mixed<4>);

// A chain of up to four projections in one dispatch (GgufChainParams): link i's workgroups are items
// link[i].first_item .. of the grid, in link order, so the device has started every workgroup of a link before any of
// the next one's, and a workgroup that waits for the link before (ChainPosition) waits only for workgroups that are
// running or done. Each link binds the eight buffers of a gguf_decode dispatch; `progress` (abi/Gguf.h) holds a count
// of finished workgroups per link, a status word that a wait that ran out of polls sets, and each link's go flags.
// A link of several formats is a plain one, as gguf_decode_mixed's. Rows of one piece (up to 64).
template <uint32_t FMT, int RT>
__device__ __forceinline__ void chain_link(DecodeShared<RT> &shared, uint32_t epilogue, const uint8_t *seg0, const uint8_t *seg1,
                                           const uint8_t *seg2, const uint8_t *table, void *out, const uint16_t *residual,
                                           float *partials, uint32_t *counters, const GgufDecodeParams &p, uint32_t item,
                                           const ChainPosition &chain) {
  switch (epilogue) {
  case GGUF_EPILOGUE_PLAIN:
    decode_workgroup<FMT, RT, GGUF_EPILOGUE_PLAIN, true>(shared, seg0, seg1, seg2, table, out, residual, partials, counters, p, item, chain);
    break;
  case GGUF_EPILOGUE_PLAIN_F32:
    decode_workgroup<FMT, RT, GGUF_EPILOGUE_PLAIN_F32, true>(shared, seg0, seg1, seg2, table, out, residual, partials, counters, p, item, chain);
    break;
  case GGUF_EPILOGUE_GATE_UP_TABLE:
    decode_workgroup<FMT, RT, GGUF_EPILOGUE_GATE_UP_TABLE, true>(shared, seg0, seg1, seg2, table, out, residual, partials, counters, p, item, chain);
    break;
  case GGUF_EPILOGUE_RESIDUAL_NORM:
    decode_workgroup<FMT, RT, GGUF_EPILOGUE_RESIDUAL_NORM, true>(shared, seg0, seg1, seg2, table, out, residual, partials, counters, p, item, chain);
    break;
  default: break;
  }
}

#define SP_CHAIN_LINK_PARAMETERS(n)                                                                                              \
  const uint8_t *__restrict__ seg0_##n, const uint8_t *__restrict__ seg1_##n, const uint8_t *__restrict__ seg2_##n,             \
      const uint8_t *__restrict__ table_##n, void *__restrict__ out_##n, const uint16_t *__restrict__ residual_##n,             \
      float *__restrict__ partials_##n, uint32_t *__restrict__ counters_##n
template <int RT>
__global__ __launch_bounds__(256) void gguf_decode_chain(SP_CHAIN_LINK_PARAMETERS(0), SP_CHAIN_LINK_PARAMETERS(1),
                                                         SP_CHAIN_LINK_PARAMETERS(2), SP_CHAIN_LINK_PARAMETERS(3),
                                                         uint32_t *__restrict__ progress, GgufChainParams cp) {
  uint32_t link = 0;
#pragma unroll
  for (uint32_t l = 1; l < GGUF_CHAIN_LINKS; ++l)
    if (l < cp.links && blockIdx.x >= cp.link[l].first_item) link = l;
  auto pick = [&](auto a, auto b, auto c, auto d) { return link == 0 ? a : link == 1 ? b : link == 2 ? c : d; };
  const uint8_t *seg0 = pick(seg0_0, seg0_1, seg0_2, seg0_3), *seg1 = pick(seg1_0, seg1_1, seg1_2, seg1_3);
  const uint8_t *seg2 = pick(seg2_0, seg2_1, seg2_2, seg2_3), *table = pick(table_0, table_1, table_2, table_3);
  void *out = pick(out_0, out_1, out_2, out_3);
  const uint16_t *residual = pick(residual_0, residual_1, residual_2, residual_3);
  float *partials = pick(partials_0, partials_1, partials_2, partials_3);
  uint32_t *counters = pick(counters_0, counters_1, counters_2, counters_3);
  const GgufChainLink &mine = cp.link[link];  // (the parameters lie in constant memory: an indexed scalar load)
  ChainPosition chain;
  auto flagsOf = [&](uint32_t l) { return progress + GGUF_CHAIN_FLAGS_AT + l * GGUF_CHAIN_FLAGS * GGUF_CHAIN_FLAG_STRIDE; };
  chain.flagsBefore = link ? flagsOf(link - 1u) : nullptr;
  chain.wait = link ? chain.flagsBefore + (blockIdx.x % GGUF_CHAIN_FLAGS) * GGUF_CHAIN_FLAG_STRIDE : nullptr;
  chain.done = progress + link;
  chain.doneTarget = mine.groups;
  chain.flags = link + 1u == cp.links ? nullptr : flagsOf(link);
  chain.spinLimit = cp.spin_limit;
  chain.status = progress + GGUF_CHAIN_LINKS;
  GgufDecodeParams p = mine.p;
  p.rows = min(p.rows, uint32_t(GGUF_MAXIMUM_ROWS));
  uint32_t item = blockIdx.x - mine.first_item;
  uint32_t format = mine.format, epilogue = mine.epilogue;
  if (mine.mixed) {
    // as gguf_decode_mixed: the workgroup's segment alone, in that segment's format
    constexpr uint32_t kGroupFloats = 4u * RT * 256u;
    const uint32_t group = item / p.splits, split = item % p.splits;
    uint32_t segment = 0, past = 0;
#pragma unroll
    for (uint32_t s = 0; s < 2u; ++s)
      if (segment == s && group >= past + p.cols[s] / 64u) {
        past += p.cols[s] / 64u;
        segment = s + 1u;
      }
    auto of = [&](const uint32_t (&field)[3]) { return segment == 0 ? field[0] : segment == 1 ? field[1] : field[2]; };
    seg0 = segment == 0 ? seg0 : segment == 1 ? seg1 : seg2;
    format = of(p.formats);
    const uint32_t columns = of(p.cols), offset = of(p.offset);
    p.cols[0] = columns;
    p.cols[1] = p.cols[2] = 0;
    p.offset[0] = offset;
    p.units = columns / GGUF_TILE_COLUMNS;
    p.whole_groups = 0;
    partials += size_t(past) * p.splits * kGroupFloats;
    counters += past;
    item = (group - past) * p.splits + split;
    epilogue = GGUF_EPILOGUE_PLAIN;
  }
  __shared__ DecodeShared<RT> shared;
  switch (format) {
  case GGUF_FMT_Q4K: chain_link<GGUF_FMT_Q4K, RT>(shared, epilogue, seg0, seg1, seg2, table, out, residual, partials, counters, p, item, chain); break;
  case GGUF_FMT_Q5K: chain_link<GGUF_FMT_Q5K, RT>(shared, epilogue, seg0, seg1, seg2, table, out, residual, partials, counters, p, item, chain); break;
  case GGUF_FMT_Q6K: chain_link<GGUF_FMT_Q6K, RT>(shared, epilogue, seg0, seg1, seg2, table, out, residual, partials, counters, p, item, chain); break;
  case GGUF_FMT_Q80: chain_link<GGUF_FMT_Q80, RT>(shared, epilogue, seg0, seg1, seg2, table, out, residual, partials, counters, p, item, chain); break;
  case GGUF_FMT_IQ4XS: chain_link<GGUF_FMT_IQ4XS, RT>(shared, epilogue, seg0, seg1, seg2, table, out, residual, partials, counters, p, item, chain); break;
  case GGUF_FMT_IQ4NL: chain_link<GGUF_FMT_IQ4NL, RT>(shared, epilogue, seg0, seg1, seg2, table, out, residual, partials, counters, p, item, chain); break;
  default: break;
  }
}
#undef SP_CHAIN_LINK_PARAMETERS
SP_REGISTER_KERNEL("gguf_decode_chain_m16", &gguf_decode_chain<1>);
SP_REGISTER_KERNEL("gguf_decode_chain_m32", &gguf_decode_chain<2>);
SP_REGISTER_KERNEL("gguf_decode_chain_m64", &gguf_decode_chain<4>);

// The routed experts of a mixture-of-experts layer (the reference's moe_expert_gguf_*, abi/MoE.h):
// grid (workgroups of one expert projection, tile slots). Tile t holds up to 16 rows routed to
// expert tile_expert[t]; it reads that expert's image (expert_bytes apart in each bound tensor), its
// own activation table (table_bytes apart) and writes its own 16 output rows (and, with the table
// epilogue, its own next table). Slots at or past tile_total[0] are empty.
template <uint32_t FMT, uint32_t EP>
__global__ __launch_bounds__(256) void gguf_moe_decode(const uint8_t *__restrict__ seg0, const uint8_t *__restrict__ seg1,
                                                       const uint8_t *__restrict__ tables, uint8_t *__restrict__ out,
                                                       uint8_t *__restrict__ next_tables, const uint32_t *__restrict__ tile_expert,
                                                       const uint32_t *__restrict__ tile_rows, const uint32_t *__restrict__ tile_total,
                                                       GgufMoeParams m) {
  const uint32_t tile = blockIdx.y;
  if (tile >= tile_total[0]) return;
  const uint32_t expert = tile_expert[tile];
  GgufDecodeParams p = m.decode;
  p.rows = tile_rows[tile];
  __shared__ DecodeShared<1> shared;
  decode_workgroup<FMT, 1, EP>(shared, seg0 + expert * m.expert_bytes, seg1 + expert * m.expert_bytes, seg0 + expert * m.expert_bytes,
                               tables + tile * m.table_bytes, out + size_t(tile) * 16u * m.out_row_bytes,
                               reinterpret_cast<const uint16_t *>(next_tables + tile * m.next_table_bytes), nullptr, nullptr, p,
                               blockIdx.x);
}
// Every image format serves the experts' one-pass gate/up (_gt) and their down projection (_a).
#define SP_GGUF_MOE_DECODE(fmt, FMT)                                                                                  \
  SP_REGISTER_KERNEL("gguf_moe_decode_" fmt "_gt", (&gguf_moe_decode<FMT, GGUF_EPILOGUE_GATE_UP_TABLE>));             \
  SP_REGISTER_KERNEL("gguf_moe_decode_" fmt "_a", (&gguf_moe_decode<FMT, GGUF_EPILOGUE_PLAIN>))
SP_GGUF_MOE_DECODE("q4k", GGUF_FMT_Q4K);
SP_GGUF_MOE_DECODE("q6k", GGUF_FMT_Q6K);
SP_GGUF_MOE_DECODE("q5k", GGUF_FMT_Q5K);
SP_GGUF_MOE_DECODE("q80", GGUF_FMT_Q80);
SP_GGUF_MOE_DECODE("iq4xs", GGUF_FMT_IQ4XS);
SP_GGUF_MOE_DECODE("iq4nl", GGUF_FMT_IQ4NL);

#define SP_GGUF_DECODE(fmt, FMT, rows, RT)                                                              \
  SP_REGISTER_KERNEL("gguf_decode_" fmt "_m" #rows "_a", &gguf_decode<FMT, RT, GGUF_EPILOGUE_PLAIN>);   \
  SP_REGISTER_KERNEL("gguf_decode_" fmt "_m" #rows "_a_f32", &gguf_decode<FMT, RT, GGUF_EPILOGUE_PLAIN_F32>); \
  SP_REGISTER_KERNEL("gguf_decode_" fmt "_m" #rows "_r", &gguf_decode<FMT, RT, GGUF_EPILOGUE_RESIDUAL>); \
  SP_REGISTER_KERNEL("gguf_decode_" fmt "_m" #rows "_g", &gguf_decode<FMT, RT, GGUF_EPILOGUE_GATE_UP>);  \
  SP_REGISTER_KERNEL("gguf_decode_" fmt "_m" #rows "_gt", &gguf_decode<FMT, RT, GGUF_EPILOGUE_GATE_UP_TABLE>); \
  SP_REGISTER_KERNEL("gguf_decode_" fmt "_m" #rows "_rn", &gguf_decode<FMT, RT, GGUF_EPILOGUE_RESIDUAL_NORM>);                             \
  SP_REGISTER_KERNEL("gguf_decode_qkv_" fmt "_m" #rows, &gguf_decode_qkv<FMT, RT>);                     \
  SP_REGISTER_KERNEL("gguf_staged_" fmt "_m" #rows "_a", &gguf_decode<FMT, RT, GGUF_EPILOGUE_PLAIN, true>); \
  SP_REGISTER_KERNEL("gguf_staged_" fmt "_m" #rows "_a_f32", &gguf_decode<FMT, RT, GGUF_EPILOGUE_PLAIN_F32, true>); \
  SP_REGISTER_KERNEL("gguf_staged_" fmt "_m" #rows "_r", &gguf_decode<FMT, RT, GGUF_EPILOGUE_RESIDUAL, true>)
SP_GGUF_DECODE("q4k", GGUF_FMT_Q4K, 16, 1);
SP_GGUF_DECODE("q4k", GGUF_FMT_Q4K, 32, 2);
SP_GGUF_DECODE("q4k", GGUF_FMT_Q4K, 64, 4);
SP_GGUF_DECODE("q6k", GGUF_FMT_Q6K, 16, 1);
SP_GGUF_DECODE("q6k", GGUF_FMT_Q6K, 32, 2);
SP_GGUF_DECODE("q6k", GGUF_FMT_Q6K, 64, 4);
SP_GGUF_DECODE("q5k", GGUF_FMT_Q5K, 16, 1);
SP_GGUF_DECODE("q5k", GGUF_FMT_Q5K, 32, 2);
SP_GGUF_DECODE("q5k", GGUF_FMT_Q5K, 64, 4);
SP_GGUF_DECODE("q80", GGUF_FMT_Q80, 16, 1);
SP_GGUF_DECODE("q80", GGUF_FMT_Q80, 32, 2);
SP_GGUF_DECODE("q80", GGUF_FMT_Q80, 64, 4);
SP_GGUF_DECODE("iq4xs", GGUF_FMT_IQ4XS, 16, 1);
SP_GGUF_DECODE("iq4xs", GGUF_FMT_IQ4XS, 32, 2);
SP_GGUF_DECODE("iq4xs", GGUF_FMT_IQ4XS, 64, 4);
SP_GGUF_DECODE("iq4nl", GGUF_FMT_IQ4NL, 16, 1);
SP_GGUF_DECODE("iq4nl", GGUF_FMT_IQ4NL, 32, 2);
SP_GGUF_DECODE("iq4nl", GGUF_FMT_IQ4NL, 64, 4);

// ---------------------------------------------------------------------------------------------
// gguf_column_<fmt>_{a,a_f32,r,g}: one or two rows under the reference's column rule (kernels/common/gguf_column_tile.h:25-68,
// kernels/decode/linear_gguf_column.metal:33-66), whose every addition is ordered, so the results are the reference's
// bit for bit: each weight rounded once to half (the staged rule's), a group's 32 products with the row added one after
// the other in input order (each product exact in fp32), the group's sum added to the sum of its part of K, the eight
// parts -- groups [s G / 8, (s + 1) G / 8) of G = K / 32 -- added in order, then the epilogue.
// A workgroup (512 threads) owns one 16-column tile; wave s sums part s. A wave decodes a record in the image's lane
// order (lane (c, kq) holds inputs gguf_operand_input(kq, 0..7) of each group of column c), lays the halves out in LDS
// by input, and lane (c, q) then runs the chains of groups 2 q and 2 q + 1 of column c; the part's running sum passes
// from q to q + 1 (and from 3 to the next record's 0), so groups are added in order. The rows are read as they are
// (bf16 [rows][K]): no activation table. Grid (the tensor's column tiles); of a one-pass gate/up, a workgroup sums
// tile t of both tensors.
// ---------------------------------------------------------------------------------------------
constexpr uint32_t kColumnParts = 8u;       // the reference's GGUF_COLUMN_SPLITS
constexpr uint32_t kColumnStride = 8u * 32u + 8u;  // halves of a column's record in LDS: eight groups and a pad against bank conflicts
struct ColumnShared {
  _Float16 weights[kColumnParts][16][kColumnStride];
  float parts[kColumnParts][2][GGUF_COLUMN_ROWS][16];
};
template <uint32_t FMT, uint32_t EP>
__global__ __launch_bounds__(512, 4) void gguf_column(const uint8_t *__restrict__ image, const uint8_t *__restrict__ upImage,
                                                        const uint16_t *__restrict__ input, void *__restrict__ out,
                                                        const uint16_t *__restrict__ residual, GgufColumnParams p) {
  constexpr bool kGateUp = EP == GGUF_EPILOGUE_GATE_UP;
  constexpr uint32_t kTensors = kGateUp ? 2u : 1u, kRecord = gguf_record_bytes(FMT);
  __shared__ ColumnShared shared;
  const uint32_t lane = threadIdx.x & 63u, part = threadIdx.x >> 6, c = lane & 15u, kq = lane >> 4;
  const uint32_t blocks = p.input_size / GGUF_BLOCK, G = p.input_size / 32u;
  const uint32_t first = uint32_t(__builtin_amdgcn_readfirstlane(int(part * G / kColumnParts)));
  const uint32_t last = uint32_t(__builtin_amdgcn_readfirstlane(int((part + 1u) * G / kColumnParts)));
  float running[kTensors][GGUF_COLUMN_ROWS];
#pragma unroll
  for (uint32_t t = 0; t < kTensors; ++t)
#pragma unroll
    for (uint32_t r = 0; r < GGUF_COLUMN_ROWS; ++r) running[t][r] = 0.f;
  _Float16 (*mine)[kColumnStride] = shared.weights[part];
  for (uint32_t b = first / 8u; 8u * b < last; ++b) {
#pragma unroll
    for (uint32_t t = 0; t < kTensors; ++t) {
      const uint8_t *tensor = (t ? upImage : image) + (size_t(blockIdx.x) * blocks + b) * kRecord;
      const Resource weights = make_resource(tensor, kRecord);
      Record<FMT> rec;
      load_record(rec, weights, 16u * lane, Cursor<FMT>::kColumnPart + 16u * c);
      uint4 ops[8];
      record_operands(rec, ops);
      const StagedCoefficients<FMT> k(rec);
#pragma unroll
      for (uint32_t g = 0; g < 8; ++g) {
        if (8u * b + g < first || 8u * b + g >= last) continue;   // the whole wave: a group of another part
        float value[8];
        staged_values(rec, k, ops[g], g, value);
        _Float16 h[8];
#pragma unroll
        for (uint32_t e = 0; e < 8; ++e) h[e] = _Float16(value[e]);
        // elements 0..3 are inputs 4 kq + {0, 2, 1, 3}, elements 4..7 those + 16
        typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
        *reinterpret_cast<f16x4 *>(&mine[c][32u * g + 4u * kq]) = f16x4{h[0], h[2], h[1], h[3]};
        *reinterpret_cast<f16x4 *>(&mine[c][32u * g + 16u + 4u * kq]) = f16x4{h[4], h[6], h[5], h[7]};
      }
      // the wave's own writes, read back by its own lanes: no other wave touches this part's rows
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0)
      __builtin_amdgcn_wave_barrier();
      float chain[2][GGUF_COLUMN_ROWS];
      bool active[2];
#pragma unroll
      for (uint32_t j = 0; j < 2; ++j) {
        const uint32_t g = 2u * kq + j, group = 8u * b + g;
        active[j] = group >= first && group < last;
#pragma unroll
        for (uint32_t r = 0; r < GGUF_COLUMN_ROWS; ++r) chain[j][r] = 0.f;
        if (!active[j]) continue;
        typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
        f16x8 w[4];
#pragma unroll
        for (uint32_t v = 0; v < 4; ++v) w[v] = *reinterpret_cast<const f16x8 *>(&mine[c][32u * g + 8u * v]);
#pragma unroll
        for (uint32_t r = 0; r < GGUF_COLUMN_ROWS; ++r) {
          if (r >= p.rows) break;
          const uint4 *x = reinterpret_cast<const uint4 *>(input + size_t(r) * p.input_size + 32u * group);
          float sum = 0.f;
#pragma unroll
          for (uint32_t v = 0; v < 4; ++v) {
            const uint4 q = x[v];
            const uint32_t words[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (uint32_t i = 0; i < 8; ++i)
              sum = __fmaf_rn(float(w[v][i]), bf16_bits_to_float((words[i >> 1] >> (16u * (i & 1u))) & 0xFFFFu), sum);
          }
          chain[j][r] = sum;
        }
      }
      // every lane has read the record's halves before the next record's land
      __builtin_amdgcn_wave_barrier();
      // the part's sum so far passes through the lanes of a column in group order
#pragma unroll
      for (uint32_t q = 0; q < 4; ++q) {
#pragma unroll
        for (uint32_t r = 0; r < GGUF_COLUMN_ROWS; ++r) {
          const float incoming = __shfl(running[t][r], int((lane + 48u) & 63u), 64);
          if (kq == q) {
            float sum = incoming;
            if (active[0]) sum += chain[0][r];
            if (active[1]) sum += chain[1][r];
            running[t][r] = sum;
          }
        }
      }
    }
  }
  if (kq == 3u) {
#pragma unroll
    for (uint32_t t = 0; t < kTensors; ++t)
#pragma unroll
      for (uint32_t r = 0; r < GGUF_COLUMN_ROWS; ++r) shared.parts[part][t][r][c] = running[t][r];
  }
  __syncthreads();
  if (threadIdx.x >= 16u * GGUF_COLUMN_ROWS) return;
  const uint32_t r = threadIdx.x >> 4, column = threadIdx.x & 15u;
  if (r >= p.rows) return;
  float total[kTensors];
#pragma unroll
  for (uint32_t t = 0; t < kTensors; ++t) {
    total[t] = 0.f;
    for (uint32_t s = 0; s < kColumnParts; ++s) total[t] += shared.parts[s][t][r][column];
  }
  const size_t at = size_t(r) * p.out_stride + p.out_offset + 16u * blockIdx.x + column;
  if constexpr (kGateUp)   // the first tensor is the gate's
    static_cast<uint16_t *>(out)[at] = uint16_t(float_to_bf16_bits(round_bf16(total[1]) * silu(round_bf16(total[0]))));
  else if constexpr (EP == GGUF_EPILOGUE_PLAIN_F32) static_cast<float *>(out)[at] = total[0];
  else if constexpr (EP == GGUF_EPILOGUE_RESIDUAL)
    static_cast<uint16_t *>(out)[at] = uint16_t(float_to_bf16_bits(total[0] + bf16_bits_to_float(residual[at])));
  else static_cast<uint16_t *>(out)[at] = uint16_t(float_to_bf16_bits(total[0]));
}
#define SP_GGUF_COLUMN(fmt, FMT)                                                                   \
  SP_REGISTER_KERNEL("gguf_column_" fmt "_a", &gguf_column<FMT, GGUF_EPILOGUE_PLAIN>);             \
  SP_REGISTER_KERNEL("gguf_column_" fmt "_a_f32", &gguf_column<FMT, GGUF_EPILOGUE_PLAIN_F32>);     \
  SP_REGISTER_KERNEL("gguf_column_" fmt "_r", &gguf_column<FMT, GGUF_EPILOGUE_RESIDUAL>);          \
  SP_REGISTER_KERNEL("gguf_column_" fmt "_g", &gguf_column<FMT, GGUF_EPILOGUE_GATE_UP>)
SP_GGUF_COLUMN("q4k", GGUF_FMT_Q4K);
SP_GGUF_COLUMN("q6k", GGUF_FMT_Q6K);
SP_GGUF_COLUMN("q5k", GGUF_FMT_Q5K);
SP_GGUF_COLUMN("q80", GGUF_FMT_Q80);
SP_GGUF_COLUMN("iq4xs", GGUF_FMT_IQ4XS);
SP_GGUF_COLUMN("iq4nl", GGUF_FMT_IQ4NL);

// ---------------------------------------------------------------------------------------------
// gguf_prefill_<fmt>_{a,a_f32,r}: the staged rule over a chunk of many rows (the reference's prefill tile,
// gguf_linear.metal:79-118: a shared stage of dequantized weights, each simdgroup its rows). Here the weights stay in
// registers and the rows pass through LDS: a workgroup owns 128 rows x 128 columns, a wave 32 of the columns (two
// records a super-block) over all of the rows, so an operand of rows read from LDS meets four MFMAs (two records, each
// the half's two bf16 parts). Rows come from the activation tables of their 64-row pieces (gguf_prepare_table), half a
// super-block at a time through two LDS buffers. Grid (columns / 128, ceil(rows / 128)), 256 threads; K whole.
// ---------------------------------------------------------------------------------------------
template <uint32_t FMT, uint32_t EP>
__global__ __launch_bounds__(256, 2) void gguf_prefill(const uint8_t *__restrict__ image, const uint8_t *__restrict__ tables,
                                                       void *__restrict__ out, const uint16_t *__restrict__ residual,
                                                       GgufPrefillParams p) {
  constexpr uint32_t kRecord = gguf_record_bytes(FMT);
  __shared__ uint4 rowsStage[2][8][4][64];   // [buffer][row tile][group of the half][lane]: 64 KiB
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, c = lane & 15u, kq = lane >> 4;
  const uint32_t blocks = p.input_size / GGUF_BLOCK, G = p.input_size / 32u;
  const uint32_t firstTile = blockIdx.y * 8u, totalTiles = (p.rows + 15u) / 16u;
  const uint32_t tilesHere = min(8u, totalTiles - firstTile);
  const uint64_t pieceBytes = gguf_table_bytes(p.input_size, GGUF_PIECE_TILES);
  // this wave's two column tiles
  const uint32_t tile0 = (blockIdx.x * 4u + wave) * 2u;
  Cursor<FMT> cursor[2];
  Record<FMT> rec[2], next[2];
#pragma unroll
  for (uint32_t r = 0; r < 2; ++r) {
    cursor[r].open(image + size_t(tile0 + r) * blocks * kRecord, lane);
    next[r].load(cursor[r]);
  }
  f32x4 acc[2][8];
#pragma unroll
  for (uint32_t r = 0; r < 2; ++r)
#pragma unroll
    for (uint32_t t = 0; t < 8; ++t) acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  // A half super-block of the rows: 8 tiles x 4 groups x 64 lanes of 16 bytes, 8 a thread.
  uint4 held[8];
  auto fetch = [&](uint32_t half) {   // half counts half super-blocks from the start of K
#pragma unroll
    for (uint32_t i = 0; i < 8; ++i) {
      const uint32_t at = threadIdx.x + 256u * i, t = at >> 8, g = (at >> 6) & 3u, l = at & 63u;
      const uint32_t tile = firstTile + t;
      held[i] = make_uint4(0u, 0u, 0u, 0u);
      if (t < tilesHere) {
        const uint4 *values = reinterpret_cast<const uint4 *>(tables + uint64_t(tile / GGUF_PIECE_TILES) * pieceBytes);
        held[i] = values[(size_t(tile % GGUF_PIECE_TILES) * G + half * 4u + g) * 64u + l];
      }
    }
  };
  auto store = [&](uint32_t buffer) {
#pragma unroll
    for (uint32_t i = 0; i < 8; ++i) (&rowsStage[buffer][0][0][0])[threadIdx.x + 256u * i] = held[i];
  };
  const uint32_t halves = 2u * blocks;
  fetch(0);
  store(0);
  __syncthreads();
  for (uint32_t block = 0; block < blocks; ++block) {
    // a new super-block: its records, and the next one's on their way
    uint4 ops[2][8];
#pragma unroll
    for (uint32_t r = 0; r < 2; ++r) {
      rec[r] = next[r];
      cursor[r].advance();
      if (block + 1 < blocks) next[r].load(cursor[r]);
      record_operands(rec[r], ops[r]);
    }
    const StagedCoefficients<FMT> k[2] = {StagedCoefficients<FMT>(rec[0]), StagedCoefficients<FMT>(rec[1])};
#pragma unroll
    for (uint32_t h = 0; h < 2; ++h) {   // the super-block's halves: LDS buffer h
      const uint32_t half = 2u * block + h;
      if (half + 1 < halves) fetch(half + 1);
#pragma unroll
      for (uint32_t r = 0; r < 2; ++r)
#pragma unroll
        for (uint32_t g = 0; g < 4; ++g) {
          bf16x8 high, low;
          staged_group(rec[r], k[r], ops[r][4u * h + g], 4u * h + g, high, low);
#pragma unroll
          for (uint32_t t = 0; t < 8; ++t) {
            if (t >= tilesHere) break;
            const bf16x8 rows = as_bf16x8(rowsStage[h][t][g][lane]);
            acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rows, high, acc[r][t], 0, 0, 0);
            acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rows, low, acc[r][t], 0, 0, 0);
          }
        }
      if (half + 1 < halves) store(h ^ 1u);
      __syncthreads();
    }
  }
  // Element (t, v) of this lane is row 16 (firstTile + t) + 4 kq + v, column 16 (tile0 + r) + c.
#pragma unroll
  for (uint32_t r = 0; r < 2; ++r)
#pragma unroll
    for (uint32_t t = 0; t < 8; ++t)
#pragma unroll
      for (uint32_t v = 0; v < 4; ++v) {
        const uint32_t row = 16u * (firstTile + t) + 4u * kq + v;
        if (row >= p.rows) continue;
        const size_t at = size_t(row) * p.out_stride + p.out_offset + 16u * (tile0 + r) + c;
        if constexpr (EP == GGUF_EPILOGUE_PLAIN_F32) static_cast<float *>(out)[at] = acc[r][t][v];
        else if constexpr (EP == GGUF_EPILOGUE_RESIDUAL)
          static_cast<uint16_t *>(out)[at] = uint16_t(float_to_bf16_bits(acc[r][t][v] + bf16_bits_to_float(residual[at])));
        else static_cast<uint16_t *>(out)[at] = uint16_t(float_to_bf16_bits(acc[r][t][v]));
      }
}
#define SP_GGUF_PREFILL(fmt, FMT)                                                                          \
  SP_REGISTER_KERNEL("gguf_prefill_" fmt "_a", &gguf_prefill<FMT, GGUF_EPILOGUE_PLAIN>);                 \
  SP_REGISTER_KERNEL("gguf_prefill_" fmt "_a_f32", &gguf_prefill<FMT, GGUF_EPILOGUE_PLAIN_F32>);         \
  SP_REGISTER_KERNEL("gguf_prefill_" fmt "_r", &gguf_prefill<FMT, GGUF_EPILOGUE_RESIDUAL>)
SP_GGUF_PREFILL("q4k", GGUF_FMT_Q4K);
SP_GGUF_PREFILL("q6k", GGUF_FMT_Q6K);
SP_GGUF_PREFILL("q5k", GGUF_FMT_Q5K);
SP_GGUF_PREFILL("q80", GGUF_FMT_Q80);
SP_GGUF_PREFILL("iq4xs", GGUF_FMT_IQ4XS);
SP_GGUF_PREFILL("iq4nl", GGUF_FMT_IQ4NL);

} // namespace splash::kernels
