// Quantized projection ABI shared by the host operators and the HIP kernels: the weight image a
// K-quant tensor is re-tiled into at load time, the activation table a projection reads, and the
// parameter structs of the kernels. The counterpart of the reference's runtime/metal/abi/Gguf.h and
// QuantFormat.h, laid out for 64-lane wavefronts and 16x16 MFMA tiles instead of 32-lane
// simdgroups.
//
// Vocabulary: a group is 32 inputs, a super-block 256 (one native K-quant block); a column tile is
// 16 output columns (one MFMA tile); a record is one column tile's bytes of one super-block.
//
// WEIGHT IMAGE  [N / 16][K / 256] records, K fastest, so a wave that walks K reads one contiguous
// stream. Lane l of a wave owns column c = l % 16 and input quarter kq = l / 16 of the tile.
//
//   Q4_K record, 2304 B (16 native blocks of 144 B, byte for byte re-ordered):
//     [   0, 2048)  nibbles: two 1024-B halves h; in half h lane l owns 16 B at 1024 h + 16 l =
//                   native qs bytes  [64 h + 4 kq, +4) [64 h + 16 + 4 kq, +4)
//                                    [64 h + 32 + 4 kq, +4) [64 h + 48 + 4 kq, +4)
//                   i.e. words w0, w1 hold inputs 4 kq + 0..3 and 16 + 4 kq + 0..3 of groups 4 h
//                   (low nibbles) and 4 h + 1 (high nibbles), w2, w3 those of groups 4 h + 2, 4 h + 3.
//     [2048, 2304)  meta: column c's native d, dmin and 12 scale bytes at 2048 + 16 c.
//
//   Q6_K record, 3360 B (16 native blocks of 210 B):
//     [   0, 2048)  low nibbles, arranged exactly as Q4_K's nibbles (code & 15 of the same inputs).
//     [2048, 3072)  high bits: lane l owns 16 B at 2048 + 16 l: word i covers groups 2 i, 2 i + 1;
//                   the 2-bit field of pair v (0..7: operand register v % 4 of group 2 i + v / 4)
//                   sits at bits 2 v (low half's code) and 16 + 2 v (high half's code).
//     [3072, 3328)  scales: column c's 16 int8 scales at 3072 + 16 c.
//     [3328, 3360)  d: column c's fp16 d at 3328 + 2 c.
//
//   Q5_K record, 2816 B (16 native blocks of 176 B):
//     [   0, 2048)  low nibbles, arranged exactly as Q4_K's nibbles.
//     [2048, 2560)  fifth bits: lane l owns 8 B at 2048 + 8 l: word h covers groups 4 h .. 4 h + 3; bit
//                   4 (g % 4) + j is the fifth bit of the low half's code of operand register j of group g,
//                   bit 16 + 4 (g % 4) + j that of its high half's.
//     [2560, 2816)  meta: column c's native d, dmin and 12 scale bytes at 2560 + 16 c (as Q4_K's).
//
//   Q8_0 record, 4352 B (16 columns of eight native 34-B blocks):
//     [   0, 4096)  values: four 1024-B parts; in part i lane l owns 16 B at 1024 i + 16 l: the int8 values of
//                   inputs 4 kq .. 4 kq + 3 and 16 + 4 kq .. + 3 of group 2 i, then those of group 2 i + 1.
//     [4096, 4352)  scales: column c's eight fp16 d (groups 0..7) at 4096 + 16 c.
//   Its operands are the bf16 128 + value (0..255, exact); the 128 leaves as Q4_K's does, through the row sums.
//
//   IQ4_XS record, 2176 B (16 native blocks of 136 B), and IQ4_NL record, 2304 B (16 columns of eight native 18-B blocks):
//     [   0, 2048)  nibbles: two 1024-B halves h; in half h lane l owns 16 B at 1024 h + 16 l, whose word i holds the
//                   lane's eight codes of group 4 h + i as the native bytes do: byte j's low nibble the code of input
//                   4 kq + j, its high nibble that of input 16 + 4 kq + j.
//     [2048, ...)   IQ4_XS: column c's native d, scales_h and four scales_l bytes at 2048 + 8 c;
//                   IQ4_NL: column c's eight fp16 d (groups 0..7) at 2048 + 16 c.
//   A code names a value of the 16-entry codebook (-127 .. 113); the operands are the bf16 128 + value, as Q8_0's.
//
// Within a group, lane (c, kq) holds eight codes as four registers of two bf16 operands
// 128 + code: register j (0..3) holds inputs 16 (j / 2) + 4 kq + (j % 2) [low half] and that + 2
// [high half]. Element e = 2 j + half of the lane's MFMA operand is therefore input
//     gguf_operand_input(kq, e) = 16 (e / 4) + 4 kq + {0, 2, 1, 3}[e % 4]
// of the group, and the activation table stores x in that order.
//
// ACTIVATION TABLE of `tiles` row tiles (16 rows each, rows past the live ones zero) and G = K / 32
// groups: values bf16 [tiles][G][64 lanes][8]: lane (r = l % 16, kq = l / 16) holds inputs
// gguf_operand_input(kq, 0..7) of row 16 t + r; then sums32 fp32 [tiles][G][16 rows] and sums16
// fp32 [tiles][2 G][16 rows], the fp32 sums of each row's 32 and 16 inputs in input order; then
// squares fp32 [K / 64][gguf_squares_stride(tiles)], read only of a table whose rows still lack a per-row scale
// (GgufDecodeParams::deferred_scale): entry (j, r), r < 16 tiles, is the sum of squares of row r's values over
// columns 64 j .. 64 j + 63 of the rows the table was normed from. An entry fills whole 128-byte lines, as a group's
// values and a workgroup's 16-input sums do: each has one writer (the workgroup that owns those columns), which is what
// lets a projection chained behind the writer read them through its cache (gguf_decode_chain).
#pragma once
#include <stdint.h>

#define GGUF_FMT_Q4K 0u
#define GGUF_FMT_IQ4XS 1u
#define GGUF_FMT_IQ4NL 2u
#define GGUF_FMT_Q5K 3u
#define GGUF_FMT_Q6K 4u
#define GGUF_FMT_Q80 6u
#define GGUF_FMT_COUNT 26u

#define GGUF_BLOCK 256u
#define GGUF_TILE_COLUMNS 16u
#define GGUF_Q4K_NATIVE 144u
#define GGUF_Q5K_NATIVE 176u
#define GGUF_Q6K_NATIVE 210u
#define GGUF_Q80_NATIVE 272u  // eight 34-byte blocks: the bytes of 256 inputs
#define GGUF_IQ4XS_NATIVE 136u
#define GGUF_IQ4NL_NATIVE 144u  // eight 18-byte blocks
#define GGUF_IQ4XS_RECORD (GGUF_TILE_COLUMNS * GGUF_IQ4XS_NATIVE)  // 2176
#define GGUF_IQ4NL_RECORD (GGUF_TILE_COLUMNS * GGUF_IQ4NL_NATIVE)  // 2304
#define GGUF_IQ4_SCALES 2048u
#define GGUF_Q4K_RECORD (GGUF_TILE_COLUMNS * GGUF_Q4K_NATIVE)  // 2304
#define GGUF_Q6K_RECORD (GGUF_TILE_COLUMNS * GGUF_Q6K_NATIVE)  // 3360
#define GGUF_Q5K_RECORD (GGUF_TILE_COLUMNS * GGUF_Q5K_NATIVE)  // 2816
#define GGUF_Q80_RECORD (GGUF_TILE_COLUMNS * GGUF_Q80_NATIVE)  // 4352
#define GGUF_Q5K_HIGH 2048u
#define GGUF_Q5K_META 2560u
#define GGUF_Q80_SCALES 4096u
#define GGUF_Q6K_HIGH 2048u
#define GGUF_Q6K_SCALES 3072u
#define GGUF_Q6K_D 3328u
#define GGUF_ROW_TILE 16u
// The most rows one workgroup takes: four lanes of sixteen verify rows. A dispatch of more rows
// (eight lanes) runs pieces of this many rows side by side (grid.y); a piece's activation table,
// output and residual rows, partials and counters follow those of the piece before it.
#define GGUF_MAXIMUM_ROWS 64u
#define GGUF_MAXIMUM_DISPATCH_ROWS 256u
#define GGUF_MAXIMUM_SEGMENTS 3u
#define GGUF_MAXIMUM_SPLITS 16u

#if defined(__HIPCC__) || defined(__cplusplus)
#define GGUF_INLINE constexpr inline
#if defined(__HIPCC__)
#undef GGUF_INLINE
#define GGUF_INLINE __host__ __device__ constexpr inline
#endif

GGUF_INLINE uint32_t gguf_record_bytes(uint32_t format) {
  return format == GGUF_FMT_Q4K   ? GGUF_Q4K_RECORD
         : format == GGUF_FMT_Q6K ? GGUF_Q6K_RECORD
         : format == GGUF_FMT_Q5K ? GGUF_Q5K_RECORD
         : format == GGUF_FMT_Q80 ? GGUF_Q80_RECORD
         : format == GGUF_FMT_IQ4XS ? GGUF_IQ4XS_RECORD
         : format == GGUF_FMT_IQ4NL ? GGUF_IQ4NL_RECORD
                                  : 0u;
}
GGUF_INLINE uint32_t gguf_native_bytes(uint32_t format) {
  return format == GGUF_FMT_Q4K   ? GGUF_Q4K_NATIVE
         : format == GGUF_FMT_Q6K ? GGUF_Q6K_NATIVE
         : format == GGUF_FMT_Q5K ? GGUF_Q5K_NATIVE
         : format == GGUF_FMT_Q80 ? GGUF_Q80_NATIVE
         : format == GGUF_FMT_IQ4XS ? GGUF_IQ4XS_NATIVE
         : format == GGUF_FMT_IQ4NL ? GGUF_IQ4NL_NATIVE
                                  : 0u;
}
// Kernel-name tag of a format.
GGUF_INLINE const char *gguf_format_name(uint32_t format) {
  return format == GGUF_FMT_Q4K     ? "q4k"
         : format == GGUF_FMT_Q6K   ? "q6k"
         : format == GGUF_FMT_Q5K   ? "q5k"
         : format == GGUF_FMT_Q80   ? "q80"
         : format == GGUF_FMT_IQ4XS ? "iq4xs"
         : format == GGUF_FMT_IQ4NL ? "iq4nl"
                                    : "";
}
// Bytes of the image of an [N, K] tensor (N a multiple of 16, K of 256): those of its native rows.
GGUF_INLINE uint64_t gguf_image_bytes(uint32_t format, uint32_t n, uint32_t k) {
  return uint64_t(n / GGUF_TILE_COLUMNS) * (k / GGUF_BLOCK) * gguf_record_bytes(format);
}
GGUF_INLINE uint32_t gguf_operand_input(uint32_t kq, uint32_t e) {
  return 16u * (e >> 2) + 4u * kq + (((e & 1u) << 1) | ((e >> 1) & 1u));
}
GGUF_INLINE uint32_t gguf_row_tiles(uint32_t rows) { return (rows + GGUF_ROW_TILE - 1) / GGUF_ROW_TILE; }
// Activation table geometry, in bytes from the table's start.
GGUF_INLINE uint64_t gguf_table_values_bytes(uint32_t k, uint32_t tiles) { return uint64_t(tiles) * k * 16u * 2u; }
GGUF_INLINE uint64_t gguf_table_sums32_offset(uint32_t k, uint32_t tiles) { return gguf_table_values_bytes(k, tiles); }
GGUF_INLINE uint64_t gguf_table_sums16_offset(uint32_t k, uint32_t tiles) {
  return gguf_table_sums32_offset(k, tiles) + uint64_t(tiles) * (k / 32u) * 16u * 4u;
}
GGUF_INLINE uint64_t gguf_table_squares_offset(uint32_t k, uint32_t tiles) {
  return gguf_table_sums16_offset(k, tiles) + uint64_t(tiles) * (k / 16u) * 16u * 4u;
}
GGUF_INLINE uint32_t gguf_squares_stride(uint32_t tiles) { return tiles < 2u ? 32u : tiles * 16u; }  // floats an entry
GGUF_INLINE uint64_t gguf_table_bytes(uint32_t k, uint32_t tiles) {
  return gguf_table_squares_offset(k, tiles) + uint64_t(k / 64u) * gguf_squares_stride(tiles) * 4u;
}
// Row tiles of a piece, and the tables of `tiles` row tiles in all: whole pieces' tables of four row
// tiles each, then the last piece's (the single table of up to four row tiles is its own case).
#define GGUF_PIECE_TILES (GGUF_MAXIMUM_ROWS / GGUF_ROW_TILE)
GGUF_INLINE uint64_t gguf_tables_bytes(uint32_t k, uint32_t tiles) {
  const uint32_t whole = tiles / GGUF_PIECE_TILES, rest = tiles % GGUF_PIECE_TILES;
  return whole * gguf_table_bytes(k, GGUF_PIECE_TILES) + (rest ? gguf_table_bytes(k, rest) : 0u);
}
#endif

// gguf_prepare_table: bf16 rows [rows][input_size] -> the activation table of `tiles` row tiles.
// Grid (K / 32, tiles), 64 threads.
struct GgufPrepareParams {
  uint32_t input_size;
  uint32_t rows;
  uint32_t tiles;
  uint32_t row_stride;  // elements between input rows
};

// gguf_prefill_<fmt>_{a,a_f32,r}: a chunk of rows under the staged rule. Binds the segment's image, the rows' activation
// tables (64-row pieces one after the other, each gguf_table_bytes(input_size, GGUF_PIECE_TILES) on from the one before),
// out (bf16, or fp32 for _a_f32) and the residual rows (bf16; any buffer when unused). Grid (columns / 128,
// ceil(rows / 128)), 256 threads.
struct GgufPrefillParams {
  uint32_t input_size;
  uint32_t rows;
  uint32_t columns;     // of this segment: a multiple of 128
  uint32_t out_stride;  // elements between output (and residual) rows
  uint32_t out_offset;  // the segment's first output column
  uint32_t reserved[3];
};

// gguf_column_<fmt>_{a,a_f32,r,g}: one or two rows under the reference's column rule (its GgufColumnParams,
// metal/abi/Gguf.h:45-55; GGUF_COLUMN_SPLITS parts of K there and here). Binds the tensor's image, a one-pass gate/up's
// up image (the first is the gate's; the tensor's again otherwise), the rows (bf16 [rows][input_size]), out and the
// residual rows (any buffer when unused). Grid (the tensor's 16-column tiles), 512 threads.
#define GGUF_COLUMN_ROWS 2u
struct GgufColumnParams {
  uint32_t rows;        // 1 to GGUF_COLUMN_ROWS
  uint32_t input_size;
  uint32_t out_stride;  // elements between output (and residual) rows
  uint32_t out_offset;  // the tensor's first output column
  uint32_t reserved[4];
};

// Epilogues of a decode projection (the reference's LinearEpilogue, runtime/ops/Linear.hpp:77).
#define GGUF_EPILOGUE_PLAIN 0u     // out = bf16(v)         kernel suffix _a
#define GGUF_EPILOGUE_PLAIN_F32 1u // out = v               kernel suffix _a_f32
#define GGUF_EPILOGUE_RESIDUAL 2u  // out = bf16(v + res)   kernel suffix _r
#define GGUF_EPILOGUE_GATE_UP 3u   // out = bf16(bf16(up) * silu(bf16(gate)))   kernel suffix _g
// The same, and `out` also leaves as the next projection's activation table, written to the buffer
// bound in the residual's place (columns a multiple of 256): kernel suffix _gt.
#define GGUF_EPILOGUE_GATE_UP_TABLE 4u
// out = bf16(v + res), and those rows leave as the activation table of the projection after their RMS
// norm (the norm's weights bound in the second segment's slot, the table in the third's): kernel
// suffix _rn. A row's inverse RMS needs every column of the row, which no workgroup of the dispatch
// has; so the table holds bf16(out * weight) and, in its squares region, each 64-column group's sums
// of squares of `out`. The projection that reads the table sums them to the row's inverse RMS and
// multiplies its sums by it (deferred_scale): a per-row factor commutes with the projection. One
// tensor, whole super-blocks of output columns.
#define GGUF_EPILOGUE_RESIDUAL_NORM 5u
// out = bf16(v), the fused q|k|v rows, and on them the work of attention_q8_qkv (abi/PagedAttention.h): the q and k heads'
// RMS norms, RoPE, the staged queries and their sums, the block's keys and values quantized into their page slots: kernels
// gguf_decode_qkv_<fmt>_m<rows> and gguf_decode_qkv_mixed_m<rows> (GgufQkvParams). A head's 64 or 128 columns lie in one
// or two workgroups times `splits` parts of K; all of them leave partials and the last to arrive finishes the head, so
// the dispatch keeps partials and counters even unsplit, every workgroup takes a part (whole_groups 0), and the
// segments hold whole heads.
#define GGUF_EPILOGUE_QKV_PREPARE 6u

// gguf_decode_<fmt>_m<16|32|64>_<a|a_f32|r|g>: up to three column segments of one format in one
// dispatch (the reference's GgufDecodeFusedParams, runtime/metal/abi/Gguf.h:168-178), tiles in
// segment order; a single tensor is one segment. A gate/up pair binds gate as segment 0 and up as
// segment 1, both of cols[0] columns. Grid (whole_groups + (groups - whole_groups) * splits), 256 threads: a wave per unit.
// gguf_decode_mixed_m<16|32|64>_a: segments of different formats (formats[]), each whole workgroups
// (multiples of 64 columns), whole_groups 0: grid groups * splits.
struct GgufDecodeParams {
  uint32_t input_size;  // K
  uint32_t rows;        // live rows
  uint32_t splits;      // K partitions of the workgroups past the whole ones; 1 = no cross-workgroup reduction
  uint32_t whole_groups;  // leading workgroups (four units each) that walk all of K; the others take one of `splits` parts
  uint32_t out_stride;  // columns of a destination row
  uint32_t cols[3];     // columns per segment (multiples of 16); 0 past the last
  uint32_t offset[3];   // first destination column per segment
  uint32_t units;       // wave work units: one column tile each (gate/up: gate tile j is unit 2 j, up tile j unit 2 j + 1)
  // Nonzero: the table's rows lack their RMS scale; every sum is multiplied by
  // 1 / sqrt(sum of the row's squares entries / K + 1e-6) before the epilogue.
  uint32_t deferred_scale;
  uint32_t formats[3];  // gguf_decode_mixed_*: each segment's format; the kernels of one format leave it zero
};

// gguf_decode_chain_m<16|32|64>: up to four projections of up to 64 rows in one dispatch, each a gguf_decode (or, with
// `mixed`, a gguf_decode_mixed) dispatch of its own eight buffers, link i + 1 reading what link i's epilogue wrote (the
// next projection's table, the residual rows). Grid: the links' grids one after the other; 256 threads. After the
// links' buffers the kernel binds `progress`, GGUF_CHAIN_PROGRESS_WORDS words that are zero between dispatches:
// GGUF_CHAIN_LINKS counts of finished workgroups; a status word, nonzero once a workgroup's wait for the link before it
// ran out of polls (the results are then not to be used); and from word GGUF_CHAIN_FLAGS_AT each link's GGUF_CHAIN_FLAGS
// go flags, GGUF_CHAIN_FLAG_STRIDE words apart (a flag a 256-byte block, so that the workgroups that wait, each
// polling flag `its index % GGUF_CHAIN_FLAGS`, spread over the memory channels: a word that every waiting workgroup of
// the device polls slows the whole dispatch down). The workgroup that completes a link's count sets that link's flags
// and clears the flags of the link before. Every link has its own table, partials and counters, and no buffer a link
// writes is read earlier in the dispatch.
#define GGUF_CHAIN_LINKS 4u
#define GGUF_CHAIN_FLAGS 64u
#define GGUF_CHAIN_FLAG_STRIDE 64u
#define GGUF_CHAIN_FLAGS_AT 64u
#define GGUF_CHAIN_PROGRESS_WORDS (GGUF_CHAIN_FLAGS_AT + GGUF_CHAIN_LINKS * GGUF_CHAIN_FLAGS * GGUF_CHAIN_FLAG_STRIDE)
struct GgufChainLink {
  struct GgufDecodeParams p;
  uint32_t first_item;  // the link's first workgroup of the dispatch
  uint32_t format;      // GGUF_FMT_* of its segments (the formats of a mixed link are p.formats)
  uint32_t epilogue;    // GGUF_EPILOGUE_PLAIN, _PLAIN_F32, _GATE_UP_TABLE or _RESIDUAL_NORM
  uint32_t mixed;       // nonzero: segments of several formats, plain bf16 rows
  uint32_t groups;      // workgroups that write the link's results: each counts itself in when they are out
  uint32_t reserved[3];
};
struct GgufChainParams {
  uint32_t links;       // 1..GGUF_CHAIN_LINKS
  uint32_t spin_limit;  // polls of a workgroup's wait before it gives up
  uint32_t reserved[2];
  struct GgufChainLink link[GGUF_CHAIN_LINKS];
};

#ifdef ATTENTION_MAXIMUM_SEQUENCES
// gguf_decode_qkv_*: a decode projection's parameters and the attention block's (abi/PagedAttention.h, included first).
// Binds seg0..2, table, out, partials, counters, then the query and key norm weights, the RoPE cosine and sine tables,
// the staged queries and their sums, the page table and the layer's pool, as attention_q8_qkv does.
struct GgufQkvParams {
  struct GgufDecodeParams decode;
  struct AttentionParams attention;
};
#endif

// gguf_dequant_<fmt>: the image's fp32 values [N][K], for the bit-exactness test
// (the reference's gguf_dequant_test.metal). Grid (K / 256, N / 16), 64 threads.
struct GgufDequantParams {
  uint32_t input_size;
  uint32_t output_size;
};

// gguf_embed_<fmt>: out[r][:] = bf16(decode(table row tokens[r])) from NATIVE rows; a token at or
// past the vocabulary gives zeros (the reference's GgufEmbedParams, abi/Gguf.h:180-185).
struct GgufEmbedParams {
  uint32_t rows;
  uint32_t vocabulary;
  uint32_t hidden;
};

#ifdef __cplusplus
static_assert(sizeof(GgufPrepareParams) == 16, "prepare parameters are 16 bytes on both sides");
static_assert(sizeof(GgufDecodeParams) == 64, "decode parameters are 64 bytes on both sides");
static_assert(sizeof(GgufChainLink) == 96 && sizeof(GgufChainParams) == 400, "chain parameters are 400 bytes on both sides");
static_assert(sizeof(GgufDequantParams) == 8, "dequant parameters are 8 bytes on both sides");
static_assert(sizeof(GgufEmbedParams) == 12, "embedding parameters are 12 bytes on both sides");
#endif
