// Parameters of the glue kernels on the verify path: RMS norm, RoPE tables, token embedding
// (the reference's abi/RoPE.h, abi/Embedding.h and the `uint width` of its norm kernels).
#pragma once
#include <stdint.h>

#define SPLASH_RMS_EPSILON 1e-6f

// norm_rms / norm_rms_table16: one workgroup of 256 threads per row. norm_rms_table16 also writes
// the projection activation table of the normalized rows (abi/Gguf.h), as the reference's
// norm_rms_table16_decode does for its register tile.
struct NormParams {
  uint32_t width;
  uint32_t rows;
  uint32_t tiles;  // row tiles of the table (norm_rms_table16)
  uint32_t reserved;
};

// rope_build_tree_tables: cos and sin of (anchor[sequence] + depth[row]) * inverse_frequency[pair]
// per packed row (the reference's RopeTreeParams, abi/RoPE.h). Grid (rows), `pairs` threads.
struct RopeTreeParams {
  uint32_t pairs;
  uint32_t rows;
  uint32_t sequences;
  uint32_t reserved;
  uint32_t first_row[8];  // per sequence
  uint32_t row_count[8];
  uint32_t anchor[8];     // position of the sequence's row 0
};

// copy_rows_bf16: `rows` rows of `width` bf16 values between two row regions (the reference's
// RowCopyParams, abi/RowCopy.h). One thread per value.
struct RowCopyParams {
  uint32_t rows, width;
  uint32_t from_row, from_stride, from_column;
  uint32_t to_row, to_stride, to_column;
};

// swiglu_rows: out = bf16(up * silu(gate)) over `count` bf16 values, eight a thread (the epilogue of the one-pass gate/up
// projection, GGUF_EPILOGUE_GATE_UP, as a pass of its own for rows whose gate and up were projected apart).
struct SwiGluRowsParams {
  uint64_t count;
};

// gguf_float_<f32|bf16>_<f32|bf16>: the fp32 projection of weights kept as rows (the reference's GgufFloatParams,
// abi/Gguf.h:204, kernels/shared/gguf_float.metal): out[r][out_offset + n] = sum_k x[r][k] W[n][k], x the bf16 rows,
// W F32 or BF16 rows as stored, every operand exact in fp32. A sum runs four chains of fused multiply-adds, chain j
// over the inputs k = j mod 4 in ascending order, and adds them as (c0 + c1) + (c2 + c3): it depends neither on the
// grid nor on the row count. Grid (ceil(output_size / 16), ceil(rows / 16)), 256 threads: a thread an output.
#define GGUF_FLOAT_STEP 64u   // inputs a workgroup stages at a time
struct GgufFloatParams {
  uint32_t rows;
  uint32_t input_size;   // K, a multiple of 8
  uint32_t output_size;  // N
  uint32_t out_stride;   // values of a destination row
  uint32_t out_offset;   // the projection's first column in it
  uint32_t reserved[3];
};

#ifdef __cplusplus
static_assert(sizeof(GgufFloatParams) == 32, "float projection parameters are 32 bytes on both sides");
static_assert(sizeof(RowCopyParams) == 32, "row copy parameters are 32 bytes on both sides");
static_assert(sizeof(NormParams) == 16, "norm parameters are 16 bytes on both sides");
static_assert(sizeof(RopeTreeParams) == 112, "RoPE tree parameters are 112 bytes on both sides");
#endif
