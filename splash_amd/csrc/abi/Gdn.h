// Gated DeltaNet verify step: state cells, the decode tape and the kernels' parameters, shared by
// the host operator (ops/Gdn) and the HIP kernels. The counterpart of the reference's
// runtime/metal/abi/GDN.h and runtime/ops/GDN.hpp:16-160.
//
// A packed row of a layer's projection, bf16 [packed_width]:
//   [ q (key_heads * 128) | k (key_heads * 128) | v (value_heads * 128) | z (value_heads * 128) |
//     b (value_heads) | a (value_heads) ]
// The first conv_dim = (2 key_heads + value_heads) * 128 columns pass the short convolution.
//
// A lane's state cell: the convolution carry of every layer (the three rows of conv_dim inputs
// before the next token, bf16, conv_layer_bytes apart), then from convolution_state_bytes every
// layer's recurrent state fp32 [value_heads][128 value dims][128 key dims], recurrent_layer_bytes
// apart. Cells are double-buffered: a step reads `current` and writes `next`.
//
// Rollback is free (the reference's Runtime.cpp:2701-2707): which rows of a step are accepted is
// known only after it, so the state a step writes is the state BEFORE its rows; it leaves every
// row's convolution inputs, k, v and gates on the lane's tape, and the lane's next step first folds
// the accepted path (`pending_path`, a mask of the previous step's rows) into the state.
#pragma once
#include <stdint.h>

#define GDN_CONVOLUTION_TAPS 4u
#define GDN_HEAD_DIMENSION 128u
#define GDN_MAXIMUM_ROWS 16u   // rows of one lane's verify block
#define GDN_MAXIMUM_LANES 8u

// flags
#define GDN_TILED_HEADS 1u   // value head h leaves at (h % heads per key) * key heads + h / heads per key
#define GDN_SIGMOID_GATE 2u  // gate by sigmoid(z) instead of silu(z)
#define GDN_FLOAT_NORM 4u    // the output norm's weights are fp32, not bf16

#if defined(__HIPCC__)
#define GDN_INLINE __host__ __device__ inline
#else
#define GDN_INLINE inline
#endif

// One layer's tape of one lane's step, room for GDN_MAXIMUM_ROWS rows: the rows' convolution
// inputs bf16 [row][conv_dim], their k then v rows bf16 [row][kv_width], decay fp32
// [row][value_heads], beta bf16 [row][value_heads] (the reference's gdn_tape_*, abi/GDN.h:44-67).
GDN_INLINE uint64_t gdn_tape_kv_offset(uint32_t conv_dim) { return uint64_t(GDN_MAXIMUM_ROWS) * conv_dim * 2; }
GDN_INLINE uint64_t gdn_tape_decay_offset(uint32_t conv_dim, uint32_t kv_width) {
  return gdn_tape_kv_offset(conv_dim) + uint64_t(GDN_MAXIMUM_ROWS) * kv_width * 2;
}
GDN_INLINE uint64_t gdn_tape_beta_offset(uint32_t conv_dim, uint32_t kv_width, uint32_t value_heads) {
  return gdn_tape_decay_offset(conv_dim, kv_width) + uint64_t(GDN_MAXIMUM_ROWS) * value_heads * 4;
}
GDN_INLINE uint64_t gdn_tape_layer_bytes(uint32_t conv_dim, uint32_t kv_width, uint32_t value_heads) {
  return (gdn_tape_beta_offset(conv_dim, kv_width, value_heads) + uint64_t(GDN_MAXIMUM_ROWS) * value_heads * 2 + 15) / 16 * 16;
}

struct GdnShapeParams {
  uint32_t key_heads, value_heads;
  uint32_t conv_dim;      // (2 key_heads + value_heads) * 128
  uint32_t packed_width;  // >= conv_dim + value_heads * 128 + 2 value_heads
};

// One lane of a decode step (the reference's per-lane fields of GDNDecodeBatchParams and its
// SplashLaneRows): byte offsets into the bound state and tape buffers.
struct GdnLane {
  uint32_t first_row;     // its first packed row (packed, tree, hidden)
  uint32_t rows;          // rows of its block, 1..16
  uint32_t pending_path;  // rows of its previous step it accepted and its state does not hold yet (a row mask)
  uint32_t reserved;
  uint64_t pending_tape;  // this layer's tape of its previous step
  uint64_t step_tape;     // this layer's tape of this step
  uint64_t current_cell;  // its state cell the step reads
  uint64_t next_cell;     // and the one it writes: the state before this step's rows
};

// gdn_decode: grid (value_heads, lanes), 1024 threads.
struct GdnDecodeParams {
  struct GdnShapeParams shape;
  uint32_t flags;
  uint32_t layer;
  uint32_t lanes;
  uint32_t table_tiles;  // nonzero: the hidden rows also leave as the activation table (abi/Gguf.h, pieces of 64 rows,
                         // table_tiles row tiles in all) of the projection that reads them
  uint64_t conv_layer_bytes;
  uint64_t recurrent_layer_bytes;
  uint64_t convolution_state_bytes;
  struct GdnLane lane[GDN_MAXIMUM_LANES];
};

// gdn_fold: grid (value_heads, layers), 1024 threads: folds the first `rows` rows of the path a lane
// retained of a step (retained[0], the mask its acceptance wrote) into the state before them, every
// layer's tape tape_layer_bytes after `step_tape`, and writes the cell a next step would hold to
// `fold_cell` (the reference's GDNFoldParams with exact cached states). Nothing when the path
// holds fewer rows.
struct GdnFoldParams {
  struct GdnShapeParams shape;
  uint32_t rows;
  uint32_t reserved;
  uint64_t conv_layer_bytes;
  uint64_t recurrent_layer_bytes;
  uint64_t convolution_state_bytes;
  uint64_t step_tape;
  uint64_t tape_layer_bytes;
  uint64_t state_cell;  // the cell the step wrote
  uint64_t fold_cell;   // the cell the fold writes
};

// gdn_prefill_prepare / gdn_prefill_scan / gdn_prefill_gate: one run of a prompt chunk of one lane, `tokens`
// rows that all enter the state (the reference's GDNPrefillParams, runtime/ops/GDN.cpp:176-222): the run reads
// the layer's convolution carry and recurrent state of `current_cell` and writes those after its rows to
// `next_cell`, another cell. No tape: a prompt's rows are never rolled back.
#define GDN_SCAN_STATE_ROWS 8u    // state rows of one scan workgroup (the reference's SPLASH_GDN_SCAN_STATE_ROWS is 16)
#define GDN_SCAN_BLOCK 16u        // tokens a scan workgroup stages at a time
struct GdnPrefillParams {
  struct GdnShapeParams shape;
  uint32_t flags;
  uint32_t layer;
  uint32_t tokens;        // rows of the run
  uint32_t first;         // the run's first row in the chunk's buffers (packed rows and every buffer of rows)
  uint64_t conv_layer_bytes;
  uint64_t recurrent_layer_bytes;
  uint64_t convolution_state_bytes;
  uint64_t current_cell;
  uint64_t next_cell;
};

#ifdef __cplusplus
static_assert(sizeof(GdnPrefillParams) == 72, "GDN prefill parameters are 72 bytes on both sides");
static_assert(sizeof(GdnLane) == 48, "a GDN lane is 48 bytes on both sides");
static_assert(sizeof(GdnDecodeParams) == 56 + 48 * GDN_MAXIMUM_LANES, "GDN decode parameters are 440 bytes on both sides");
static_assert(sizeof(GdnFoldParams) == 80, "GDN fold parameters are 80 bytes on both sides");
#endif
