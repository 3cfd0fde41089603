// The draft model's attention block, shared by the host operator and the HIP kernels (the counterpart of the
// reference's runtime/metal/abi/DraftAttention.h and of the draft constants of abi/ExecutionGeometry.h:6-7, :37, :47):
// 32 query heads over 8 KV heads of 128 dimensions, eight query rows a lane, a ring of 2048 slots a KV head for the
// context's keys and values, the dynamic convolutions around the attention and the MLP, and the 4-bit context window.
#pragma once
#include <stdint.h>

#define DRAFT_ATTENTION_QUERY_ROWS 8u
#define DRAFT_ATTENTION_QUERY_HEADS 32u
#define DRAFT_ATTENTION_KV_HEADS 8u
#define DRAFT_ATTENTION_HEAD_DIMENSION 128u
#define DRAFT_ATTENTION_WIDTH (DRAFT_ATTENTION_QUERY_HEADS * DRAFT_ATTENTION_HEAD_DIMENSION)                       // 4096
#define DRAFT_ATTENTION_KV_WIDTH (DRAFT_ATTENTION_KV_HEADS * DRAFT_ATTENTION_HEAD_DIMENSION)                       // 1024
#define DRAFT_ATTENTION_QKV_WIDTH (DRAFT_ATTENTION_WIDTH + 2u * DRAFT_ATTENTION_KV_WIDTH)                          // 6144
// A KV head's attention rows: its four query heads' eight query rows, row 8 j + r query head 4 h + j's row r.
#define DRAFT_ATTENTION_ROWS (DRAFT_ATTENTION_QUERY_HEADS / DRAFT_ATTENTION_KV_HEADS * DRAFT_ATTENTION_QUERY_ROWS)  // 32
#define DRAFT_ATTENTION_WINDOW 2048u      // slots of a ring: position p lives in slot p % 2048
#define DRAFT_ATTENTION_ROPE_PAIRS 64u    // dimension i turns with i + 64
// A lane's RoPE rows hold its verify block's positions (sixteen a lane): its draft's rows take the first eight, its
// context commit one per row it retains.
#define DRAFT_ATTENTION_ROPE_LANE_ROWS 16u
#define DRAFT_ATTENTION_MAXIMUM_LANES 8u
// The ring's slots in tiles of 128: a workgroup of the split pass takes one tile, a wave 32 of its slots; one more
// workgroup takes the eight current rows. A tile with no live slot leaves row maxima of -inf, which the merge skips.
#define DRAFT_ATTENTION_TILE 128u
#define DRAFT_ATTENTION_RING_TILES (DRAFT_ATTENTION_WINDOW / DRAFT_ATTENTION_TILE)  // 16
#define DRAFT_ATTENTION_SPLITS (DRAFT_ATTENTION_RING_TILES + 1u)                     // 17
// A split's partial: fp32 [32 rows][128] unnormalized outputs, then the rows' maxima, then their sums.
#define DRAFT_ATTENTION_PARTIAL_FLOATS (DRAFT_ATTENTION_ROWS * (DRAFT_ATTENTION_HEAD_DIMENSION + 2u))

// The dynamic convolutions of a draft layer (draft_conv), each in two stages, before its attention or MLP and after
// it with the residual: a stage weighs a channel's row and the row before it (its two taps), each by a base weight
// plus the dynamic weight of the channel's group of 16 channels, which the draft projects for every row, stage and tap.
#define DRAFT_CONVOLUTION_STAGES 2u
#define DRAFT_CONVOLUTION_TAPS 2u
#define DRAFT_CONVOLUTION_GROUP 16u
// A context window holds, per ring slot, the draft's context row in 4-bit codes over groups of 64 values: all slots'
// codes first, then each slot's and group's fp16 scale and minimum.
#define DRAFT_CONTEXT_GROUP 64u

#if defined(__HIPCC__) || defined(__cplusplus)
constexpr inline uint32_t draft_dynamic_width(uint32_t hidden) {
  return DRAFT_CONVOLUTION_STAGES * DRAFT_CONVOLUTION_TAPS * (hidden / DRAFT_CONVOLUTION_GROUP);
}
constexpr inline uint64_t draft_ring_bytes() {
  return uint64_t(DRAFT_ATTENTION_KV_HEADS) * DRAFT_ATTENTION_WINDOW * DRAFT_ATTENTION_HEAD_DIMENSION * 2u;
}
constexpr inline uint64_t draft_context_codes_bytes(uint32_t width) { return uint64_t(DRAFT_ATTENTION_WINDOW) * (width / 2u); }
constexpr inline uint64_t draft_context_window_bytes(uint32_t width) {
  return draft_context_codes_bytes(width) + uint64_t(DRAFT_ATTENTION_WINDOW) * (width / DRAFT_CONTEXT_GROUP) * 4u;
}
#endif

// draft_conv: grid (ceil(8 hidden / 256), lanes), 256 threads. finish: the second stage, which adds the residual.
struct DraftConvParams {
  uint32_t finish;
  uint32_t hidden;
};

// draft_attention_qkv: grid (40, lanes) of 512 threads: a wave a (row, head) task of the 8 x (32 + 8) a lane, every
// thread a share of the value rows' transpose. draft_attention_merge: grid (8 KV heads, lanes), 1024 threads.
struct DraftLanesParams {
  uint32_t lanes;
};

// draft_attention_split: grid (8 KV heads, lanes, 17), 256 threads.
// Lane l's key ring starts keys[l] bytes into the bound rings buffer, its value ring values[l] bytes.
struct DraftAttentionParams {
  uint32_t lanes;
  uint32_t padding;
  uint32_t cache_length[DRAFT_ATTENTION_MAXIMUM_LANES];
  uint64_t keys[DRAFT_ATTENTION_MAXIMUM_LANES];
  uint64_t values[DRAFT_ATTENTION_MAXIMUM_LANES];
};

// draft_context_kv: grid (rows x 8 KV heads, lanes), 64 threads: context row r's head into the slot of its position.
// commit 0: lane 0 alone, rows 0..rows-1 of the bound rows at positions start_position[0] + r, RoPE row r.
// commit 1: lane l's path row i is the i-th set bit b of retained[l] (while i < its lane rows' count), bound row
// lane_rows[l].first + b, at position start_position[l] + i, RoPE row 16 l + i.
struct DraftContextParams {
  uint32_t rows;
  uint32_t commit;
  uint32_t start_position[DRAFT_ATTENTION_MAXIMUM_LANES];
  uint64_t keys[DRAFT_ATTENTION_MAXIMUM_LANES];
  uint64_t values[DRAFT_ATTENTION_MAXIMUM_LANES];
};

// draft_context_store / _load: grid (ceil(rows x width / 64 / 4)), 256 threads: a wave a (row, group) of 64 values.
// commit 1 (store only): row i is the i-th set bit b of retained[0] (while i < lane_rows[0].rows), bound row
// lane_rows[0].first + b.
struct DraftWindowParams {
  uint32_t rows;
  uint32_t start_position;
  uint32_t width;
  uint32_t commit;
};

// draft_mask_rows: grid (ceil(width / 256), 7, lanes), 256 threads: rows 1..7 of each lane's eight take the mask row.
struct DraftMaskRowsParams {
  uint32_t width;
};

#if defined(__cplusplus)
static_assert(sizeof(DraftConvParams) == 8, "draft convolution parameters are 8 bytes on both sides");
static_assert(sizeof(DraftAttentionParams) == 168, "draft attention parameters are 168 bytes on both sides");
static_assert(sizeof(DraftContextParams) == 168, "draft context parameters are 168 bytes on both sides");
static_assert(sizeof(DraftWindowParams) == 16, "draft window parameters are 16 bytes on both sides");
#endif
