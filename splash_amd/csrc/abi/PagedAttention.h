// Paged INT8 KV cache layout and the attention kernels' parameters, shared by the host operator
// (ops/PagedAttention) and the HIP kernels. The counterpart of the reference's
// runtime/metal/abi/PagedAttention.h, KvExtent.h and VerifyTree.h at the geometry this backend
// serves: 256-token pages, fp16 scales per (token, KV head), 64-lane wavefronts.
//
// A layer's KV pool is an array of physical pages. One page, for H KV heads of D dimensions and
// T = ATTENTION_PAGE_TOKENS tokens:
//   keys          int8 [H][T][D]            token-major: a token's D codes are contiguous
//   values        int8 [H][T / 64][D][64]   per block of 64 tokens, dimension-major: the 64 codes of
//                                           one dimension are contiguous (what the P.V MFMA reads)
//   key_scales    fp16 [H][T]
//   value_scales  fp16 [H][T]
// value = code * scale, code in [-127, 127], scale = max|v| / 127 rounded to fp16 (the reference's
// store rule, attention_store.h:52-85, with BASELINE's fp16 scale). The page table maps a
// sequence's logical pages to physical ones; its entries are 64-bit (physical page index).
#pragma once
#include <stdint.h>

#define ATTENTION_PAGE_TOKENS 256u
#define ATTENTION_STEP_TOKENS 64u    // tokens the split kernel takes at a time; history splits hold whole steps
#define ATTENTION_VALUE_BLOCK 64u
#define ATTENTION_MAXIMUM_ROWS 16u      // rows of one sequence's verify block (SPLASH_TARGET_VERIFY_ROWS)
#define ATTENTION_MAXIMUM_SEQUENCES 8u  // sequences of one dispatch
#define ATTENTION_MAXIMUM_SPLITS 128u   // SPLASH_ATTENTION_MAXIMUM_SPLITS

#if defined(__HIPCC__) || defined(__cplusplus)
#if defined(__HIPCC__)
#define ATTENTION_INLINE __host__ __device__ inline
#else
#define ATTENTION_INLINE inline
#endif
ATTENTION_INLINE uint64_t attention_page_keys_bytes(uint32_t kv_heads, uint32_t head_dim) {
  return uint64_t(kv_heads) * ATTENTION_PAGE_TOKENS * head_dim;
}
ATTENTION_INLINE uint64_t attention_page_scales_bytes(uint32_t kv_heads) { return uint64_t(kv_heads) * ATTENTION_PAGE_TOKENS * 2u; }
// Byte offsets of a page's four tensors, and its size.
ATTENTION_INLINE uint64_t attention_page_values_offset(uint32_t h, uint32_t d) { return attention_page_keys_bytes(h, d); }
ATTENTION_INLINE uint64_t attention_page_key_scales_offset(uint32_t h, uint32_t d) { return 2u * attention_page_keys_bytes(h, d); }
ATTENTION_INLINE uint64_t attention_page_value_scales_offset(uint32_t h, uint32_t d) {
  return 2u * attention_page_keys_bytes(h, d) + attention_page_scales_bytes(h);
}
ATTENTION_INLINE uint64_t attention_page_bytes(uint32_t h, uint32_t d) {
  return 2u * attention_page_keys_bytes(h, d) + 2u * attention_page_scales_bytes(h);
}
// Element indices inside a page's tensors.
ATTENTION_INLINE uint64_t attention_key_index(uint32_t head, uint32_t token, uint32_t dim, uint32_t head_dim) {
  return (uint64_t(head) * ATTENTION_PAGE_TOKENS + token) * head_dim + dim;
}
ATTENTION_INLINE uint64_t attention_value_index(uint32_t head, uint32_t token, uint32_t dim, uint32_t head_dim) {
  return ((uint64_t(head) * (ATTENTION_PAGE_TOKENS / ATTENTION_VALUE_BLOCK) + token / ATTENTION_VALUE_BLOCK) * head_dim + dim) *
             ATTENTION_VALUE_BLOCK + token % ATTENTION_VALUE_BLOCK;
}
ATTENTION_INLINE uint64_t attention_scale_index(uint32_t head, uint32_t token) {
  return uint64_t(head) * ATTENTION_PAGE_TOKENS + token;
}
#endif

// A packed row of a verify block (the reference's SplashTreeRow, abi/VerifyTree.h:24-38): bit j of
// `ancestors` is set when block row j (itself included) is visible to the row; a chain's row r has
// ancestors (2 << r) - 1, parent r - 1 and depth r.
struct AttentionTreeRow {
  uint32_t ancestors;
  uint16_t parent;
  uint16_t depth;
};

// One sequence of a dispatch (the reference's SplashAttentionSequence, abi/PagedAttention.h:126-160).
struct AttentionSequence {
  uint32_t first_row;        // its first packed row in the qkv rows, tree rows and outputs
  uint32_t committed;        // tokens in its cache before the block; row r is stored at slot committed + r
  uint32_t table_first;      // its first entry in the page table
  uint16_t rows;             // rows of its block, 1..16
  uint16_t steps_per_split;  // steps (ATTENTION_STEP_TOKENS tokens) of one history split, from its own length alone,
                             // so that batching never changes a sequence's result; the last split takes the rest
};

struct AttentionParams {
  uint32_t q_heads, kv_heads, head_dim;
  uint32_t rotary_pairs;     // pairs (i, i + pairs) rotated by RoPE; 0 for none
  uint32_t normalize;        // 1: q and k heads are RMS-normed with the bound weights first
  uint32_t qkv_stride;       // elements of a packed qkv row: (q_heads + 2 kv_heads) * head_dim, or with gates
                             // (2 q_heads + 2 kv_heads) * head_dim: each query head's queries, then its gate
  uint32_t splits;           // grid.y of the split kernel: the most splits of any sequence
  uint32_t sequences;
  uint32_t table_tiles;      // attention_reduce_*_t: row tiles of the activation table it writes
  uint32_t gated;            // 1: the output rows are multiplied by the sigmoid of their heads' gates (attention_gate.h:19-44)
  uint32_t int8_queries;     // 1: queries are staged as INT8 codes with one scale a (row, head) and scored by an
                             // INT8 x INT8 product (the reference's q8q kernels, paged_attention_tile.h:294-322)
  uint32_t reserved;
  uint64_t page_bytes;       // bytes between physical pages of the layer's pool
  struct AttentionSequence sequence[ATTENTION_MAXIMUM_SEQUENCES];
};

// attention_q8_commit: moves the retained path's K/V slots to their depths
// (the reference's SplashKvPathCommitParams, kv_path_commit.metal:21-48).
struct AttentionCommitParams {
  uint32_t kv_heads, head_dim;
  uint32_t sequences;
  uint32_t layers;         // grid.z: the layers' pools lie layer_bytes apart from the bound pool
  uint64_t page_bytes;
  uint64_t layer_bytes;
  struct AttentionSequence sequence[ATTENTION_MAXIMUM_SEQUENCES];
};

#ifdef __cplusplus
static_assert(sizeof(AttentionTreeRow) == 8, "a tree row is 8 bytes on both sides");
static_assert(sizeof(AttentionSequence) == 16, "an attention sequence is 16 bytes on both sides");
static_assert(sizeof(AttentionParams) == 56 + 16 * ATTENTION_MAXIMUM_SEQUENCES, "attention parameters are 184 bytes on both sides");
static_assert(sizeof(AttentionCommitParams) == 32 + 16 * ATTENTION_MAXIMUM_SEQUENCES, "commit parameters are 160 bytes on both sides");
#endif
