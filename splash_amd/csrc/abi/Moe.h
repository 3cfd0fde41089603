// Mixture-of-experts routing of a verify block: parameters shared by the host operator (ops/Moe)
// and the HIP kernels. The counterpart of the reference's runtime/metal/abi/MoE.h:23-245.
//
// A row's router scores (fp32, one per expert) select top_k experts, ranked by (score descending,
// expert id ascending); route (row, rank) carries the weight exp2((s_rank - s_0) log2 e) / sum over
// the k selected, summed in rank order. Routes are grouped by expert into tiles of up to 16 rows (one
// MFMA row tile): tile t serves expert tile_expert[t] with tile_rows[t] rows in grouped slots
// 16 t .. 16 t + tile_rows[t] - 1; route_slot[route] names a route's slot and slot_row[slot] the
// row a slot gathers (0xFFFFFFFF for an empty slot). An expert's routes keep their route order.
#pragma once
#include <stdint.h>
#include "abi/Gguf.h"

#define MOE_MAXIMUM_EXPERTS 256u
#define MOE_MAXIMUM_TOP 16u
#define MOE_TILE_ROWS 16u
#define MOE_NO_ROW 0xFFFFFFFFu
// Words of moe_group_routes' bit matrix, a row an expert and a bit a route: experts * ceil(routes / 32) at most
// (128 experts of 4096 routes, 256 experts of 2048).
#define MOE_GROUP_WORDS 16384u

// The most tiles `routes` routes over `experts` experts can take.
#if defined(__HIPCC__)
__host__ __device__
#endif
inline uint32_t moe_maximum_tiles(uint32_t routes, uint32_t experts) {
  const uint32_t full = routes / MOE_TILE_ROWS, partial = experts < routes ? experts : routes;
  return full + partial;
}

// moe_route_select: grid (rows), 64 threads. A row's routes are its top_k routed experts and then the `shared` slices
// of the shared expert, ids `experts` on, which every row visits (the reference's moe_shared_slice, moe.metal:5-8):
// weighted by the sigmoid of the row's product with the block's fp32 scalar gate (shared_gated), or by 1.
struct MoeRouteParams {
  uint32_t rows, experts, top_k;
  uint32_t score_stride;  // floats between rows of scores
  uint32_t shared;        // slices of the shared expert
  uint32_t shared_gated;
  uint32_t input_size;    // of the rows the scalar gate multiplies (bf16)
  // 0: the softmax of the selected scores; 1: each one's sigmoid over the sum of theirs plus 1e-20, summed in rank
  // order (the reference's MoeRouter::SigmoidNormalized, moe.metal:104-110).
  uint32_t sigmoid_router;
};
// moe_group_routes: one workgroup of 1024 threads.
struct MoeGroupParams {
  uint32_t routes;  // rows * top_k
  uint32_t experts, top_k;
  uint32_t maximum_tiles;
};
// moe_gather_table: grid (hidden / 32, maximum tiles), 64 threads: a tile's rows as its activation table.
struct MoeGatherParams {
  uint32_t hidden;
  uint32_t maximum_tiles;
  uint64_t table_bytes;  // between tiles' tables
};
// moe_combine: grid (rows, hidden / 256), 256 threads: out = bf16(residual + sum_rank w y[slot]) in rank order.
// table_tiles nonzero (hidden a multiple of 256): the rows also leave as the activation table (abi/Gguf.h, pieces of
// 64 rows, table_tiles row tiles in all) of the projection after their RMS norm, as a residual projection's _rn
// epilogue writes it: bf16(out * norm weight) and each 64-column group's sums of squares of `out`.
struct MoeCombineParams {
  uint32_t rows, hidden, top_k;
  uint32_t table_tiles;
};

// gguf_moe_decode_<fmt>_<a|gt>: grid (workgroups of one expert projection, maximum tiles), 256 threads.
struct GgufMoeParams {
  struct GgufDecodeParams decode;  // rows is the tile's, from tile_rows; splits 1
  uint64_t expert_bytes;           // between experts' images of a tensor
  uint64_t table_bytes;            // between tiles' activation tables
  uint64_t next_table_bytes;       // between tiles' next tables (table epilogue)
  uint32_t out_row_bytes;          // bytes of an output row
  uint32_t reserved;
};

#ifdef __cplusplus
static_assert(sizeof(MoeRouteParams) == 32 && sizeof(MoeGroupParams) == 16 && sizeof(MoeGatherParams) == 16 &&
                  sizeof(MoeCombineParams) == 16 && sizeof(GgufMoeParams) == 96,
              "MoE parameters have the same size on both sides");
#endif
