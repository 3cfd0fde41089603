// Paged INT8-KV attention of a verify block: the counterpart of the reference's
// ops::PagedAttention (runtime/ops/PagedAttention.hpp:179-366, PagedAttention.cpp:125-146,
// :351-389, :441-667) and kv::Layout (runtime/ops/PagedKv.hpp:155-260) over the gfx950 kernels of
// kernels/paged_attention.hip. Every add* validates its buffers and throws std::invalid_argument
// before it adds a dispatch.
#pragma once
#include "abi/PagedAttention.h"
#include "hip/Backend.hpp"
#include "ops/Linear.hpp"

#include <cstdint>
#include <vector>

namespace splash::ops {

namespace kv {
// A layer's page geometry (PagedKv.hpp:155-260 in the reference; 256-token pages, fp16 scales here).
struct Layout final {
  uint32_t kvHeads = 0;
  uint32_t headDimension = 0;
  static constexpr uint32_t kPageTokens = ATTENTION_PAGE_TOKENS;
  [[nodiscard]] uint64_t bytesPerLayerPage() const noexcept { return attention_page_bytes(kvHeads, headDimension); }
  [[nodiscard]] uint64_t bytesPerToken() const noexcept { return bytesPerLayerPage() / kPageTokens; }
  [[nodiscard]] static uint32_t pagesFor(uint64_t tokens) noexcept { return uint32_t((tokens + kPageTokens - 1) / kPageTokens); }
};
} // namespace kv

struct AttentionGeometry final {
  uint32_t qHeads = 0, kvHeads = 0, headDimension = 0;
  uint32_t rotaryPairs = 0;  // pairs (i, i + pairs) RoPE rotates
  bool normalize = false;    // RMS-norm q and k heads (q_norm, k_norm weights)
  // The projection row holds each query head's queries, then its gate, and the output rows are
  // multiplied by the gates' sigmoids (the reference's Gated geometries, attention_gate.h:19-44).
  bool gated = false;
  // The block's queries score as INT8 codes with one scale per head and row against the INT8 keys, exact in int32 (the
  // reference's "q8q" kernels, PagedAttention.cpp:380-383, paged_attention_tile.h:287-332); otherwise as the bf16 rows.
  bool int8Queries = false;
  [[nodiscard]] uint32_t group() const noexcept { return kvHeads ? qHeads / kvHeads : 0; }
  [[nodiscard]] uint32_t packedWidth() const noexcept { return ((gated ? 2 : 1) * qHeads + 2 * kvHeads) * headDimension; }
  [[nodiscard]] kv::Layout layout() const noexcept { return {kvHeads, headDimension}; }
};

// One sequence's rows of a dispatch (the reference's AttentionRows / AttentionHistory).
struct AttentionRows final {
  uint32_t firstRow = 0;    // first packed row
  uint32_t rows = 0;        // 1..16
  uint32_t committed = 0;   // tokens cached before the block
  uint32_t tableFirst = 0;  // first page-table entry of the sequence
};

// History splits of a sequence of `tokens` tokens (committed + rows): a split holds
// stepsPerSplit steps of ATTENTION_STEP_TOKENS tokens; the partition follows the sequence alone
// (PagedAttention.cpp:125-146 in the reference states the same rule for its geometry).
struct AttentionSplits final {
  uint32_t splits = 1;
  uint32_t stepsPerSplit = 1;
};
[[nodiscard]] AttentionSplits attentionSplits(uint64_t tokens) noexcept;

struct AttentionWorkspaceSize final {
  uint64_t queries = 0, querySums = 0, partials = 0, partialSums = 0;
};
struct AttentionWorkspace final {
  hip::Buffer queries;      // staged fp16 query rows
  hip::Buffer querySums;    // their fp32 sums
  hip::Buffer partials;     // fp16 split outputs, each divided by its sum
  hip::Buffer partialSums;  // fp32 (max, sum) per split and fused row
};

class AttentionPlan final {
public:
  [[nodiscard]] const AttentionGeometry &geometry() const noexcept { return geometry_; }
  [[nodiscard]] const std::vector<AttentionRows> &sequences() const noexcept { return sequences_; }
  [[nodiscard]] uint32_t splits() const noexcept { return splits_; }
  [[nodiscard]] AttentionWorkspaceSize workspace() const noexcept;
  [[nodiscard]] AttentionParams params(uint64_t pageBytes) const noexcept;

private:
  friend class PagedAttention;
  AttentionGeometry geometry_;
  std::vector<AttentionRows> sequences_;
  std::vector<AttentionSplits> partition_;
  uint32_t splits_ = 1;
};

// A prompt chunk of one sequence (the reference's kv::ChunkedPrefillParams with its rows' place in the command,
// PagedAttention.hpp:28-39): `tokens` rows at positions from `committed`, attending causally. It runs as tiles of
// ATTENTION_MAXIMUM_ROWS rows (the reference's tiles of kAttentionTileRows, :42-50), tile t a block of the sequence
// whose history ends where tile t - 1's rows end, ATTENTION_MAXIMUM_SEQUENCES tiles a dispatch.
struct AttentionChunk final {
  uint32_t firstRow = 0;    // first packed row
  uint32_t tokens = 0;      // 1..kMaximumChunkRows
  uint32_t committed = 0;   // tokens cached before the chunk
  uint32_t tableFirst = 0;  // first page-table entry of the sequence
};
inline constexpr uint32_t kMaximumChunkRows = 2048;  // SPLASH_PREFILL_TOKEN_BUDGET, ExecutionGeometry.h:36

// The dispatches of a command's chunks: each a plan of up to eight tiles. A tile's history splits follow its own
// length alone (attentionSplits), so a row's result is, bit for bit, the one its tile gives as a verify block.
class AttentionChunkPlan final {
public:
  [[nodiscard]] const AttentionGeometry &geometry() const noexcept { return geometry_; }
  [[nodiscard]] const std::vector<AttentionPlan> &dispatches() const noexcept { return dispatches_; }
  [[nodiscard]] uint32_t tiles() const noexcept { return tiles_; }
  [[nodiscard]] uint32_t rows() const noexcept { return rows_; }
  // Staged queries for every tile (a tile's survive from the projection pass to its attention), partials for the
  // dispatch that needs the most (dispatches run one after the other).
  [[nodiscard]] AttentionWorkspaceSize workspace() const noexcept;

private:
  friend class PagedAttention;
  AttentionGeometry geometry_;
  std::vector<AttentionPlan> dispatches_;
  uint32_t tiles_ = 0, rows_ = 0;
};

struct AttentionProjectionBuffers final {
  hip::Buffer qkv;             // bf16 [packed rows][(q + 2 kv) heads * D]
  hip::Buffer queryNorm, keyNorm;  // bf16 [D]; used when geometry.normalize
  hip::Buffer ropeCos, ropeSin;    // fp32 [packed rows][rotaryPairs]; used when rotaryPairs
};
struct KvPages final {
  hip::Buffer pageTable;  // uint64 physical page per logical page
  hip::Buffer pool;       // the layer's physical pages
  uint64_t pageBytes = 0; // bytes between pages (>= layout.bytesPerLayerPage())
};

class PagedAttention final {
public:
  // Throws for a geometry no kernel is compiled for, no or too many sequences, or rows outside 1..16.
  [[nodiscard]] static AttentionPlan plan(const AttentionGeometry &geometry, std::vector<AttentionRows> sequences);
  // q/k norm + RoPE + query staging + INT8 store of the block's K and V (PagedAttention.cpp:441-464).
  static void addProjection(hip::CommandGraph &graph, const AttentionPlan &plan, const AttentionProjectionBuffers &buffers,
                            const AttentionWorkspace &workspace, const KvPages &pages);
  // The q|k|v projection and addProjection's work in ONE dispatch (Linear::addWithAttention), where the reference runs the
  // projection and its prepare kernel one after the other (QwenTarget.cpp:457-470): `projection` writes the packed
  // rows into buffers.qkv (which is `linear.output`) and the last workgroup of each head prepares it. The same packed
  // rows, staged queries and cache bytes as the two dispatches. fusesProjection: whether the kernels take the pair.
  [[nodiscard]] static bool fusesProjection(const AttentionPlan &plan, const Projection &projection, const LinearPlan &linearPlan) noexcept;
  static PreparedInput addFusedProjection(hip::CommandGraph &graph, const Linear &linear, LinearBuffers linearBuffers,
                                          const Projection &projection, const LinearPlan &linearPlan, const AttentionPlan &plan,
                                          const AttentionProjectionBuffers &buffers, const AttentionWorkspace &workspace,
                                          const KvPages &pages);
  // Split + reduce (PagedAttention.cpp:466-607): output bf16 [packed rows][q heads * D].
  // outputTable (optional): the reduce also writes the rows as the activation table of the
  // projection that follows (gguf_table_bytes(q heads * D, rows)), which then needs no table pass; tableRows: the
  // rows that table holds when they are more than this dispatch's (a chunk's dispatches share one table).
  static void addAttention(hip::CommandGraph &graph, const AttentionPlan &plan, const AttentionWorkspace &workspace,
                           const hip::Buffer &treeRows, const KvPages &pages, const hip::Buffer &output,
                           const hip::Buffer &outputTable = {}, const hip::Buffer &packed = {}, uint32_t tableRows = 0);
  // Prompt chunks (the reference's plan over kv::ChunkedPrefillParams, PagedAttention.hpp:270-275, PagedAttention.cpp:351-389):
  // throws for a chunk of no or more than kMaximumChunkRows rows. addChunkProjection runs the projection pass of every
  // dispatch, so that every row's K and V are stored before any row attends; addChunkAttention then splits and merges
  // dispatch by dispatch. Buffers as addProjection's and addAttention's, over all the chunks' rows.
  [[nodiscard]] static AttentionChunkPlan planChunks(const AttentionGeometry &geometry, const std::vector<AttentionChunk> &chunks);
  static void addChunkProjection(hip::CommandGraph &graph, const AttentionChunkPlan &plan, const AttentionProjectionBuffers &buffers,
                                 const AttentionWorkspace &workspace, const KvPages &pages);
  static void addChunkAttention(hip::CommandGraph &graph, const AttentionChunkPlan &plan, const AttentionWorkspace &workspace,
                                const hip::Buffer &treeRows, const KvPages &pages, const hip::Buffer &output,
                                const hip::Buffer &outputTable = {}, const hip::Buffer &packed = {});
  // Moves the retained path's slots to their depths (PagedAttention.cpp:647-667); retained is a
  // uint32 mask per sequence.
  // `layers` pools lie layerBytes apart from pages.pool (one dispatch commits them all, as the
  // reference's grid of layers x KV heads does).
  static void addPathCommit(hip::CommandGraph &graph, const AttentionPlan &plan, const hip::Buffer &retained,
                            const KvPages &pages, uint32_t layers = 1, uint64_t layerBytes = 0);
};

} // namespace splash::ops
