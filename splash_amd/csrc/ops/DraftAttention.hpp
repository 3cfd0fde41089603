// ops::DraftAttention of the reference (runtime/ops/DraftAttention.hpp:12-152, DraftAttention.cpp:85-309) over
// kernels/draft_attention.hip: the attention block of the draft model that proposes a verify step's rows. A lane's
// eight query rows attend to its ring of 2048 context positions and to themselves; the dynamic convolutions run before
// and after the attention and the MLP; the context writers fill the rings from prompt rows and from the rows a step
// retained; the context window keeps the rows the rings are computed from in 4-bit codes.
// Every add* validates its buffers and throws std::invalid_argument before it adds a dispatch.
#pragma once
#include "abi/DraftAttention.h"
#include "hip/Backend.hpp"
#include "ops/DraftSelector.hpp"  // StepRows

#include <cstdint>
#include <span>

namespace splash::ops {

struct DraftAttentionShape final {
  uint32_t hiddenSize = 0;
  uint32_t dynamicSize = 0;
  uint32_t qkvSize = 0;
  uint32_t attentionSize = 0;
  uint32_t queryHeads = 0;
  uint32_t kvHeads = 0;
  uint32_t headDimension = 0;
  bool operator==(const DraftAttentionShape &) const = default;
  // The shape the kernels are compiled for, over a hidden state of `hidden` values.
  [[nodiscard]] static constexpr DraftAttentionShape of(uint32_t hidden) noexcept {
    return {hidden, draft_dynamic_width(hidden), DRAFT_ATTENTION_QKV_WIDTH, DRAFT_ATTENTION_WIDTH, DRAFT_ATTENTION_QUERY_HEADS,
            DRAFT_ATTENTION_KV_HEADS, DRAFT_ATTENTION_HEAD_DIMENSION};
  }
};

struct DraftAttentionWorkspace final {
  uint64_t convolutionBytes = 0;
  uint64_t qkvBytes = 0;
  uint64_t groupedQueriesBytes = 0;  // the grouped query rows and, behind them, the splits' partials
  uint64_t queryKeysBytes = 0;
  uint64_t queryValuesBytes = 0;
};

// Constructed only by DraftAttention::plan, so the shape, the lanes and the workspace cannot disagree.
class DraftAttentionPlan final {
public:
  [[nodiscard]] DraftAttentionShape shape() const noexcept { return shape_; }
  [[nodiscard]] uint32_t lanes() const noexcept { return lanes_; }
  [[nodiscard]] DraftAttentionWorkspace workspace() const noexcept;

private:
  DraftAttentionPlan(DraftAttentionShape shape, uint32_t lanes) : shape_(shape), lanes_(lanes) {}
  DraftAttentionShape shape_;
  uint32_t lanes_;
  friend class DraftAttention;
};

enum class DraftConvolutionStage : uint8_t { Prepare, Residual };

struct DraftConvolutionBuffers final {
  hip::Buffer input;     // bf16 [lanes * 8][hidden]
  hip::Buffer dynamic;   // bf16 [lanes * 8][dynamicSize]: [stage][tap][group of 16 channels]
  hip::Buffer weights;   // bf16 [stage][tap][hidden]
  hip::Buffer residual;  // bf16 [lanes * 8][hidden]; read by the Residual stage
  hip::Buffer output;    // bf16 [lanes * 8][hidden]
};

struct DraftPrepareBuffers final {
  hip::Buffer qkv;             // bf16 [lanes * 8][6144]
  hip::Buffer groupedQueries;  // bf16 [lanes][query head][8][128]
  hip::Buffer queryNorm, keyNorm;  // bf16 [128]
  hip::Buffer ropeCos, ropeSin;    // fp32 [lane][16][64]: a lane's rows take the first eight of its sixteen
  hip::Buffer queryKeys;       // bf16 [lanes][KV head][8][128]
  hip::Buffer queryValues;     // bf16 [lanes][KV head][128][8]
};

// A layer's rings: lane l's keys [KV head][slot][128] start keys[l] bytes into `buffer`, its values
// [KV head][128][slot] values[l] bytes; each draft_ring_bytes() long.
struct DraftRings final {
  hip::Buffer buffer;
  std::span<const uint64_t> keys;
  std::span<const uint64_t> values;
};

struct DraftDecodeAttentionBuffers final {
  // The prepared query rows, grouped by query head, and the splits' partials behind them. The attention leaves its
  // rows in the query rows' place, in [row][query head][dimension] order, the output projection's input.
  hip::Buffer groupedQueries;
  DraftRings rings;
  hip::Buffer queryKeys;
  hip::Buffer queryValues;
};

class DraftAttention final {
public:
  // Throws for no lanes, more than DRAFT_ATTENTION_MAXIMUM_LANES, or a shape no kernel is compiled for.
  [[nodiscard]] static DraftAttentionPlan plan(DraftAttentionShape shape, uint32_t lanes);

  static void addConvolution(hip::CommandGraph &graph, const DraftConvolutionBuffers &buffers, const DraftAttentionPlan &plan,
                             DraftConvolutionStage stage);
  static void addPrepare(hip::CommandGraph &graph, const DraftPrepareBuffers &buffers, const DraftAttentionPlan &plan);
  static void addDecode(hip::CommandGraph &graph, const DraftDecodeAttentionBuffers &buffers, std::span<const uint32_t> cacheLengths,
                        const DraftAttentionPlan &plan);
  // The context writers. A row of contextKv holds its keys, then its values (1024 each); its normalized, rotated keys
  // and its values go to its position's slot of the ring. The prefill writes `tokens` rows of one lane from
  // startPosition on, row r rotated by RoPE row r.
  static void addContextPrefill(hip::CommandGraph &graph, const hip::Buffer &contextKv, const hip::Buffer &keyNorm,
                                const hip::Buffer &ropeCos, const hip::Buffer &ropeSin, const hip::Buffer &rings, uint64_t keys,
                                uint64_t values, uint32_t tokens, uint32_t startPosition, DraftAttentionShape shape);
  // Each lane's retained rows of a decode step (a mask of its rows, which acceptance writes) among its rows of the
  // step (laneRows: {first, rows} a lane, which the step's proposer writes): the path's i-th at the lane's start
  // position plus i, rotated by the lane's RoPE row i.
  static void addContextCommit(hip::CommandGraph &graph, const hip::Buffer &contextKv, const hip::Buffer &keyNorm,
                               const hip::Buffer &ropeCos, const hip::Buffer &ropeSin, const DraftRings &rings,
                               const hip::Buffer &retainedRows, const hip::Buffer &laneRows,
                               std::span<const uint32_t> startPositions, const StepRows &step, DraftAttentionShape shape);

  // A context window: for each slot of a ring, the bf16 context row of `width` values the slot's keys and values are
  // computed from, in 4-bit codes of 64-value groups with each group's fp16 scale and minimum.
  [[nodiscard]] static uint64_t contextWindowBytes(uint32_t width);
  // Stores `rows` context rows in the slots of positions startPosition on.
  static void addWindowStore(hip::CommandGraph &graph, const hip::Buffer &context, const hip::Buffer &window, uint32_t rows,
                             uint32_t startPosition, uint32_t width);
  // Stores the first `rows` (at most a verify block's) of the context rows one lane retained of its rows of a step of
  // `contextRows` context rows, the path's i-th at position startPosition + i.
  static void addWindowCommit(hip::CommandGraph &graph, const hip::Buffer &context, const hip::Buffer &window,
                              const hip::Buffer &retained, const hip::Buffer &laneRows, uint32_t contextRows, uint32_t rows,
                              uint32_t startPosition, uint32_t width);
  // Loads the rows of positions startPosition on back into `rows` rows.
  static void addWindowLoad(hip::CommandGraph &graph, const hip::Buffer &window, const hip::Buffer &context, uint32_t rows,
                            uint32_t startPosition, uint32_t width);
  // Rows 1..7 of each lane's eight input rows take the mask embedding (the reference's Embedding::addDraftMaskRows,
  // runtime/ops/Embedding.cpp:49-58); row 0 is the lane's anchor token's.
  static void addMaskRows(hip::CommandGraph &graph, const hip::Buffer &mask, const hip::Buffer &rows, uint32_t width, uint32_t lanes);
};

} // namespace splash::ops
