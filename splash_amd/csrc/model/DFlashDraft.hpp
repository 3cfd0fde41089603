// The draft model that proposes a verify step's rows (the reference's model::DFlashDraft, runtime/model/DFlashDraft.hpp:
// 66-356, DFlashDraft.cpp:184-430): per lane eight query rows (the anchor token's embedding, then seven mask rows)
// through layers of dynamic convolution -> attention over the lane's rings of context keys and values -> dynamic
// convolution -> SwiGLU MLP, then the target's vocabulary head and the selector's projection; and the writers of the
// context the rings hold (the target's captured hidden rows projected, normalized, kept as the 4-bit window and
// projected into every layer's keys and values).
// A driver of operators: every projection is an ops::Linear plan over a weight image of any format the kernels read,
// so the draft's own formats (the reference quantizes its projections in groups of 64 columns, DraftCheckpoint.cpp) are
// the loader's business, not this file's.
#pragma once
#include "hip/Backend.hpp"
#include "ops/DraftAttention.hpp"
#include "ops/Linear.hpp"
#include "ops/Weights.hpp"

#include <array>
#include <cstdint>
#include <span>
#include <vector>

namespace splash::model {

struct DFlashDraftLayout final {
  uint32_t layers = 0;
  uint32_t hiddenSize = 0;
  uint32_t vocabularySize = 0;
  uint32_t intermediateSize = 0;
  uint32_t targetLayerCount = 0;   // the target layers whose hidden rows a context row concatenates
  [[nodiscard]] constexpr uint32_t dynamicSize() const noexcept { return draft_dynamic_width(hiddenSize); }
  [[nodiscard]] constexpr uint32_t targetHiddenSize() const noexcept { return hiddenSize * targetLayerCount; }
  [[nodiscard]] constexpr uint32_t contextKvSize() const noexcept { return 2 * DRAFT_ATTENTION_KV_WIDTH; }
  [[nodiscard]] constexpr ops::DraftAttentionShape attentionShape() const noexcept { return ops::DraftAttentionShape::of(hiddenSize); }
  // Bytes of a lane's rings of every layer (keys, then values, layer by layer) and of its context window.
  [[nodiscard]] constexpr uint64_t ringBytes() const noexcept { return uint64_t{layers} * 2 * draft_ring_bytes(); }
  [[nodiscard]] constexpr uint64_t windowBytes() const noexcept { return draft_context_window_bytes(hiddenSize); }
};

struct DFlashDraftLayerWeights final {
  hip::Buffer inputNorm;             // bf16 [hidden]
  hip::Buffer attentionConvolution;  // bf16 [stage][tap][hidden]
  ops::Projection attentionDynamic;  // hidden -> dynamicSize
  ops::Projection qkvProjection;     // hidden -> 6144
  hip::Buffer queryNorm, keyNorm;    // bf16 [128]
  ops::Projection outputProjection;  // 4096 -> hidden
  hip::Buffer postAttentionNorm;
  hip::Buffer mlpConvolution;
  ops::Projection mlpDynamic;
  ops::Projection gateProjection, upProjection;  // hidden -> intermediate
  ops::Projection downProjection;                // intermediate -> hidden
  // The key and value rows of qkvProjection (its columns from 4096 on) as a projection of their own, which the context
  // writers run: a view of the same image, no copy (DFlashDraft.cpp:33-42 in the reference).
  ops::Projection contextKvProjection;
};

struct DFlashDraftWeights final {
  DFlashDraftLayout layout;
  std::vector<DFlashDraftLayerWeights> layers;
  ops::Projection contextProjection;   // targetHiddenSize -> hidden
  hip::Buffer hiddenNorm, finalNorm;   // bf16 [hidden]
  ops::Projection selectorProjection;  // hidden -> DRAFT_SELECTOR_RANK
  hip::Buffer maskEmbedding;           // bf16 [hidden]; may be empty
};

// The rows of a q|k|v projection of one segment from column `first` on, as a projection over a slice of its image
// (an image is rows of sixteen columns, so a range that starts on one is contiguous in it).
[[nodiscard]] ops::Projection projectionRowsFrom(const ops::Projection &projection, uint32_t first);

// One lane's place in the draft's state: its rings of layer 0 (the layers follow, 2 rings apart) and its window.
struct DFlashLaneState final {
  uint64_t rings = 0;    // bytes into the rings buffer: layer l's keys at rings + 2 l R, its values R after (R = draft_ring_bytes())
  uint64_t window = 0;   // bytes into the windows buffer
};

struct DFlashDecodeBuffers final {
  ops::LinearScratch scratch;
  std::array<hip::Buffer, 2> hidden;  // bf16 [lanes * 8][hidden]: layer l reads hidden[l & 1]
  hip::Buffer normalized, dynamic, convolved, proposalQkv, attention, projected, residual, intermediate;
  hip::Buffer finalHidden;     // bf16 [lanes * 8][hidden]
  hip::Buffer logits;          // fp32 [lanes * 8][vocabulary]
  hip::Buffer selectorHidden;  // bf16 [lanes * 8][DRAFT_SELECTOR_RANK]
  hip::Buffer queryKeys, queryValues;
  hip::Buffer ropeCos, ropeSin;  // fp32 [lane][16][64]: a lane's rows at positions cache length + r
  hip::Buffer rings;
};

struct DFlashContextBuffers final {
  ops::LinearScratch scratch;
  hip::Buffer capturedTargetHidden;  // bf16 [rows][targetHiddenSize]
  hip::Buffer projected, hidden;     // bf16 [rows][hidden]
  hip::Buffer contextKv;             // bf16 [rows][2048]
  hip::Buffer ropeCos, ropeSin;      // fp32: a prompt's rows one each; a step's [lane][16][64]
  hip::Buffer rings, windows;
};

class DFlashDraft final {
public:
  // `head`: the target's vocabulary head (fp32 logits), which the draft shares: whole, or a view of the rows of a subset
  // of the tokens (ops::Projection::rows over DraftVocabulary's two ranges), whose columns the logits rows then hold.
  DFlashDraft(const DFlashDraftWeights &weights, const ops::Linear &linear, const ops::Projection &head);

  [[nodiscard]] const DFlashDraftLayout &layout() const noexcept { return weights_.layout; }
  // The scratch every plan of up to `rows` rows of the draft's projections and of the head needs.
  [[nodiscard]] ops::LinearScratchSize scratchSize(uint32_t rows) const;

  // Rows 1..7 of each lane's eight rows of `rows` take the mask embedding.
  void addMaskRows(hip::CommandGraph &graph, const hip::Buffer &rows, uint32_t lanes) const;
  // The draft's forward pass of one step: lane l's eight rows at positions cacheLengths[l] on. Leaves the logits of the
  // whole vocabulary and the selector's rows (what ops::DraftSelector::addCandidates reads).
  void addDecode(hip::CommandGraph &graph, const DFlashDecodeBuffers &buffers, std::span<const DFlashLaneState> lanes,
                 std::span<const uint32_t> cacheLengths) const;
  // `rows` prompt rows of one lane at positions startPosition on: their context rows into its window and every
  // layer's keys and values into its rings.
  void addContextPrefill(hip::CommandGraph &graph, const DFlashContextBuffers &buffers, const DFlashLaneState &lane, uint32_t rows,
                         uint32_t startPosition) const;
  // The rows each lane retained of a verify step (masks and lane rows read from the device), the path's i-th at
  // startPositions[l] + i.
  void addContextCommit(hip::CommandGraph &graph, const DFlashContextBuffers &buffers, std::span<const DFlashLaneState> lanes,
                        const hip::Buffer &retainedRows, const hip::Buffer &laneRows, std::span<const uint32_t> startPositions,
                        const ops::StepRows &step) const;
  // A lane's rings rebuilt from its window: `rows` rows of positions startPosition on (a state restored from its
  // cached form keeps the window alone).
  void addContextRebuild(hip::CommandGraph &graph, const DFlashContextBuffers &buffers, const DFlashLaneState &lane, uint32_t rows,
                         uint32_t startPosition) const;

private:
  void addContextKv(hip::CommandGraph &graph, const DFlashContextBuffers &buffers, const DFlashLaneState &lane, uint32_t rows,
                    uint32_t startPosition) const;
  const DFlashDraftWeights &weights_;
  const ops::Linear &linear_;
  const ops::Projection &head_;
};

} // namespace splash::model
