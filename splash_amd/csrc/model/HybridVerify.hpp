// The target part of one speculative-decoding cycle for a hybrid mixture-of-experts decoder
// (the reference's Qwen3.5 family with Gated DeltaNet mixers and a MoE FFN, model/QwenTarget.cpp:
// 206-255 the GDN mixer, :263-347 the attention mixer, :372-395 the MoE routing, :457-496 the layer
// recipe; Runtime.cpp:2701-2707 the tape parity and pending path): embedding -> N x {RMSNorm ->
// mixer input projection -> [GDN decode | q/k norm + RoPE + INT8 store + paged attention] ->
// output projection + residual -> RMSNorm -> router -> top-k routing -> routed experts + combine}
// -> final norm -> LM head -> verify -> acceptance -> KV path commit. Every fourth layer attends,
// the others run Gated DeltaNet.
//
// A lane's recurrent state is never rolled back: a step writes the state BEFORE its rows and leaves
// its rows on the lane's tape, and the lane's next step folds the accepted path (the acceptance's
// retained-rows mask, which its caller hands back as `pendingPath`) first. Cells and tapes are
// double-buffered by the lane's step parity.
#pragma once
#include "hip/Backend.hpp"
#include "model/DenseVerify.hpp"
#include "model/LanePolicies.hpp"
#include "ops/Gdn.hpp"
#include "ops/Glue.hpp"
#include "ops/Linear.hpp"
#include "ops/Moe.hpp"
#include "ops/PagedAttention.hpp"
#include "ops/Sampling.hpp"

#include <array>
#include <cstdint>
#include <optional>
#include <vector>

namespace splash::model {

struct HybridDimensions final {
  uint32_t hidden = 0, vocabulary = 0, layers = 0;
  uint32_t attentionInterval = 4;  // layer l attends when (l + 1) % attentionInterval == 0
  uint32_t qHeads = 0, kvHeads = 0, headDimension = 0, rotaryPairs = 0;
  bool normalizeHeads = true;
  bool gatedAttention = false;  // the attention layers' rows carry output gates
  float ropeTheta = 1000000.0f;
  uint32_t gdnKeyHeads = 0, gdnValueHeads = 0;
  uint32_t gdnPackedWidth = 0;  // the GDN input projection's width (whole column tiles)
  uint32_t experts = 0, topK = 0, expertFfn = 0;
  // experts == 0: every layer's FFN is a dense SwiGLU of this width instead of a mixture of experts (the reference's
  // dense Qwen3.5 targets: the same mixers over QwenTarget::addDenseFfn, QwenTarget.cpp:351-370).
  uint32_t denseFfn = 0;
  [[nodiscard]] bool dense() const noexcept { return experts == 0; }
  // The shared expert: slices of the routed experts' width every row visits, gated by the layer's scalar gate or not.
  uint32_t sharedSlices = 0;
  bool sharedGate = false;

  [[nodiscard]] bool attends(uint32_t layer) const noexcept { return (layer + 1) % attentionInterval == 0; }
  [[nodiscard]] uint32_t attentionLayers() const noexcept { return layers / attentionInterval; }
  [[nodiscard]] uint32_t gdnLayers() const noexcept { return layers - attentionLayers(); }
  // The layer's place among the layers of its kind.
  [[nodiscard]] uint32_t mixerIndex(uint32_t layer) const noexcept {
    const uint32_t before = layer / attentionInterval;  // attention layers before it
    return attends(layer) ? before : layer - before;
  }
  [[nodiscard]] uint32_t qkvWidth() const noexcept { return ((gatedAttention ? 2 : 1) * qHeads + 2 * kvHeads) * headDimension; }
  [[nodiscard]] uint32_t attentionWidth() const noexcept { return qHeads * headDimension; }
  [[nodiscard]] uint32_t gdnWidth() const noexcept { return gdnValueHeads * GDN_HEAD_DIMENSION; }
  [[nodiscard]] ops::GdnShape gdnShape() const noexcept {
    ops::GdnShape s;
    s.keyHeads = gdnKeyHeads;
    s.valueHeads = gdnValueHeads;
    s.convolutionDimension = (2 * gdnKeyHeads + gdnValueHeads) * GDN_HEAD_DIMENSION;
    s.packedWidth = gdnPackedWidth;
    return s;
  }
  [[nodiscard]] ops::MoeShape moeShape() const noexcept { return {hidden, expertFfn, experts, topK, sharedSlices, sharedGate}; }
};

struct HybridLayer final {
  // q|k|v -> o of an attention layer; the packed row [q|k|v|z|b|a] -> out of a GDN layer
  ops::Projection mixerInput, mixerOutput;
  hip::Buffer inputNorm, postNorm;                                  // bf16 [hidden]
  hip::Buffer queryNorm, keyNorm;                                   // attention layers: bf16 [head dimension]
  hip::Buffer convolutionWeights, decay, timeBias, mixerNorm;       // GDN layers (mixerNorm bf16 [128])
  ops::Projection ffnGate, ffnUp, ffnDown;                          // a dense model's SwiGLU
  ops::Projection router;                                           // hidden -> experts, fp32 scores
  ops::MoeExperts experts;                                          // the shared slices' images after the routed experts'
  hip::Buffer sharedScalarGate;                                     // fp32 [hidden], of a gated shared expert
  // What a GGUF keeps as rows of floats (the reference's float segments, GgufImage.cpp:262-300, :353-366), each run by
  // the fp32 projection in place of a quantized one:
  ops::FloatRows routerRows;   // the router [experts][hidden], instead of `router`
  ops::FloatRows gateRows;     // a GDN layer's beta rows then alpha rows [2 value heads][hidden]: the last columns of the
                               // packed row, which mixerInput's segments then leave out
  bool mixerNormFloat = false; // mixerNorm holds fp32 values
};

struct HybridWeights final {
  ops::EmbeddingTable embedding;
  std::vector<HybridLayer> layers;
  hip::Buffer finalNorm;
  ops::Projection head;
};

// One lane of a step: its verify block, and what its previous step left.
struct HybridLane final {
  VerifyLane block;
  uint32_t pendingPath = 0;  // rows of its previous step it accepted (that step's retained-rows mask)
  // A step of parity p reads the lane's cell p and writes cell p ^ 1; its rows go to tape p and its
  // pending rows are on tape p ^ 1. The lane's next step has parity p ^ 1.
  uint32_t parity = 0;
};

class HybridVerify final {
public:
  // prefillRows: the most rows of a prompt chunk (encodePrefill), 0 for a step's most, up to ops::kMaximumChunkRows.
  HybridVerify(hip::Backend &backend, HybridDimensions dimensions, uint32_t maxLanes, uint32_t physicalPages,
               uint32_t pageTableEntries, uint32_t prefillRows = 0);
  [[nodiscard]] uint32_t prefillRows() const noexcept { return rowCapacity_; }

  [[nodiscard]] const HybridDimensions &dimensions() const noexcept { return dims_; }
  HybridWeights &weights() noexcept { return weights_; }
  [[nodiscard]] const hip::Buffer &inputTokens() const noexcept { return inputTokens_; }
  [[nodiscard]] const hip::Buffer &treeRows() const noexcept { return treeRows_; }
  [[nodiscard]] const hip::Buffer &depths() const noexcept { return depths_; }
  [[nodiscard]] const hip::Buffer &uniforms() const noexcept { return uniforms_; }
  [[nodiscard]] const hip::Buffer &tokens() const noexcept { return tokens_; }
  [[nodiscard]] const hip::Buffer &retained() const noexcept { return retained_; }
  [[nodiscard]] const hip::Buffer &acceptedCount() const noexcept { return acceptedCount_; }
  [[nodiscard]] const hip::Buffer &retainedRows() const noexcept { return retainedRows_; }
  [[nodiscard]] const hip::Buffer &pageTable() const noexcept { return pageTable_; }
  [[nodiscard]] const hip::Buffer &kvPool(uint32_t attentionLayer) const { return kvPools_.at(attentionLayer); }
  [[nodiscard]] const hip::Buffer &logits() const noexcept { return logits_; }
  [[nodiscard]] const hip::Buffer &draftProbabilities();
  [[nodiscard]] const hip::Buffer &hidden(uint32_t index) const noexcept { return hidden_[index & 1]; }
  [[nodiscard]] const hip::Buffer &gdnStates() const noexcept { return states_; }
  [[nodiscard]] const hip::Buffer &gdnTape() const noexcept { return tape_; }
  [[nodiscard]] uint64_t pageBytes() const noexcept { return pageBytes_; }
  [[nodiscard]] const ops::GdnStateStrides &gdnStrides() const noexcept { return strides_; }
  [[nodiscard]] uint64_t gdnCellBytes() const noexcept { return cellBytes_; }
  [[nodiscard]] uint64_t gdnTapeLayerBytes() const noexcept { return tapeLayerBytes_; }
  // Where lane `lane` keeps the cell and the tapes of a step of parity `parity`: the step reads the
  // cell of its parity and writes the other one; its tape is its parity's, its pending tape the other's.
  [[nodiscard]] uint64_t cellOffset(uint32_t lane, uint32_t parity) const noexcept { return (uint64_t{lane} * 2 + (parity & 1)) * cellBytes_; }
  [[nodiscard]] uint64_t tapeOffset(uint32_t lane, uint32_t parity, uint32_t gdnLayer) const noexcept {
    return ((uint64_t{lane} * 2 + (parity & 1)) * dims_.gdnLayers() + gdnLayer) * tapeLayerBytes_;
  }
  // Algorithmic bytes one step streams from HBM: dense weights once, every expert of every layer
  // once (a batch of 8 x 16 rows routes to all of them), each lane's KV and recurrent states
  // (read and written), the logits.
  [[nodiscard]] uint64_t stepBytes(const std::vector<HybridLane> &lanes) const;

  // Value head h of a GDN layer's output rows leaves at (h % heads per key) * key heads + h / heads per key, the order
  // llama.cpp's ssm_out reads them in (GgufImage.hpp:29-32): what a model loaded from a GGUF sets. Off by default.
  void setTiledGdnHeads(bool tiled) noexcept { tiledGdnHeads_ = tiled; }
  // The sampling penalties of dispatch lane `lane` for the steps encoded after (ops::SamplingPenalties; 1, 0, 0 turns them
  // off) and the table they read: lane l's row is words [l vocabulary, (l + 1) vocabulary) of penaltyWords(), which a
  // request that takes the lane uploads (ops::Sampling::rebuildPenaltyWords). A step that commits counts what a
  // penalized lane keeps into its row.
  void setPenalties(uint32_t lane, ops::SamplingPenalties penalties) { lanePolicies_.setPenalties(lane, penalties); }
  [[nodiscard]] const hip::Buffer &penaltyWords() { return lanePolicies_.words(); }
  // Dispatch lane `lane` of the steps encoded after admits only the tokens of its rows of tokenMask() (constrained), never
  // selects a stop token (excludesStopTokens); the step's stop tokens (SAMPLING_NO_TOKEN for none), at which acceptance
  // ends a lane's path (SamplingPolicy::constrained / excludesStopTokens, StopTokens in the reference's Sampling.hpp).
  void setAdmission(uint32_t lane, bool constrained, bool excludesStopTokens) { lanePolicies_.setAdmission(lane, constrained, excludesStopTokens); }
  void setStopTokens(const std::array<uint32_t, SAMPLING_STOP_TOKENS> &tokens) noexcept { lanePolicies_.setStopTokens(tokens); }
  [[nodiscard]] const hip::Buffer &tokenMask() { return lanePolicies_.tokenMask(maxRows_); }
  // The thinking cutoff of dispatch lane `lane` for the steps encoded after (ops::ThinkingCutoff; none clears it): its
  // rows from the cutoff's depth on select the end of thinking, between the step's selection and its acceptance.
  void setThinkingCutoff(uint32_t lane, std::optional<ops::ThinkingCutoff> cutoff) { lanePolicies_.setCutoff(lane, std::move(cutoff)); }
  // The hidden rows a draft's context is computed from (the reference's QwenTarget addCapture over RowCopy): after
  // layer layers[i] (ascending) every row's output goes to columns [i hidden, (i + 1) hidden) of its row of
  // `destination`, bf16 [rows][layers.size() x hidden], in a step and in a prompt chunk alike. An empty list captures nothing.
  void setCapture(std::vector<uint32_t> layers, hip::Buffer destination);
  [[nodiscard]] bool tiledGdnHeads() const noexcept { return tiledGdnHeads_; }

  void encode(hip::CommandGraph &graph, const std::vector<HybridLane> &lanes, bool commit = true);
  void encodeEmbedding(hip::CommandGraph &graph, uint32_t rows);
  // A layer (or the head) whose predecessor in the same graph left the table of its input rows, less their inverse
  // RMS, in the projection scratch passes `inputReady`; a layer that passes `feedsNext` leaves that table from its
  // combine. A part encoded on its own passes neither.
  void encodeLayer(hip::CommandGraph &graph, uint32_t layer, const std::vector<HybridLane> &lanes, bool inputReady = false,
                   bool feedsNext = false);
  void encodeHead(hip::CommandGraph &graph, uint32_t rows, bool inputReady = false);
  // A chunk of `tokens` prompt tokens (1 to prefillRows(); inputs where a step's are: tokens, a chain of tree rows a block
  // of sixteen, each row's depth in its block) of the sequence of lane `lane`, `committed` tokens already cached, through
  // layers [firstLayer, firstLayer + layerCount) (layerCount 0: to the last) and no head: the counterpart of the
  // reference's chunked prefill over its hybrid target (QwenTarget.cpp:206-347 with GDN::addPrefill, GDN.cpp:132-222, and
  // the plan over kv::ChunkedPrefillParams, PagedAttention.cpp:351-389). Attention layers store the chunk's keys and
  // values and attend causally (ops::PagedAttention::planChunks); Gated DeltaNet layers take every row into the state
  // (ops::GDN::addPrefill), from the lane's cell of `parity` to its other cell, so the lane's next step has the other
  // parity and no pending path. The embedding runs with firstLayer 0. Projections and experts run in windows of
  // ops::kMaximumDispatchRows rows.
  void encodePrefill(hip::CommandGraph &graph, uint32_t lane, uint32_t tableFirst, uint32_t committed, uint32_t tokens, uint32_t parity,
                     uint32_t firstLayer = 0, uint32_t layerCount = 0);

private:
  void encodePrefillLayer(hip::CommandGraph &graph, uint32_t layer, const ops::AttentionChunkPlan &plan, uint32_t tokens, uint64_t currentCell,
                          uint64_t nextCell);
  [[nodiscard]] ops::AttentionPlan planOf(const std::vector<HybridLane> &lanes) const;
  [[nodiscard]] hip::Buffer rowsOf(const hip::Buffer &buffer, uint32_t first, uint32_t count, uint64_t rowBytes) const {
    return backend_.view(buffer, first * rowBytes, count * rowBytes);
  }

  hip::Backend &backend_;
  HybridDimensions dims_;
  HybridWeights weights_;
  ops::Linear linear_;
  uint32_t maxRows_ = 0, maxLanes_ = 0, rowCapacity_ = 0;
  LanePolicies lanePolicies_;
  bool tiledGdnHeads_ = false;
  std::vector<uint32_t> captureLayers_;
  hip::Buffer captured_;
  void encodeCapture(hip::CommandGraph &graph, uint32_t layer, uint32_t rows) const;
  ops::GdnPrefillBuffers gdnPrefill_;  // the rows a GDN layer's prefill passes hand each other (a long chunk's)
  uint64_t pageBytes_ = 0, layerBytes_ = 0, cellBytes_ = 0, tapeLayerBytes_ = 0;
  ops::GdnStateStrides strides_;
  hip::Buffer kvAll_, states_, tape_;
  hip::Buffer hidden_[2], normalized_, packed_, mixed_, scores_, logits_, draft_;
  hip::Buffer mixedTable_;  // the activation table of the mixer's output rows, written by the mixer's last kernel
  hip::Buffer intermediate_, ffnTable_;  // a dense model's SwiGLU rows and their activation table
  hip::Buffer inverseFrequency_, ropeCos_, ropeSin_;
  hip::Buffer inputTokens_, treeRows_, depths_, uniforms_, tokens_, retained_, acceptedCount_, retainedRows_;
  hip::Buffer pageTable_;
  std::vector<hip::Buffer> kvPools_;
  ops::LinearScratch scratch_;
  ops::AttentionWorkspace attentionWorkspace_;
  ops::MoeWorkspace moeWorkspace_;
  ops::SamplingBuffers sampling_;
};

} // namespace splash::model
