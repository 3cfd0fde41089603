// The target part of one speculative-decoding cycle for a dense decoder: embedding -> N x
// {RMSNorm -> fused q|k|v -> q/k norm + RoPE + INT8 KV store -> paged attention -> o-proj + residual
// -> RMSNorm -> one-pass gate/up SwiGLU -> down + residual} -> final norm -> LM head (fp32 logits)
// -> verify (argmax or rejection sampling) -> acceptance -> KV path commit. It strings the operators
// together as the reference's model layer does (runtime/model/QwenTarget.cpp:206-395, :457-496 layer
// recipe; Runtime.cpp:2677-2717 encodeTargetDecodeForward, :2883-2892 encodeVerifyCommit) and owns
// the step's buffers; the residual stream ping-pongs between two hidden buffers.
#pragma once
#include "hip/Backend.hpp"
#include "model/LanePolicies.hpp"
#include "ops/Glue.hpp"
#include "ops/Linear.hpp"
#include "ops/PagedAttention.hpp"
#include "ops/Sampling.hpp"

#include <array>
#include <cstdint>
#include <optional>
#include <vector>

namespace splash::model {

struct DenseDimensions final {
  uint32_t hidden = 0, qHeads = 0, kvHeads = 0, headDimension = 0, ffn = 0, vocabulary = 0, layers = 0;
  uint32_t rotaryPairs = 0;
  bool normalizeHeads = true;   // per-head q/k RMS norm
  float ropeTheta = 1000000.0f;
  [[nodiscard]] uint32_t qkvWidth() const noexcept { return (qHeads + 2 * kvHeads) * headDimension; }
  [[nodiscard]] uint32_t attentionWidth() const noexcept { return qHeads * headDimension; }
};

struct DenseLayer final {
  ops::Projection qkv, output, gate, up, down;
  hip::Buffer inputNorm, postNorm, queryNorm, keyNorm;  // bf16 weights
};

struct DenseWeights final {
  ops::EmbeddingTable embedding;
  std::vector<DenseLayer> layers;
  hip::Buffer finalNorm;
  ops::Projection head;  // destination Float32
};

// One lane (request) of a step.
struct VerifyLane final {
  uint32_t rows = 0;        // rows of its verify block
  uint32_t committed = 0;   // tokens cached before the block
  uint32_t tableFirst = 0;  // its first page-table entry
  ops::SamplingPolicy policy;
  uint32_t remaining = 0xFFFFFFFFu;
};

class DenseVerify final {
public:
  // maxLanes x 16 rows a step at most; the KV pool holds `physicalPages` pages per layer. prefillRows: the most rows of
  // a prompt chunk (encodePrefill), 0 for a step's most, up to ops::kMaximumChunkRows; the rows' buffers are sized for it.
  DenseVerify(hip::Backend &backend, DenseDimensions dimensions, uint32_t maxLanes, uint32_t physicalPages,
              uint32_t pageTableEntries, uint32_t prefillRows = 0);
  [[nodiscard]] uint32_t prefillRows() const noexcept { return rowCapacity_; }

  [[nodiscard]] const DenseDimensions &dimensions() const noexcept { return dims_; }
  DenseWeights &weights() noexcept { return weights_; }
  // Host-visible step inputs and results (Shared storage).
  [[nodiscard]] const hip::Buffer &inputTokens() const noexcept { return inputTokens_; }
  [[nodiscard]] const hip::Buffer &treeRows() const noexcept { return treeRows_; }
  [[nodiscard]] const hip::Buffer &depths() const noexcept { return depths_; }
  [[nodiscard]] const hip::Buffer &uniforms() const noexcept { return uniforms_; }
  [[nodiscard]] const hip::Buffer &tokens() const noexcept { return tokens_; }
  [[nodiscard]] const hip::Buffer &retained() const noexcept { return retained_; }
  [[nodiscard]] const hip::Buffer &acceptedCount() const noexcept { return acceptedCount_; }
  [[nodiscard]] const hip::Buffer &retainedRows() const noexcept { return retainedRows_; }
  // Device buffers a host fills or inspects.
  [[nodiscard]] const hip::Buffer &pageTable() const noexcept { return pageTable_; }
  [[nodiscard]] const hip::Buffer &kvPool(uint32_t layer) const { return kvPools_.at(layer); }
  [[nodiscard]] const hip::Buffer &logits() const noexcept { return logits_; }
  [[nodiscard]] const hip::Buffer &draftProbabilities();  // allocated on first use
  // The sampled rows of tree blocks test the children their draft drew among sixteen candidates (Sampling.hpp,
  // candidateIds ..): the four host-visible buffers a draft writes, allocated on first use -- which: 0 ids uint32
  // [rows][16], 1 probabilities fp32 [rows][16], 2 drawn children bytes [rows][4], 3 child uniforms fp32 [rows][4].
  // Fetching them changes no step: setTestChildren chooses, for the steps encoded after it, whether sampled lanes
  // read them or the full-vocabulary draft probabilities (the default).
  [[nodiscard]] const hip::Buffer &candidateChildren(uint32_t which);
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
  void setTestChildren(bool on) { testChildren_ = on; if (on) (void)candidateChildren(0); }
  [[nodiscard]] bool testChildren() const noexcept { return testChildren_; }
  [[nodiscard]] const hip::Buffer &hidden(uint32_t index) const noexcept { return hidden_[index & 1]; }
  [[nodiscard]] const hip::Buffer &qkvRows() const noexcept { return qkv_; }
  [[nodiscard]] const hip::Buffer &attentionRows() const noexcept { return attention_; }
  [[nodiscard]] const hip::Buffer &ffnRows() const noexcept { return intermediate_; }
  [[nodiscard]] uint64_t pageBytes() const noexcept { return pageBytes_; }
  // Algorithmic bytes one step of `lanes` streams from HBM: weights once, each lane's KV, logits.
  [[nodiscard]] uint64_t stepBytes(const std::vector<VerifyLane> &lanes) const;

  // Appends the whole target part of a cycle to `graph`. `commit` adds the KV path commit.
  void encode(hip::CommandGraph &graph, const std::vector<VerifyLane> &lanes, bool commit = true);
  // Its parts, for per-kernel timing and tests.
  void encodeEmbedding(hip::CommandGraph &graph, uint32_t rows);
  // A layer (or the head) whose predecessor in the same graph left the table of its normalized input
  // in the projection scratch passes `inputReady`; a layer that passes `feedsNext` leaves that table
  // for its successor. A part encoded on its own passes neither.
  void encodeLayer(hip::CommandGraph &graph, uint32_t layer, const ops::AttentionPlan &plan, uint32_t rows,
                   bool inputReady = false, bool feedsNext = false);
  void encodeHead(hip::CommandGraph &graph, uint32_t rows, bool inputReady = false);
  // Whether every layer's down projection can norm its rows for the layer after it.
  [[nodiscard]] bool layersFeedNext(uint32_t rows) const noexcept;
  // A layer's four projections after its attention -- output, gate/up, down and the next layer's q|k|v (the LM head
  // after the last layer) -- leave as one dispatch (ops::Linear::addChain) where the shapes allow it: off by default.
  // The results are those of the separate dispatches, bit for bit.
  void setChained(bool chained) noexcept { chained_ = chained; }
  [[nodiscard]] bool chained() const noexcept { return chained_; }
  // A chunk of a sequence's prompt (1 to prefillRows() tokens, its input tokens, chain tree rows a block of sixteen and
  // depths where a step's are) in one pass over the layers: the chunk runs as blocks of sixteen rows of one sequence,
  // block i's history ending where block i - 1's rows end, through every layer and no head, so the tokens' keys and
  // values are in the pages and the hidden rows where a step leaves them. The counterpart of the reference's chunked
  // prefill (Runtime.cpp's prefill chunks over QwenTarget's layers) with the verify step's own kernels: the pools and
  // the hidden rows are those of the blocks run one step after the other, bit for bit. A chunk of more rows than a
  // step's runs layer by layer: the projections in windows of ops::kMaximumDispatchRows rows around one chunked
  // attention (ops::PagedAttention::planChunks) over all of them.
  void encodePrefill(hip::CommandGraph &graph, uint32_t tableFirst, uint32_t committed, uint32_t tokens);
  // A layer's q|k|v projection also prepares its attention block (ops::PagedAttention::addFusedProjection) where the
  // kernels take the pair: off by default (the projection and the prepare kernel run one after the other). The results
  // are the same bit for bit; on MI355X the one dispatch is the slower of the two at the 27B shape, since the workgroup
  // that completes a head prepares its sixteen rows alone (four a wave, about 4 us of vector arithmetic), where the
  // prepare kernel spreads them over 1280 workgroups.
  void setFusedPrepare(bool fused) noexcept { fusedPrepare_ = fused; }
  // A long prompt chunk (more rows than a step's) runs its projections through the prefill tile (ops::Linear::addPrefill:
  // 128 rows x 128 columns a workgroup under the staged rule, every weight rounded once to half), as the reference's
  // prompt chunks do (LinearTile::GgufPrefill, gguf_linear.metal:79-118): the norms and the SwiGLU are passes of their
  // own, the attention the same chunked plan. Off by default: a chunk then equals its blocks run as steps bit for bit;
  // on, it equals them to the staged rule's rounding and runs at the matrix cores' rate, not the step kernels'.
  // Every tensor's columns must be whole 128-column workgroups.
  void setStagedPrefill(bool staged);
  [[nodiscard]] bool stagedPrefill() const noexcept { return stagedPrefill_; }
  // The hidden rows a draft's context is computed from (the reference's QwenTarget addCapture over RowCopy,
  // RowCopy.hpp:17-28): after layer layers[i] (ascending), every row's output goes to columns [i hidden, (i + 1) hidden)
  // of its row of `destination`, bf16 [rows][layers.size() x hidden]; a step's rows and a prompt chunk's alike. A
  // capturing driver chains no projections. An empty list captures nothing.
  void setCapture(std::vector<uint32_t> layers, hip::Buffer destination);
  [[nodiscard]] bool fusedPrepare() const noexcept { return fusedPrepare_; }
  // Nonzero after a step in which a chained projection's wait for the one before it gave up: the step's results are
  // then not to be used. Reads the device's word (a copy of four bytes) and clears it.
  [[nodiscard]] uint32_t takeChainStatus();

private:
  hip::Backend &backend_;
  DenseDimensions dims_;
  DenseWeights weights_;
  ops::Linear linear_;
  uint32_t maxRows_ = 0, maxLanes_ = 0, rowCapacity_ = 0;
  LanePolicies lanePolicies_;
  uint64_t pageBytes_ = 0, layerBytes_ = 0;
  hip::Buffer kvAll_;
  hip::Buffer hidden_[2], normalized_, qkv_, attention_, intermediate_, logits_, draft_;
  hip::Buffer inverseFrequency_, ropeCos_, ropeSin_;
  hip::Buffer inputTokens_, treeRows_, depths_, uniforms_, tokens_, retained_, acceptedCount_, retainedRows_;
  hip::Buffer pageTable_;
  std::vector<hip::Buffer> kvPools_;
  ops::LinearScratch scratch_;
  hip::Buffer nextTable_;
  // chained projections: the gate/up and down tables, each link's partials and counters, the chain's progress words
  hip::Buffer chainTables_[2], chainProgress_;
  ops::LinearScratch chainScratch_[GGUF_CHAIN_LINKS];
  bool chained_ = false, encodedChains_ = false, fusedPrepare_ = false, testChildren_ = false;
  std::vector<uint32_t> captureLayers_;
  hip::Buffer captured_;
  void encodeCapture(hip::CommandGraph &graph, uint32_t layer, uint32_t rows) const;
  ops::SamplingBuffers children_;   // the four candidate-children buffers, bound into a step's sampling buffers when it tests them
  bool stagedPrefill_ = false;
  hip::Buffer prefillTable_, gateRows_, upRows_, swigluRows_;  // the staged prompt chunk's tables and SwiGLU rows
  void encodeStagedChunkLayer(hip::CommandGraph &graph, uint32_t layer, const ops::AttentionChunkPlan &plan, uint32_t tokens);
  hip::Buffer chunkAttentionTable_;  // a long chunk's attention rows as the output projection's tables, every window's
  void encodeChunkLayer(hip::CommandGraph &graph, uint32_t layer, const ops::AttentionChunkPlan &plan, uint32_t tokens, bool first,
                        bool feedsNext);
  void encodeChainedLayers(hip::CommandGraph &graph, const ops::AttentionPlan &plan, uint32_t rows);
  [[nodiscard]] bool chains(uint32_t rows) const noexcept;
  ops::AttentionWorkspace attentionWorkspace_;
  ops::SamplingBuffers sampling_;
  uint32_t maxSplits_ = 0;
};

} // namespace splash::model
