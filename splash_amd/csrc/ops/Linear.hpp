// Quantized projection planner and dispatcher for the verify step's 1..64-row blocks: the
// counterpart of the reference's ops::Linear (runtime/ops/Linear.hpp:138-376, LinearGguf.cpp) over
// the gfx950 MFMA tile (kernels/gguf_linear.hip). Same roles: a LinearPlan fixes tile height, K
// partitions and scratch; Linear::add validates every buffer and throws std::invalid_argument
// before any dispatch is added; producers and consumers hand the prepared activation table along
// as PreparedInput.
#pragma once
#include "abi/PagedAttention.h"

#include "abi/Gguf.h"
#include "hip/Backend.hpp"
#include "ops/Weights.hpp"

#include <algorithm>
#include <compare>
#include <cstdint>
#include <string>
#include <vector>

namespace splash::ops {

struct LinearMatrix final {
  uint32_t outputSize = 0;
  uint32_t inputSize = 0;
  auto operator<=>(const LinearMatrix &) const = default;
};

// Linear.hpp:77 in the reference; UpWithGate (its two-pass gate/up) has no use here: the MFMA tile
// runs every gate/up pair in one pass.
// ResidualNorm: the residual epilogue, and the RMS norm of its rows as the activation table of the
// projection after it (the reference's residual projections feed a norm_rms_table16 dispatch; here
// the projection's own workgroups write the table once every column group's sums of squares are in).
enum class LinearEpilogue : uint8_t { None, Residual, GateUp, ResidualNorm };
// 16-column MFMA tiles of 16/32/64 rows under one of two arithmetic rules: GgufMfma, the register rule (exact operands
// 128 + code, one fp32 multiply-add a group; the reference's Apple9 register tile), and GgufStaged, the staged rule
// (every weight decoded with fp32 group coefficients and rounded once to half, the products accumulated in fp32; the
// reference's staged tile, kernels/common/gguf_staged.h:12-66), which takes plain and residual plans of one format.
// GgufColumn: a plan of one or two rows under the reference's column rule (kernels/common/gguf_column_tile.h:25-68:
// half weights, every addition in a fixed order, eight parts of K), whose results are the reference's bit for bit;
// unsplit, every epilogue but the norming one, a dispatch a tensor. It reads the rows as they are, no activation table.
enum class LinearTile : uint8_t { GgufMfma, GgufStaged, GgufColumn };
inline constexpr uint32_t kMaximumDecodeTileRows = GGUF_MAXIMUM_ROWS;
// A dispatch of more rows runs pieces of kMaximumDecodeTileRows rows side by side.
inline constexpr uint32_t kMaximumDispatchRows = GGUF_MAXIMUM_DISPATCH_ROWS;

// The tile height that holds `rows` rows (the reference's stagedTileRows, Linear.hpp:118-120).
[[nodiscard]] constexpr uint32_t mfmaTileRows(uint32_t rows) noexcept { return rows <= 16 ? 16 : rows <= 32 ? 32 : 64; }
[[nodiscard]] constexpr uint32_t rowPieces(uint32_t rows) noexcept { return (rows + kMaximumDecodeTileRows - 1) / kMaximumDecodeTileRows; }

struct LinearWorkload final {
  LinearMatrix matrix;
  uint32_t rows = 0;
  LinearEpilogue epilogue = LinearEpilogue::None;
  // The widest record format among the projection's segments: it sets how many workgroups a
  // compute unit holds at once.
  uint32_t formatId = GGUF_FMT_Q4K;
  // Segments of different formats (one dispatch of the mixed kernel): whole 64-column workgroups a
  // segment, every workgroup one part of K, bf16 rows without an epilogue.
  bool severalFormats = false;
  auto operator<=>(const LinearWorkload &) const = default;
};

// A plan's workload for `rows` rows of a projection: its matrix, its segments' widest record format and
// whether they differ.
[[nodiscard]] LinearWorkload workloadOf(const Projection &projection, uint32_t rows, LinearEpilogue epilogue);

struct LinearConfig final {
  LinearTile tile = LinearTile::GgufMfma;
  // Cross-workgroup K partitions, 1 to kMaximumSplits.
  uint32_t splits = 1;
  static constexpr uint32_t kMaximumSplits = GGUF_MAXIMUM_SPLITS;
  // Leading workgroups (four column tiles each) that walk all of K themselves; only the
  // workgroups past them are partitioned. With G workgroups on C compute units, G - G % C whole
  // ones and the remainder partitioned C / (G % C) ways leaves every unit the same work.
  uint32_t wholeGroups = 0;
  [[nodiscard]] constexpr bool validSplits() const noexcept {
    return splits && splits <= kMaximumSplits;
  }
  bool operator==(const LinearConfig &) const = default;
};

// Reused serially within one command stream; counters are zeroed at allocation and restored by
// each completed split dispatch (Linear.hpp:183-196 in the reference).
struct LinearScratch final {
  hip::Buffer input;     // the activation table (values and sums, abi/Gguf.h)
  hip::Buffer partials;
  hip::Buffer counters;
};
struct LinearScratchSize final {
  uint64_t input = 0, partials = 0, counters = 0;
  LinearScratchSize &include(const LinearScratchSize &other) noexcept {
    input = std::max(input, other.input);
    partials = std::max(partials, other.partials);
    counters = std::max(counters, other.counters);
    return *this;
  }
};
struct SwiGluProjections final {
  const Projection *gate = nullptr;
  const Projection *up = nullptr;
  const Projection *down = nullptr;
};
// A block's buffers of its dense FFN: the intermediate rows and the linear scratch.
struct FfnBuffers final {
  hip::Buffer normalized, intermediate;
  LinearScratch scratch;
  // Optional second activation table: the gate/up pass then writes the down projection's table
  // from its epilogue and the separate table pass is dropped.
  hip::Buffer nextTable{};
  // Optional norm of the block's output rows: the down projection then also writes their RMS norm
  // under these weights as the activation table of the projection that follows the block.
  hip::Buffer followingNorm{}, followingTable{};
};

enum class LinearInput : uint8_t {
  Plain,    // bf16 [rows][K]
  Table16,  // the activation table of abi/Gguf.h
  // The table a ResidualNorm plan wrote: rows times the norm's weights, and the sums of squares
  // their inverse RMS comes from. The projection that reads it scales its own sums by that.
  TableUnscaled,
};
// The scratch table currently holds `source` in `layout` (Linear.hpp:250-256 in the reference).
struct PreparedInput final {
  hip::Buffer source;
  LinearInput layout = LinearInput::Plain;
};

class LinearPlan final {
public:
  [[nodiscard]] LinearWorkload workload() const noexcept { return workload_; }
  [[nodiscard]] LinearConfig configuration() const noexcept { return config_; }
  [[nodiscard]] FloatOutput destination() const noexcept { return destination_; }
  [[nodiscard]] uint32_t storageRows() const noexcept { return mfmaTileRows(workload_.rows); }
  [[nodiscard]] LinearInput input() const noexcept { return LinearInput::Table16; }
  [[nodiscard]] LinearScratchSize scratchSize() const noexcept;

private:
  friend class Linear;
  LinearPlan(LinearWorkload workload, LinearConfig config, FloatOutput destination = FloatOutput::BFloat16);
  void requireConfiguration() const;
  LinearWorkload workload_;
  LinearConfig config_;
  FloatOutput destination_;
};

struct LinearBuffers final {
  hip::Buffer input;
  hip::Buffer output;
  hip::Buffer residual;
  LinearScratch scratch{};
  PreparedInput prepared{};
  // Gate/up plans: where the epilogue also writes `output` as an activation table. ResidualNorm
  // plans: where it writes the normalized rows' table.
  hip::Buffer nextTable{};
  // ResidualNorm plans: the norm's weights, bf16 [output size].
  hip::Buffer normWeight{};
};

// What the plans read of the device (the reference's KernelCalibration, ops/KernelCalibration.hpp):
// measured on MI355X, overridable for sweeps.
struct KernelCalibration final {
  uint32_t computeUnits = 256;
  // Workgroups a compute unit holds at once (what the kernel's registers allow): a projection
  // partitions K until one round of them fills the device, and no further. Q6_K records keep more
  // registers live than Q4_K ones.
  uint32_t groupsPerUnit = 4;
  // Fewest super-blocks a workgroup's K range keeps.
  uint32_t minimumBlocksPerWave = 5;
  uint32_t groupsPerUnitQ6K = 3;
  // Polls of a chained projection's workgroup for the link before it (about a microsecond each) before it gives up.
  uint32_t chainSpinLimit = 1u << 16;
};

class Linear;
// One projection of a chain (Linear::addChain): what Linear::add takes.
struct ChainedProjection final {
  LinearBuffers buffers;
  const Projection *projection = nullptr;
  LinearPlan plan;
  const Projection *gate = nullptr;
};

// What the fused q|k|v projection binds of its attention block (kernels gguf_decode_qkv_*): attention_q8_qkv's buffers
// after the packed rows, in that kernel's order, and its parameters.
struct AttentionPrepareBindings final {
  hip::Buffer queryNorm, keyNorm, ropeCos, ropeSin, queries, querySums, pageTable, pool;
  AttentionParams params{};
};

class Linear final {
public:
  explicit Linear(const sp_device_info &device) noexcept;
  explicit Linear(KernelCalibration calibration) noexcept : calibration_(calibration) {}
  [[nodiscard]] const KernelCalibration &calibration() const noexcept { return calibration_; }

  [[nodiscard]] LinearPlan plan(LinearWorkload workload, FloatOutput destination = FloatOutput::BFloat16) const;
  [[nodiscard]] LinearPlan plan(const Projection &projection, uint32_t rows,
                                LinearEpilogue epilogue = LinearEpilogue::None) const;
  [[nodiscard]] static LinearPlan plan(LinearWorkload workload, LinearConfig config, FloatOutput destination);
  [[nodiscard]] uint32_t storageRows(uint32_t rows) const noexcept { return mfmaTileRows(rows); }
  // The scratch of every plan of up to `rows` rows of a projection of `matrix`, every epilogue.
  [[nodiscard]] LinearScratchSize scratchSize(LinearMatrix matrix, uint32_t rows) const;

  // Writes the activation table of `rows` rows of `input` into scratch.input.
  static void addPrepare(hip::CommandGraph &graph, const hip::Buffer &input, const LinearScratch &scratch, uint32_t width,
                         uint32_t rows);
  // Returns what the scratch table describes after the dispatch.
  PreparedInput add(hip::CommandGraph &graph, LinearBuffers buffers, const Projection &projection,
                    const LinearPlan &plan, const Projection *gate = nullptr) const;
  // Up to four projections of up to 64 rows as one dispatch, each reading what the one before it wrote (the table its
  // epilogue leaves, the residual rows): the next link's workgroups fetch their first weights while the link before
  // them drains, and wait for its count of finished workgroups instead of a kernel boundary. Every link's input is
  // prepared (a table that exists or that the link before writes), its table, partials and counters are its own, and
  // `progress` (GGUF_CHAIN_PROGRESS_WORDS words, zero before the first dispatch) is the chain's; its last word reads
  // nonzero after a dispatch in which a wait gave up.
  void addChain(hip::CommandGraph &graph, std::vector<ChainedProjection> links, const hip::Buffer &progress) const;
  // The q|k|v projection of an attention block with the block's head norms, RoPE, query staging and cache store as its
  // epilogue (GGUF_EPILOGUE_QKV_PREPARE), in place of the projection and attention_q8_qkv after it: the same packed
  // rows, staged queries and cache bytes. preparesAttention: whether the kernels take the pair (a plain bf16 plan of one
  // piece of rows whose workgroups all take a part of K, heads of 64 or 128 dimensions that lie whole in the
  // projection's segments, fp16 queries, no gates). The dispatch keeps partials and counters whatever the plan's parts
  // (attentionScratchSize).
  [[nodiscard]] static bool preparesAttention(const Projection &projection, const LinearPlan &plan, const AttentionParams &attention) noexcept;
  [[nodiscard]] static LinearScratchSize attentionScratchSize(const LinearPlan &plan) noexcept;
  PreparedInput addWithAttention(hip::CommandGraph &graph, LinearBuffers buffers, const Projection &projection,
                                 const LinearPlan &plan, const AttentionPrepareBindings &attention) const;
  // A chunk of many rows (a prompt's, up to kMaximumPrefillRows) under the staged rule, a workgroup 128 rows x 128
  // columns with K whole (kernels gguf_prefill_*; the reference's prefill tile, gguf_linear.metal:79-118, and
  // LinearTile::GgufPrefill): output = bf16 or fp32 (the projection's destination) of input x W^T, plus the residual
  // rows when `residual` names them. Every segment's columns are a multiple of 128. `table` holds the rows'
  // activation tables (prefillTableBytes), which the dispatch writes first.
  static constexpr uint32_t kMaximumPrefillRows = 16384;
  [[nodiscard]] static uint64_t prefillTableBytes(uint32_t inputSize, uint32_t rows) noexcept;
  static void addPrefill(hip::CommandGraph &graph, const hip::Buffer &input, const Projection &projection, const hip::Buffer &output,
                         const hip::Buffer &residual, const hip::Buffer &table, uint32_t rows);
  void addProjection(hip::CommandGraph &graph, hip::Buffer input, const Projection &projection, hip::Buffer output,
                     uint32_t rows, LinearScratch scratch) const;
  void addResidualProjection(hip::CommandGraph &graph, hip::Buffer input, const Projection &projection,
                             hip::Buffer residual, hip::Buffer output, uint32_t rows, LinearScratch scratch) const;
  // Whether a residual projection of this shape may also norm its rows (LinearEpilogue::ResidualNorm).
  [[nodiscard]] bool normsRows(const Projection &projection, uint32_t rows) const noexcept;
  // output = residual + down(silu(gate x) * up x) of `rows` normalized rows.
  void addSwiGlu(hip::CommandGraph &graph, const SwiGluProjections &ffn, const FfnBuffers &buffers, hip::Buffer residual,
                 hip::Buffer output, uint32_t rows, PreparedInput normalized = {}) const;

private:
  struct Resolved;
  PreparedInput addColumn(hip::CommandGraph &graph, LinearBuffers buffers, const Projection &projection, const LinearPlan &plan,
                          const Projection *gate) const;
  [[nodiscard]] Resolved resolve(LinearBuffers buffers, const Projection &projection, const LinearPlan &plan,
                                 const Projection *gate) const;
  KernelCalibration calibration_;
};

// Throws std::invalid_argument unless `buffer` holds `bytes` bytes ("<what> buffer is too small").
void requireBytes(const hip::Buffer &buffer, uint64_t bytes, const char *what);

} // namespace splash::ops
