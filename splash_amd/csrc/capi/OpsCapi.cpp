// The C entry points of include/splash_ops.h over the C++ operators.
#include "splash_ops.h"
#include "backend/Internal.hpp"
#include "capi/Guard.hpp"
#include "capi/Handles.hpp"
#include "ops/GgufImage.hpp"
#include "ops/Linear.hpp"

#include <cstring>

using namespace splash;



namespace {
ops::LinearPlan toPlan(const ops::Projection &projection, const spo_linear_plan &p) {
  if (p.epilogue > 3) throw std::invalid_argument("unknown linear epilogue");
  ops::LinearConfig config;
  config.splits = p.splits;
  config.wholeGroups = p.whole_groups;
  if (p.tile > 2) throw std::invalid_argument("unknown linear tile");
  config.tile = static_cast<ops::LinearTile>(p.tile);
  return ops::Linear::plan(ops::workloadOf(projection, p.rows, static_cast<ops::LinearEpilogue>(p.epilogue)), config,
                           p.float32 ? ops::FloatOutput::Float32 : ops::FloatOutput::BFloat16);
}
void fromPlan(const ops::LinearPlan &plan, spo_linear_plan *out) {
  const ops::LinearScratchSize size = plan.scratchSize();
  out->rows = plan.workload().rows;
  out->epilogue = uint32_t(plan.workload().epilogue);
  out->splits = plan.configuration().splits;
  out->whole_groups = plan.configuration().wholeGroups;
  out->storage_rows = plan.storageRows();
  out->float32 = plan.destination() == ops::FloatOutput::Float32;
  out->tile = uint32_t(plan.configuration().tile);
  out->reserved = 0;
  out->scratch_input = size.input;
  out->scratch_partials = size.partials;
  out->scratch_counters = size.counters;
}
ops::LinearScratch scratchOf(sp_buffer *table, sp_buffer *partials, sp_buffer *counters) {
  return {hip::Buffer::share(table), hip::Buffer::share(partials), hip::Buffer::share(counters)};
}
} // namespace

extern "C" {

sp_status spo_graph_create(spo_graph **out) {
  return capi::guard([&] { capi::require(out, "result"); *out = new spo_graph; });
}
void spo_graph_destroy(spo_graph *graph) { delete graph; }
uint32_t spo_graph_size(const spo_graph *graph) { return graph ? uint32_t(graph->graph.size()) : 0; }
size_t spo_graph_kernel(const spo_graph *graph, uint32_t index, char *out, size_t capacity) {
  if (!graph || index >= graph->graph.size()) return 0;
  const std::string &name = graph->graph.dispatches()[index].pipelineName;
  if (out && capacity) {
    const size_t n = std::min(capacity - 1, name.size());
    std::memcpy(out, name.data(), n);
    out[n] = 0;
  }
  return name.size() + 1;
}
sp_status spo_graph_add(spo_graph *graph, const char *kernel, sp_buffer *const *buffers, uint32_t buffer_count,
                        const void *params, uint32_t params_bytes, const uint32_t grid[3], const uint32_t block[3]) {
  return capi::guard([&] {
    capi::require(graph && kernel && grid && block && params && params_bytes, "graph, kernel, grid, block or params");
    if (params_bytes > 256) throw std::invalid_argument("parameter structs are at most 256 bytes");
    struct Blob { unsigned char bytes[256]; } blob{};
    std::memcpy(blob.bytes, params, params_bytes);
    std::vector<hip::Buffer> bound;
    for (uint32_t i = 0; i < buffer_count; ++i) bound.push_back(hip::Buffer::share(buffers[i]));
    graph->graph.add(kernel, std::move(bound), blob, {grid[0], grid[1], grid[2]}, {block[0], block[1], block[2]});
    // The graph copied sizeof(Blob) bytes; the dispatch binds the struct's own size.
    const_cast<hip::ComputeDispatch &>(graph->graph.dispatches().back()).bytesSize = params_bytes;
  });
}
sp_status spo_graph_submit(sp_backend *backend, const spo_graph *graph, sp_ticket **out) {
  if (!backend || !graph || !out) return capi::guard([] { capi::require(false, "backend, graph or result"); });
  // The backend's own status (SP_BUSY, SP_UNKNOWN_KERNEL, ...) and message pass through unchanged.
  hip::LoweredDispatches lowered(graph->graph.dispatches());
  return sp_submit(backend, lowered.records.data(), uint32_t(lowered.records.size()), nullptr, nullptr, out);
}
sp_status spo_graph_record(sp_backend *backend, const spo_graph *graph, sp_command **out) {
  if (!backend || !graph || !out) return capi::guard([] { capi::require(false, "backend, graph or result"); });
  hip::LoweredDispatches lowered(graph->graph.dispatches());
  return sp_command_create(backend, lowered.records.data(), uint32_t(lowered.records.size()), out);
}

uint64_t spo_gguf_image_bytes(uint32_t format, uint32_t rows, uint32_t input_size) {
  return gguf_image_bytes(format, rows, input_size);
}
uint64_t spo_gguf_table_bytes(uint32_t input_size, uint32_t rows) { return gguf_tables_bytes(input_size, gguf_row_tiles(rows)); }
sp_status spo_gguf_pack_image(uint32_t format, const uint8_t *native, uint32_t rows, uint32_t input_size, uint8_t *image) {
  return capi::guard([&] { capi::require(native && image, "rows or image"); ops::packGgufImage(format, native, rows, input_size, image); });
}
sp_status spo_gguf_unpack_image(uint32_t format, const uint8_t *image, uint32_t rows, uint32_t input_size, uint8_t *native) {
  return capi::guard([&] { capi::require(native && image, "rows or image"); ops::unpackGgufImage(format, image, rows, input_size, native); });
}
uint32_t spo_gguf_rewrite_format(uint32_t ggml_type) {
  const ops::NativeRewrite *rewrite = ops::nativeRewriteOf(ggml_type);
  return rewrite ? rewrite->imageFormat : 0xFFFFFFFFu;
}
sp_status spo_gguf_rewrite(uint32_t ggml_type, const uint8_t *source, uint64_t super_blocks, uint8_t *out) {
  return capi::guard([&] { capi::require(source && out, "blocks"); ops::rewriteNative(ggml_type, source, super_blocks, out); });
}
sp_status spo_gguf_add_dequant(spo_graph *graph, uint32_t format, sp_buffer *image, sp_buffer *out, uint32_t rows,
                               uint32_t input_size) {
  return capi::guard([&] {
    capi::require(graph && image && out, "graph or buffers");
    if (!gguf_record_bytes(format) || !rows || rows % 16 || !input_size || input_size % 256)
      throw std::invalid_argument("a weight image holds whole tiles of a K-quant format");
    ops::requireBytes(hip::Buffer::share(image), gguf_image_bytes(format, rows, input_size), "weight image");
    ops::requireBytes(hip::Buffer::share(out), uint64_t{rows} * input_size * 4, "dequantized values");
    graph->graph.add(std::string("gguf_dequant_") + gguf_format_name(format),
                     {hip::Buffer::share(image), hip::Buffer::share(out)}, GgufDequantParams{input_size, rows},
                     {input_size / 256, rows / 16, 1}, {64, 1, 1});
  });
}

sp_status spo_projection_create(uint32_t segments, const uint32_t *formats, const uint32_t *output_sizes, uint32_t input_size,
                                sp_buffer *const *images, int float32_destination, spo_projection **out) {
  return capi::guard([&] {
    capi::require(formats && output_sizes && images && out, "segments or result");
    ops::BlockWeights weights;
    uint32_t covered = 0;
    for (uint32_t s = 0; s < segments; ++s) {
      weights.segments.push_back(ops::QuantizedSegment::ofImage(formats[s], output_sizes[s], input_size,
                                                              hip::Buffer::share(images[s]), covered));
      covered += output_sizes[s];
    }
    auto *p = new spo_projection{ops::Projection(covered, input_size, std::move(weights))};
    p->projection.destination = float32_destination ? ops::FloatOutput::Float32 : ops::FloatOutput::BFloat16;
    *out = p;
  });
}
sp_status spo_projection_rows(const spo_projection *projection, const uint32_t *firsts, const uint32_t *counts, uint32_t ranges,
                              spo_projection **out) {
  return capi::guard([&] {
    capi::require(projection && firsts && counts && out, "projection, ranges or result");
    if (!ranges || ranges > 2) throw std::invalid_argument("a row view takes one or two ranges");
    const ops::Projection &p = projection->projection;
    *out = new spo_projection{ranges == 1 ? p.rows({{firsts[0], counts[0]}}) : p.rows({{firsts[0], counts[0]}, {firsts[1], counts[1]}})};
  });
}
void spo_projection_destroy(spo_projection *projection) { delete projection; }
uint64_t spo_projection_weight_bytes(const spo_projection *projection) {
  return projection ? projection->projection.weightBytes() : 0;
}

sp_status spo_linear_create(sp_backend *backend, spo_linear **out) {
  return capi::guard([&] {
    capi::require(backend && out, "backend or result");
    sp_device_info info{};
    hip::throwStatus(sp_backend_device_info(backend, &info));
    *out = new spo_linear{ops::Linear(info)};
  });
}
sp_status spo_linear_create_calibrated(uint32_t compute_units, uint32_t groups_per_unit, uint32_t minimum_blocks_per_wave,
                                       spo_linear **out) {
  return capi::guard([&] {
    capi::require(out, "result");
    if (!compute_units || !groups_per_unit || !minimum_blocks_per_wave) throw std::invalid_argument("a calibration has no zero entry");
    ops::KernelCalibration calibration{compute_units, groups_per_unit, minimum_blocks_per_wave};
    calibration.groupsPerUnitQ6K = std::min(calibration.groupsPerUnitQ6K, groups_per_unit);
    *out = new spo_linear{ops::Linear(calibration)};
  });
}
void spo_linear_destroy(spo_linear *linear) { delete linear; }
sp_status spo_linear_set_chain_spin_limit(spo_linear *linear, uint32_t polls) {
  return capi::guard([&] {
    capi::require(linear, "linear");
    ops::KernelCalibration calibration = linear->linear.calibration();
    calibration.chainSpinLimit = polls;
    linear->linear = ops::Linear(calibration);
  });
}

sp_status spo_linear_plan_for(const spo_linear *linear, const spo_projection *projection, uint32_t rows, uint32_t epilogue,
                              spo_linear_plan *out) {
  return capi::guard([&] {
    capi::require(linear && projection && out, "linear, projection or result");
    if (epilogue > 3) throw std::invalid_argument("unknown linear epilogue");
    fromPlan(linear->linear.plan(projection->projection, rows, static_cast<ops::LinearEpilogue>(epilogue)), out);
  });
}
sp_status spo_linear_plan_with(const spo_projection *projection, spo_linear_plan *plan) {
  return capi::guard([&] {
    capi::require(projection && plan, "projection or plan");
    fromPlan(toPlan(projection->projection, *plan), plan);
  });
}
sp_status spo_linear_add(const spo_linear *linear, spo_graph *graph, const spo_projection *projection,
                         const spo_projection *gate, const spo_linear_plan *plan, sp_buffer *input, sp_buffer *output,
                         sp_buffer *residual, sp_buffer *table, sp_buffer *partials, sp_buffer *counters, int prepared) {
  return capi::guard([&] {
    capi::require(linear && graph && projection && plan, "linear, graph, projection or plan");
    ops::LinearBuffers buffers;
    buffers.input = hip::Buffer::share(input);
    buffers.output = hip::Buffer::share(output);
    buffers.residual = hip::Buffer::share(residual);
    buffers.scratch = scratchOf(table, partials, counters);
    if (prepared) buffers.prepared = {buffers.input, prepared == 2 ? ops::LinearInput::TableUnscaled : ops::LinearInput::Table16};
    linear->linear.add(graph->graph, std::move(buffers), projection->projection, toPlan(projection->projection, *plan),
                       gate ? &gate->projection : nullptr);
  });
}
sp_status spo_linear_add_residual_norm(const spo_linear *linear, spo_graph *graph, const spo_projection *projection,
                                       const spo_linear_plan *plan, sp_buffer *input, sp_buffer *output, sp_buffer *residual,
                                       sp_buffer *norm_weight, sp_buffer *next_table, sp_buffer *table, sp_buffer *partials,
                                       sp_buffer *counters, int prepared) {
  return capi::guard([&] {
    capi::require(linear && graph && projection && plan, "linear, graph, projection or plan");
    ops::LinearBuffers buffers;
    buffers.input = hip::Buffer::share(input);
    buffers.output = hip::Buffer::share(output);
    buffers.residual = hip::Buffer::share(residual);
    buffers.normWeight = hip::Buffer::share(norm_weight);
    buffers.nextTable = hip::Buffer::share(next_table);
    buffers.scratch = scratchOf(table, partials, counters);
    if (prepared) buffers.prepared = {buffers.input, prepared == 2 ? ops::LinearInput::TableUnscaled : ops::LinearInput::Table16};
    const ops::LinearPlan full = toPlan(projection->projection, *plan);
    if (full.workload().epilogue != ops::LinearEpilogue::ResidualNorm) throw std::invalid_argument("the plan does not norm its rows");
    linear->linear.add(graph->graph, std::move(buffers), projection->projection, full);
  });
}
extern "C++" {
namespace {
ops::ChainedProjection linkOf(const spo_chain_link &l) {
  capi::require(l.projection, "a link's projection");
  ops::LinearBuffers buffers;
  buffers.input = hip::Buffer::share(l.input);
  buffers.output = hip::Buffer::share(l.output);
  buffers.residual = hip::Buffer::share(l.residual);
  buffers.normWeight = hip::Buffer::share(l.norm_weight);
  buffers.nextTable = hip::Buffer::share(l.next_table);
  buffers.scratch = scratchOf(l.table, l.partials, l.counters);
  if (l.prepared) buffers.prepared = {buffers.input, l.prepared == 2 ? ops::LinearInput::TableUnscaled : ops::LinearInput::Table16};
  return {std::move(buffers), &l.projection->projection, toPlan(l.projection->projection, l.plan), l.gate ? &l.gate->projection : nullptr};
}
} // namespace
} // extern "C++"
sp_status spo_linear_add_chain(const spo_linear *linear, spo_graph *graph, const spo_chain_link *links, uint32_t count,
                               sp_buffer *progress) {
  return capi::guard([&] {
    capi::require(linear && graph && links && progress, "linear, graph, links or progress");
    std::vector<ops::ChainedProjection> chain;
    for (uint32_t i = 0; i < count; ++i) chain.push_back(linkOf(links[i]));
    linear->linear.addChain(graph->graph, std::move(chain), hip::Buffer::share(progress));
  });
}
sp_status spo_linear_add_link(const spo_linear *linear, spo_graph *graph, const spo_chain_link *link) {
  return capi::guard([&] {
    capi::require(linear && graph && link, "linear, graph or link");
    ops::ChainedProjection one = linkOf(*link);
    linear->linear.add(graph->graph, std::move(one.buffers), *one.projection, one.plan, one.gate);
  });
}
int spo_attention_fuses_projection(const spo_attention_plan *plan, const spo_projection *projection, const spo_linear_plan *linear_plan) {
  if (!plan || !projection || !linear_plan) return 0;
  try {
    return ops::PagedAttention::fusesProjection(plan->plan, projection->projection, toPlan(projection->projection, *linear_plan)) ? 1 : 0;
  } catch (...) {
    return 0;
  }
}
sp_status spo_attention_add_fused_projection(const spo_linear *linear, spo_graph *graph, const spo_chain_link *qkv,
                                             const spo_attention_plan *plan, sp_buffer *query_norm, sp_buffer *key_norm,
                                             sp_buffer *rope_cos, sp_buffer *rope_sin, sp_buffer *queries, sp_buffer *query_sums,
                                             sp_buffer *page_table, sp_buffer *pool, uint64_t page_bytes) {
  return capi::guard([&] {
    capi::require(linear && graph && qkv && plan, "linear, graph, projection or plan");
    ops::ChainedProjection one = linkOf(*qkv);
    ops::AttentionProjectionBuffers b{one.buffers.output, hip::Buffer::share(query_norm), hip::Buffer::share(key_norm),
                                      hip::Buffer::share(rope_cos), hip::Buffer::share(rope_sin)};
    ops::AttentionWorkspace w{hip::Buffer::share(queries), hip::Buffer::share(query_sums), {}, {}};
    ops::PagedAttention::addFusedProjection(graph->graph, linear->linear, std::move(one.buffers), *one.projection, one.plan, plan->plan, b, w,
                                            ops::KvPages{hip::Buffer::share(page_table), hip::Buffer::share(pool), page_bytes});
  });
}
sp_status spo_linear_add_swiglu(const spo_linear *linear, spo_graph *graph, const spo_projection *gate,
                                const spo_projection *up, const spo_projection *down, sp_buffer *normalized,
                                sp_buffer *intermediate, sp_buffer *residual, sp_buffer *output, uint32_t rows,
                                sp_buffer *table, sp_buffer *partials, sp_buffer *counters, sp_buffer *next_table) {
  return capi::guard([&] {
    capi::require(linear && graph && gate && up && down, "linear, graph or projections");
    ops::FfnBuffers buffers{hip::Buffer::share(normalized), hip::Buffer::share(intermediate), scratchOf(table, partials, counters),
                            hip::Buffer::share(next_table)};
    linear->linear.addSwiGlu(graph->graph, {&gate->projection, &up->projection, &down->projection}, buffers,
                             hip::Buffer::share(residual), hip::Buffer::share(output), rows);
  });
}
uint64_t spo_linear_prefill_table_bytes(uint32_t input_size, uint32_t rows) {
  return input_size && input_size % GGUF_BLOCK == 0 && rows ? ops::Linear::prefillTableBytes(input_size, rows) : 0;
}
sp_status spo_linear_add_prefill(spo_graph *graph, const spo_projection *projection, sp_buffer *input, sp_buffer *output,
                                 sp_buffer *residual, sp_buffer *table, uint32_t rows) {
  return capi::guard([&] {
    capi::require(graph && projection, "graph or projection");
    ops::Linear::addPrefill(graph->graph, hip::Buffer::share(input), projection->projection, hip::Buffer::share(output),
                            hip::Buffer::share(residual), hip::Buffer::share(table), rows);
  });
}
sp_status spo_linear_scratch_size(const spo_linear *linear, uint32_t output_size, uint32_t input_size, uint32_t rows,
                                  uint64_t *table, uint64_t *partials, uint64_t *counters) {
  return capi::guard([&] {
    capi::require(linear, "linear");
    const ops::LinearScratchSize size = linear->linear.scratchSize({output_size, input_size}, rows);
    if (table) *table = size.input;
    if (partials) *partials = size.partials;
    if (counters) *counters = size.counters;
  });
}

} // extern "C"
