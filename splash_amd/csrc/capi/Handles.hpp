// The C shim's opaque handles, shared by its translation units.
#pragma once
#include "splash_ops.h"
#include "hip/Backend.hpp"

#include "ops/Linear.hpp"
#include "ops/PagedAttention.hpp"

struct spo_graph { splash::hip::CommandGraph graph; };
struct spo_projection { splash::ops::Projection projection; };
struct spo_linear { splash::ops::Linear linear; };
struct spo_attention_plan { splash::ops::AttentionPlan plan; };
struct spo_attention_chunk_plan { splash::ops::AttentionChunkPlan plan; };

struct spg_file;
namespace splash::model {
class GgufFile;
}

namespace splash::capi {
// The parsed file behind a handle of include/splash_gguf.h.
const model::GgufFile &ggufOf(const spg_file *file);
inline hip::CommandGraph &graphOf(spo_graph *graph) { return graph->graph; }
inline const ops::Projection &projectionOf(const spo_projection *projection) { return projection->projection; }
} // namespace splash::capi
