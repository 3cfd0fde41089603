// The C shim's opaque handles, shared by its translation units.
#pragma once
#include "splash_ops.h"
#include "hip/Backend.hpp"

#include "ops/Linear.hpp"

struct spo_graph { splash::hip::CommandGraph graph; };
struct spo_projection { splash::ops::Projection projection; };
struct spo_linear { splash::ops::Linear linear; };

namespace splash::capi {
inline hip::CommandGraph &graphOf(spo_graph *graph) { return graph->graph; }
inline const ops::Projection &projectionOf(const spo_projection *projection) { return projection->projection; }
} // namespace splash::capi
