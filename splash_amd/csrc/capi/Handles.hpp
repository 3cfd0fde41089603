// The C shim's opaque handles, shared by its translation units.
#pragma once
#include "splash_ops.h"
#include "hip/Backend.hpp"

struct spo_graph { splash::hip::CommandGraph graph; };

namespace splash::capi {
inline hip::CommandGraph &graphOf(spo_graph *graph) { return graph->graph; }
} // namespace splash::capi
