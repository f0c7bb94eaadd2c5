// Graph-to-graph optimizer kept from the reference pipeline (kn-graph/src/optimizer/mod.rs:11-57).
#pragma once

#include "graph.h"

namespace kn {

struct OptimizerSettings {
    bool optimize = true;
    bool force_bias_through_conv = false;
    bool fuse_layernorm = true;
    bool div_to_mul = true;
};

Graph optimize_graph(const Graph &graph, const OptimizerSettings &settings);

}  // namespace kn
