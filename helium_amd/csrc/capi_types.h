// Definitions of the opaque handle types shared by the C-ABI translation units.
#pragma once
#include <memory>

#include "fusion_ir.h"
#include "ir.h"
#include "kernels.h"

struct he_graph_s {
    std::shared_ptr<he::ir::OpGraph> g = std::make_shared<he::ir::OpGraph>();
};
struct he_fgraph_s {
    he::fir::OpGraph g;
};
struct he_tile_kernel_s {
    std::unique_ptr<he::KernelBase> k;
};
