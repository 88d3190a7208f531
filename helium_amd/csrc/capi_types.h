// Definitions of the opaque handle types shared by the C-ABI translation units.
#pragma once
#include <mutex>
#include <memory>

#include "exec.h"
#include "fusion_ir.h"
#include "ir.h"
#include "kernels.h"

struct he_graph_s {
    std::shared_ptr<he::ir::OpGraph> g = std::make_shared<he::ir::OpGraph>();
    // What he_execute_graph prepared on an earlier call (optimised copy and its plan), valid while the graph has
    // `prepared_nodes` nodes and the backend options are `prepared_options`; the fields are guarded by `mu`.
    std::mutex mu;
    std::shared_ptr<const he::exec::Prepared> prepared;
    size_t prepared_nodes = 0;
    uint64_t prepared_options = 0;
};
struct he_fgraph_s {
    he::fir::OpGraph g;
};
struct he_tile_kernel_s {
    std::shared_ptr<he::KernelBase> k;  // shared with the plan when the handle came from he_plan_instruction_kernel
};
