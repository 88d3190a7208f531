// Plan generation for a helium-ir graph: one instruction per op, greedy pairwise fusion, level-ised steps, late
// scheduling and tensor lifetimes — helium/src/backend/plan_generation.rs, with the HIP backend's op -> instruction
// mapping (helium/src/cuda.rs:33-60) and its instruction kinds (helium/src/cuda/instr.rs).
#pragma once
#include <atomic>
#include <functional>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "ir.h"
#include "kernels.h"
#include "permute.h"

namespace he::plan {

using ir::NodeId;

enum class InstrKind : int { Gemm = 0, Pointwise = 1, Permute = 2 };

// SwapDims nodes with more elements than this become Permute instructions (cuda.rs:38-41).
constexpr int64_t kPermuteThreshold = 1000000;

class Instr {
public:
    Instr(InstrKind kind, ir::OpSubgraph sg) : kind_(kind), sg_(std::move(sg)) {}
    Instr(const Instr& o) : kind_(o.kind_), sg_(o.sg_), kernel_(o.kernel_), permute_(o.permute_) {}
    InstrKind kind() const { return kind_; }
    const ir::OpSubgraph& subgraph() const { return sg_; }
    std::vector<NodeId> inputs() const { return sg_.inputs(); }   // Instruction::inputs (backend.rs:86)
    std::vector<NodeId> outputs() const { return sg_.leafs(); }   // Instruction::outputs (backend.rs:87)
    bool can_fuse_with(const Instr& next) const;                   // instr.rs:71-84
    Instr fuse_with(const Instr& next) const;                      // instr.rs:86-99

    // precompile (instr.rs:44-51): builds (or fetches from the kernel cache) the compiled kernel.
    void precompile() const;
    bool compiled() const {
        std::lock_guard<std::mutex> lk(mu_);
        return kernel_ || permute_ || absorbed_;
    }
    // execute (instr.rs:27-42): `storage(node)` returns the device address of a tensor.
    void execute(const std::function<void*(NodeId)>& storage, hipStream_t stream) const;
    std::string describe(bool origins = true) const;  // origins: name nodes by OpGraph::origin

    // Beyond the reference: `small` (a pointwise instruction over the columns of this instruction's column reductions:
    // the per-channel arithmetic behind a batch norm's sums) is evaluated by the launch that folds those reductions.
    // It stays in the plan where it was and launches nothing; this instruction's execution needs its inputs and
    // writes its outputs as well.
    void carry(const std::shared_ptr<Instr>& small) {
        carried_ = small;
        small->absorbed_ = true;
    }
    const std::shared_ptr<Instr>& carried() const { return carried_; }
    bool absorbed() const { return absorbed_; }
    // The compiled kernel (compiling it if need be); null for a permute instruction and an absorbed one.
    std::shared_ptr<KernelBase> kernel() const {
        precompile();
        std::lock_guard<std::mutex> lk(mu_);
        return kernel_;
    }
    // Beyond the reference: the executor runs this instruction on its side stream, beside the chain of instructions
    // that everything else waits for (exec.cpp: side_stream_split). Told before the kernel is made, a filter gradient
    // then splits its k range over fewer workgroups: it has time, and the CUs it leaves alone keep the main chain going.
    void runs_beside_main_chain() const { beside_main_.store(true); }
    bool beside_main_chain() const { return beside_main_.load(); }
    std::vector<NodeId> all_inputs() const;   // inputs() plus what the carried instruction reads from elsewhere
    std::vector<NodeId> all_outputs() const;  // outputs() plus the carried instruction's

private:
    std::shared_ptr<Instr> carried_;
    bool absorbed_ = false;
    mutable std::atomic<bool> beside_main_{false};
    InstrKind kind_;
    ir::OpSubgraph sg_;
    mutable std::shared_ptr<KernelBase> kernel_;   // Gemm / Pointwise
    mutable std::shared_ptr<Permute> permute_;     // Permute
    mutable std::mutex mu_;
};

// enumerate_swaps (permute_dims.rs:112-142): the chain of (axis_a, axis_b) when the subgraph is a linear chain of
// SwapDims on one input; empty optional-like flag otherwise.
bool enumerate_swaps(const ir::OpSubgraph& sg, std::vector<std::pair<int, int>>* swaps);

Instr make_instr_for_op(const std::shared_ptr<const ir::OpGraph>& g, NodeId node);  // cuda.rs:33-60

struct Step {
    std::vector<std::shared_ptr<Instr>> instrs;
    std::vector<NodeId> tensors_to_release;
    // The instructions must run one after the other, in this order: one of them carries an instruction that reads what
    // an earlier one of the same step writes.
    bool in_order = false;
};
struct Plan {
    std::vector<Step> steps;
    std::string describe(bool origins = true) const;  // one line per step: instruction kinds, node sets, releases
};

// Whether pointwise / reduce ops downstream of a Matmul may join its instruction (on by default). Off gives the
// reference's grouping, where a matmul instruction never fuses.
void set_fuse_matmul_epilogue(bool on);
bool fuse_matmul_epilogue();
// Whether a large SwapDims whose values all end in reductions stays in the pointwise instruction instead of becoming
// a permute instruction of its own (on by default). Off gives the reference's choice by element count alone.
uint64_t option_mask();  // the options above as bits: what a generated plan depends on besides the graph
void set_fold_swap_into_reduce(bool on);
bool fold_swap_into_reduce();

// Whether values that are cheap to compute again are computed per use instead of travelling through memory
// (ir::rematerialized; on by default, off plans the graph as recorded, like the reference).
void set_rematerialize(bool on);
bool rematerialize();
// Whether transpositions that undo each other are taken out of the graph first (ir::transposes_cancelled; on by default).
void set_cancel_transposes(bool on);
bool cancel_transposes();
// Whether pointwise ops whose operands are all one broadcast are applied before it (ir::broadcasts_hoisted; on by default).
void set_hoist_broadcasts(bool on);
bool hoist_broadcasts();
// True when every value computed from `node` ends in a Reduce, through pointwise ops only.
bool feeds_only_reductions(const ir::OpGraph& g, ir::NodeId node, int budget = 64);
// Bytes the plan's kernels read and write: the sizes of every instruction's inputs and outputs.
int64_t plan_traffic_bytes(const Plan& plan);
// The graph the backend plans and runs for `g` (already pruned): `g` itself, or the form the two rewrites above give it
// when that form's plan moves fewer bytes. Input and Output nodes of the result map back through OpGraph::origin.
std::shared_ptr<const ir::OpGraph> graph_for_execution(const std::shared_ptr<const ir::OpGraph>& g);

// generate_plan (plan_generation.rs:22-26).
std::shared_ptr<const Plan> generate_plan(const std::shared_ptr<const ir::OpGraph>& g);
// generate_cached_plan (:16-19): LRU of 256 plans keyed by the graph's structure.
std::shared_ptr<const Plan> generate_cached_plan(const std::shared_ptr<const ir::OpGraph>& g);
void plan_cache_stats(uint64_t* hits, uint64_t* misses);

// GEMM problem of a Matmul-anchored helium-ir subgraph (MatmulGenerator::new,
// helium-kernel-generator/src/generators/matmul.rs:88-130). Throws HE_ERR_UNSUPPORTED for an UnsupportedFusion.
GemmProblem gemm_problem_from_ir(const ir::OpSubgraph& sg);
// For a subgraph that is one ConvBackwardData with a stride: one product per class of output pixels (row and column
// modulo the stride), each over the taps that reach the class; empty otherwise. `any_empty`: some class is reached by
// no tap, so its pixels have to be zeroed.
std::vector<GemmProblem> strided_data_gradient_classes(const ir::OpSubgraph& sg, bool* any_empty);
// The kernel of a Gemm instruction: one fused GEMM, or the classes of a strided data gradient one after the other.
std::unique_ptr<KernelBase> make_gemm_kernel(const ir::OpSubgraph& sg, const ir::OpSubgraph* carried = nullptr, bool beside_main_chain = false);

}  // namespace he::plan
