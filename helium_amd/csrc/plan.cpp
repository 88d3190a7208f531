#include "plan.h"

#include <limits>

#include <atomic>
#include <future>
#include <list>
#include <map>
#include <set>
#include <sstream>
#include <unordered_map>

namespace he::plan {

// ---------------------------------------------------------------------------------------------------------
// Instructions
// ---------------------------------------------------------------------------------------------------------
bool enumerate_swaps(const ir::OpSubgraph& sg, std::vector<std::pair<int, int>>* swaps) {
    swaps->clear();
    if (sg.inputs().size() != 1) return false;
    const ir::OpGraph& g = *sg.graph();
    // entry_node (permute_dims.rs:144-153): the member that consumes the single input
    NodeId current = ir::kNoNode;
    for (NodeId c : g.outbound(sg.inputs()[0]))
        if (sg.contains(c)) {
            current = c;
            break;
        }
    if (current == ir::kNoNode) return false;
    std::vector<NodeId> visited{current};
    for (;;) {
        const ir::Node& n = g.get(current);
        if (n.kind != ir::Node::Intermediate || n.op.kind != ir::OpKind::SwapDims) return false;
        swaps->emplace_back((int)n.op.axis_a, (int)n.op.axis_b);
        const auto& next = g.outbound(current);
        if (next.size() == 1 && sg.contains(next[0])) {
            current = next[0];
            visited.push_back(current);
        } else {
            break;
        }
    }
    for (NodeId n : sg.nodes())
        if (std::find(visited.begin(), visited.end(), n) == visited.end()) return false;
    return true;
}

std::unique_ptr<KernelBase> make_gemm_kernel(const ir::OpSubgraph& sg, const ir::OpSubgraph* carried, bool beside_main_chain);
bool gemm_can_carry(const ir::OpSubgraph& large, const ir::OpSubgraph& small);
namespace {
std::atomic<bool> g_fuse_matmul_epilogue{true};
std::atomic<bool> g_fold_swap_into_reduce{true};
std::atomic<bool> g_rematerialize{true};
std::atomic<bool> g_cancel_transposes{true};
std::atomic<bool> g_hoist_broadcasts{true};

}  // namespace
// True when every value computed from `node` inside the graph ends in a Reduce, through pointwise ops only: nothing
// then needs the transposed tensor in memory.
bool feeds_only_reductions(const ir::OpGraph& g, NodeId node, int budget) {
    const auto& users = g.outbound(node);
    if (users.empty() || budget <= 0) return false;
    for (NodeId u : users) {
        const ir::Node& n = g.get(u);
        if (n.kind != ir::Node::Intermediate) return false;
        switch (n.op.kind) {
            case ir::OpKind::Reduce: break;
            case ir::OpKind::UnaryPointwise:
            case ir::OpKind::BinaryPointwise:
            case ir::OpKind::ChangeDataType:
            case ir::OpKind::Compare:
            case ir::OpKind::Select:
                if (!feeds_only_reductions(g, u, budget - 1)) return false;
                break;
            default: return false;
        }
    }
    return true;
}
void set_fuse_matmul_epilogue(bool on) { g_fuse_matmul_epilogue.store(on); }
bool fuse_matmul_epilogue() { return g_fuse_matmul_epilogue.load(); }
uint64_t option_mask() {
    // the hash of the tuning overrides (0 unless tuning is on) rides along: plans keep their kernels
    return (fuse_matmul_epilogue() ? 1u : 0u) | (g_fold_swap_into_reduce.load() ? 2u : 0u) | (g_rematerialize.load() ? 4u : 0u) | (g_cancel_transposes.load() ? 8u : 0u) | (g_hoist_broadcasts.load() ? 16u : 0u) | ((uint64_t)tuning::hash() << 5);
}
void set_fold_swap_into_reduce(bool on) { g_fold_swap_into_reduce.store(on); }
void set_rematerialize(bool on) { g_rematerialize.store(on); }
bool rematerialize() { return g_rematerialize.load(); }
void set_cancel_transposes(bool on) { g_cancel_transposes.store(on); }
bool cancel_transposes() { return g_cancel_transposes.load(); }
void set_hoist_broadcasts(bool on) { g_hoist_broadcasts.store(on); }
bool hoist_broadcasts() { return g_hoist_broadcasts.load(); }
bool fold_swap_into_reduce() { return g_fold_swap_into_reduce.load(); }

bool Instr::can_fuse_with(const Instr& next) const {
    // (a large SwapDims is a Permute instruction: it joins a following Matmul as a transposed operand the same way)
    const bool gemm_and_pointwise = (kind_ == InstrKind::Gemm && next.kind_ == InstrKind::Pointwise) ||
                                    ((kind_ == InstrKind::Pointwise || kind_ == InstrKind::Permute) && next.kind_ == InstrKind::Gemm);
    if (gemm_and_pointwise && fuse_matmul_epilogue()) {
        // Beyond the reference, whose matmul instruction never fuses: pointwise and reduce ops that follow a Matmul
        // join it when they can run on the accumulators as the fused GEMM's epilogue; so do the ops that only prepare
        // epilogue operands (a bias broadcast), whichever of the two the greedy pass visits first.
        try {
            const ir::OpSubgraph merged = sg_.merge_with(next.sg_);
            // A value that was copied so that its consumer computes it is not to become an output of the product (the
            // greedy pass visits the copy next to its producer first): it waits for its consumer, and the product is
            // offered the finished group again.
            for (NodeId leaf : merged.leafs())
                if (merged.graph()->made_for_consumer(leaf)) return false;
            (void)gemm_problem_from_ir(merged);
            return true;
        } catch (const Error&) {
            return false;
        }
    }
    if (kind_ != next.kind_) return false;  // only instructions of one kind fuse (instr.rs:71-84)
    switch (kind_) {
        case InstrKind::Gemm: return false;  // the reference's matmul instruction never fuses (cudnn_graph.rs:319-321)
        case InstrKind::Pointwise: return tp::pointwise_supports(sg_.merge_with(next.sg_));
        case InstrKind::Permute: {
            std::vector<std::pair<int, int>> swaps;
            return enumerate_swaps(sg_.merge_with(next.sg_), &swaps);
        }
    }
    return false;
}

Instr Instr::fuse_with(const Instr& next) const {
    const InstrKind kind = (kind_ == InstrKind::Gemm || next.kind_ == InstrKind::Gemm) ? InstrKind::Gemm : kind_;
    return Instr(kind, sg_.merge_with(next.sg_));
}

Instr make_instr_for_op(const std::shared_ptr<const ir::OpGraph>& g, NodeId node) {
    const ir::Node& n = g->get(node);
    HE_REQUIRE(n.kind == ir::Node::Intermediate, HE_ERR_INVALID, "node %u is not an op", node);
    ir::OpSubgraph sg(g, {node});
    switch (n.op.kind) {
        case ir::OpKind::SwapDims:
            // Heuristic of the reference: the tiled permute kernel for large tensors, the pointwise kernel (which
            // can fuse) for small ones.
            // Beyond the reference: a transposition that only feeds reductions is never written to memory; the
            // pointwise kernel folds the leading dims of the untransposed tensor in one pass over it.
            if (ir::num_elements(n.desc.shape) > kPermuteThreshold && !(fold_swap_into_reduce() && feeds_only_reductions(*g, node)))
                return Instr(InstrKind::Permute, sg);
            return Instr(InstrKind::Pointwise, sg);
        case ir::OpKind::Constant:
        case ir::OpKind::UnaryPointwise:
        case ir::OpKind::BinaryPointwise:
        case ir::OpKind::ChangeDataType:
        case ir::OpKind::Reduce:
        case ir::OpKind::Broadcast:
        case ir::OpKind::Reshape:
        case ir::OpKind::Compare:
        case ir::OpKind::Select: return Instr(InstrKind::Pointwise, sg);
        case ir::OpKind::Matmul: return Instr(InstrKind::Gemm, sg);
        // The reference hands convolutions to cuDNN (cuda.rs:55-58, cudnn_graph.rs:193-204); here the forward
        // convolution is the fused GEMM with an implicit im2col gather as its A operand.
        case ir::OpKind::Conv:
        case ir::OpKind::ConvBackwardData:
        case ir::OpKind::ConvBackwardFilter: return Instr(InstrKind::Gemm, sg);
        default: fail(HE_ERR_INVALID, "unknown op kind");
    }
}

namespace {
template <class V>
class KernelCache {
public:
    explicit KernelCache(size_t cap) : cap_(cap) {}
    template <class F>
    std::shared_ptr<V> get_or_insert(const std::string& key, F&& make) {
        {
            std::lock_guard<std::mutex> lk(mu_);
            auto it = map_.find(key);
            if (it != map_.end()) return it->second;
        }
        // built outside the lock: a redundant build by a racing thread is an accepted cost (cache.rs:40-49)
        std::shared_ptr<V> v = make();
        std::lock_guard<std::mutex> lk(mu_);
        if (map_.size() >= cap_) map_.erase(map_.begin());
        return map_.emplace(key, v).first->second;
    }

private:
    size_t cap_;
    std::mutex mu_;
    std::unordered_map<std::string, std::shared_ptr<V>> map_;
};
KernelCache<KernelBase> g_tile_kernels(1024);  // pointwise.rs:45, permute_dims.rs:61 use 1024 entries
KernelCache<Permute> g_permutes(1024);
}  // namespace

std::vector<NodeId> Instr::all_inputs() const {
    std::vector<NodeId> in = sg_.inputs();
    if (carried_) {
        const std::vector<NodeId> own = sg_.leafs();
        for (NodeId n : carried_->sg_.inputs())
            if (std::find(own.begin(), own.end(), n) == own.end() && std::find(in.begin(), in.end(), n) == in.end()) in.push_back(n);
    }
    return in;
}

std::vector<NodeId> Instr::all_outputs() const {
    std::vector<NodeId> out = sg_.leafs();
    if (carried_)
        for (NodeId n : carried_->sg_.leafs()) out.push_back(n);
    return out;
}

void Instr::precompile() const {
    std::lock_guard<std::mutex> lk(mu_);
    if (kernel_ || permute_ || absorbed_) return;
    switch (kind_) {
        case InstrKind::Pointwise:
            kernel_ = g_tile_kernels.get_or_insert(
                tuning::key() + "pw:" + sg_.cache_key() + (carried_ ? "+carries:" + carried_->sg_.cache_key() : std::string()), [&] {
                    tp::Program prog = tp::lower_pointwise(sg_);
                    if (carried_)
                        HE_REQUIRE(tp::attach_post(&prog, tp::lower_pointwise(carried_->sg_)), HE_ERR_INTERNAL,
                                   "the carried instruction does not fit the fold launch any more");
                    return std::shared_ptr<KernelBase>(new TileKernel(std::move(prog), "pointwise_kernel"));
                });
            break;
        case InstrKind::Gemm:
            kernel_ = g_tile_kernels.get_or_insert(
                tuning::key() + (beside_main_chain() ? "mm-beside:" : "mm:") + sg_.cache_key() + (carried_ ? "+carries:" + carried_->sg_.cache_key() : std::string()),
                [&] { return std::shared_ptr<KernelBase>(make_gemm_kernel(sg_, carried_ ? &carried_->sg_ : nullptr, beside_main_chain())); });
            break;
        case InstrKind::Permute: {
            std::vector<std::pair<int, int>> swaps;
            HE_REQUIRE(enumerate_swaps(sg_, &swaps), HE_ERR_INTERNAL, "permute instruction is not a chain of swaps");
            const ir::Descriptor& d = sg_.graph()->get(sg_.inputs()[0]).desc;
            std::vector<int> perm = perm_from_swaps((int)d.shape.size(), swaps);
            std::ostringstream key;
            key << tuning::key() << d.dtype << ':';
            for (int64_t e : d.shape) key << e << ',';
            key << ':';
            for (int p : perm) key << p << ',';
            permute_ = g_permutes.get_or_insert(key.str(), [&] { return std::make_shared<Permute>(d.shape, perm, d.dtype); });
            break;
        }
    }
}

void Instr::execute(const std::function<void*(NodeId)>& storage, hipStream_t stream) const {
    if (absorbed_) return;  // the instruction that carries it has done the work
    precompile();
    if (kind_ == InstrKind::Permute) {
        permute_->execute(storage(sg_.inputs()[0]), storage(sg_.leafs()[0]), stream);
        return;
    }
    const auto& args = kernel_->args();
    std::vector<void*> ptrs(args.size());
    for (size_t i = 0; i < args.size(); i++) ptrs[i] = storage((NodeId)args[i].node);
    kernel_->execute(ptrs.data(), stream);
}

std::string Instr::describe(bool origins) const {
    std::ostringstream s;
    s << (kind_ == InstrKind::Gemm ? "gemm" : kind_ == InstrKind::Pointwise ? "pointwise" : "permute") << "{";
    // (a rematerialised graph's nodes are named by the nodes they stand for)
    bool first = true;
    for (NodeId node : sg_.nodes()) {
        const NodeId name = origins ? sg_.graph()->origin(node) : node;
        if (name == ir::kNoNode) continue;  // a node a rewrite added that stands for none of the planned graph's
        s << (first ? "" : ",") << name;
        first = false;
    }
    s << "}";
    return s.str();
}

// ---------------------------------------------------------------------------------------------------------
// Instruction graph (plan_generation.rs:87-236)
// ---------------------------------------------------------------------------------------------------------
namespace {
struct InstrGraph {
    std::map<uint64_t, std::shared_ptr<Instr>> instrs;
    uint64_t next_id = 0;
    std::map<NodeId, uint64_t> producers;
    std::map<NodeId, std::set<uint64_t>> consumers;
    std::map<uint64_t, std::set<uint64_t>> dependencies, dependents;

    // Ids order the greedy fusion and the steps. The reference keeps instructions in a slotmap (slotmap 1.0.7),
    // whose keys compare by slot index first and whose free list is last-in-first-out: the instruction made by
    // fusing a into b therefore takes b's slot, and `slot` lets fuse() say so.
    uint64_t insert(std::shared_ptr<Instr> instr, int64_t slot = -1) {
        const uint64_t id = slot >= 0 ? (uint64_t)slot : next_id++;
        const auto inputs = instr->inputs(), outputs = instr->outputs();
        instrs[id] = std::move(instr);
        for (NodeId in : inputs) {
            consumers[in].insert(id);
            auto p = producers.find(in);
            if (p != producers.end()) dependents[p->second].insert(id);
        }
        for (NodeId out : outputs) {
            HE_REQUIRE(!producers.count(out), HE_ERR_INTERNAL, "node %u has two producers", out);
            producers[out] = id;
            for (uint64_t c : consumers[out]) dependencies[c].insert(id);
        }
        std::set<uint64_t>& dts = dependents[id];
        for (NodeId out : outputs)
            for (uint64_t c : consumers[out]) dts.insert(c);
        std::set<uint64_t>& dps = dependencies[id];
        for (NodeId in : inputs) {
            auto p = producers.find(in);
            if (p != producers.end()) dps.insert(p->second);
        }
        return id;
    }

    std::shared_ptr<Instr> remove(uint64_t id) {
        std::shared_ptr<Instr> instr = instrs.at(id);
        instrs.erase(id);
        for (NodeId in : instr->inputs()) {
            consumers[in].erase(id);
            auto p = producers.find(in);
            if (p != producers.end()) dependents[p->second].erase(id);
        }
        for (NodeId out : instr->outputs()) {
            producers.erase(out);
            for (uint64_t c : consumers[out]) dependencies[c].erase(id);
        }
        dependencies.erase(id);
        dependents.erase(id);
        return instr;
    }

    // Is there a path a -> ... -> b besides the direct edge? Fusing across one would create a cycle.
    bool exist_multiple_paths(uint64_t a, uint64_t b) const {
        std::vector<uint64_t> stack;
        std::set<uint64_t> visited;
        for (uint64_t d : dependents.at(a))
            if (d != b) {
                stack.push_back(d);
                visited.insert(d);
            }
        while (!stack.empty()) {
            uint64_t cur = stack.back();
            stack.pop_back();
            if (cur == b) return true;
            for (uint64_t n : dependents.at(cur))
                if (visited.insert(n).second) stack.push_back(n);
        }
        return false;
    }

    bool can_fuse(uint64_t a, uint64_t b) const {
        return instrs.at(a)->can_fuse_with(*instrs.at(b)) && !exist_multiple_paths(a, b);
    }

    uint64_t fuse(uint64_t a, uint64_t b) {
        std::shared_ptr<Instr> ia = remove(a), ib = remove(b);
        return insert(std::make_shared<Instr>(ia->fuse_with(*ib)), (int64_t)b);
    }
};

bool intersects(const std::vector<NodeId>& a, const std::vector<NodeId>& b) {
    for (NodeId x : a)
        for (NodeId y : b)
            if (x == y) return true;
    return false;
}
}  // namespace

std::shared_ptr<const Plan> generate_plan(const std::shared_ptr<const ir::OpGraph>& g) {
    // make_instr_graph (:259-270): one instruction per intermediate node, in node order
    InstrGraph ig;
    for (NodeId n : g->nodes())
        if (g->get(n).kind == ir::Node::Intermediate) ig.insert(std::make_shared<Instr>(make_instr_for_op(g, n)));

    // A value that was copied so that its consumer computes it joins that consumer before anything else: the greedy
    // pass below walks from producers to consumers and would put the copy into its producer's kernel, to be written
    // out from there. Last copies first, so that a chain of copies ends up in the kernel at its end.
    if (g->has_origins()) {
        std::vector<uint64_t> ids;
        for (auto& kv : ig.instrs) ids.push_back(kv.first);
        for (auto it = ids.rbegin(); it != ids.rend(); ++it) {
            auto found = ig.instrs.find(*it);
            if (found == ig.instrs.end()) continue;
            const auto& nodes = found->second->subgraph().nodes();
            if (nodes.size() != 1 || !g->made_for_consumer(nodes[0])) continue;
            const auto& next = ig.dependents.at(*it);
            if (next.size() == 1 && ig.can_fuse(*it, *next.begin())) ig.fuse(*it, *next.begin());
        }
    }

    // do_fusions (:243-256)
    auto do_fusions = [&] {
        bool fused = false;
        std::set<uint64_t> work;
        for (auto& kv : ig.instrs) work.insert(kv.first);
        while (!work.empty()) {
            const uint64_t cur = *work.begin();
            work.erase(work.begin());
            std::vector<uint64_t> nexts(ig.dependents.at(cur).begin(), ig.dependents.at(cur).end());
            for (uint64_t nxt : nexts)
                if (ig.can_fuse(cur, nxt)) {
                    uint64_t merged = ig.fuse(cur, nxt);
                    work.erase(nxt);
                    work.insert(merged);
                    fused = true;
                    break;
                }
        }
        return fused;
    };
    // The reference makes one pass: an instruction whose dependents all refuse it is not looked at again. Here a
    // dependent may become acceptable later (a transposition joins its reduction, and only then the ops before it
    // can follow), so when the graph is not planned as recorded the pass is repeated until nothing fuses.
    while (do_fusions() && rematerialize()) {
    }

    // Beyond the reference: kernels that reduce over the same index space and read a tensor in common share one pass
    // over it. The greedy pass merges along producer -> consumer edges only, and the sums of one backward pass (a
    // batch norm's sum of dy and sum of dy * xhat) are siblings: each would read both tensors again. Two such kernels
    // merge when neither depends on the other; four reductions per kernel at most (each keeps its own accumulators;
    // six or eight measured the same). A full-size output next to the reductions, written through their walk, does
    // not stand in the way: merging those too took the training step at batch 128 from 5.14 to 4.95 ms, monotonically
    // in the size admitted (HELIUM_HIP_SIBLING_MAX: the largest such output in elements, 0 = kernels of reductions
    // only).
    if (rematerialize()) {
        int64_t sibling_max = std::numeric_limits<int64_t>::max();
        if (const char* env = tuning::get("HELIUM_HIP_SIBLING_MAX")) sibling_max = atoll(env);
        auto reduces_columns = [&](const Instr& instr, ir::Shape* shape, uint32_t* depth, size_t* count) {
            if (instr.kind() != InstrKind::Pointwise) return false;
            *count = 0;
            for (NodeId leaf : instr.subgraph().leafs()) {
                const ir::Node& n = g->get(leaf);
                if (n.op.kind != ir::OpKind::Reduce) {
                    if (ir::num_elements(n.desc.shape) > sibling_max) return false;
                    continue;
                }
                *shape = g->get(n.op.inputs[0]).desc.shape;
                *depth = n.op.depth;
                ++*count;
            }
            return *count > 0;
        };
        auto reaches = [&](uint64_t from, uint64_t to) {
            std::vector<uint64_t> stack{from};
            std::set<uint64_t> visited{from};
            while (!stack.empty()) {
                const uint64_t cur = stack.back();
                stack.pop_back();
                if (cur == to) return true;
                for (uint64_t n : ig.dependents.at(cur))
                    if (visited.insert(n).second) stack.push_back(n);
            }
            return false;
        };
        for (bool changed = true; changed;) {
            changed = false;
            for (auto& [tensor, readers] : ig.consumers) {
                if (readers.size() < 2 || ir::num_elements(g->get(tensor).desc.shape) < (1 << 16)) continue;
                const std::vector<uint64_t> ids(readers.begin(), readers.end());
                for (size_t i = 0; i < ids.size() && !changed; i++)
                    for (size_t j = i + 1; j < ids.size() && !changed; j++) {
                        ir::Shape sa, sb;
                        uint32_t da = 0, db = 0;
                        size_t na = 0, nb = 0;
                        if (!reduces_columns(*ig.instrs.at(ids[i]), &sa, &da, &na) || !reduces_columns(*ig.instrs.at(ids[j]), &sb, &db, &nb)) continue;
                        if (sa != sb || da != db || na + nb > 4) continue;
                        if (reaches(ids[i], ids[j]) || reaches(ids[j], ids[i])) continue;
                        if (!ig.instrs.at(ids[i])->can_fuse_with(*ig.instrs.at(ids[j]))) continue;
                        ig.fuse(ids[i], ids[j]);
                        changed = true;
                    }
                if (changed) break;  // the maps changed under the loops
            }
        }
    }

    // Beyond the reference, with the epilogue option on: the greedy pass visits a product before the pointwise group
    // that reduces it has formed (a SwapDims alone is no epilogue; SwapDims + Reduce is a column reduction), so
    // products are offered their finished pointwise dependents once more.
    if (fuse_matmul_epilogue()) {
        for (bool changed = true; changed;) {
            changed = false;
            for (auto& kv : ig.instrs) {
                if (kv.second->kind() != InstrKind::Gemm) continue;
                const uint64_t cur = kv.first;
                std::vector<uint64_t> nexts(ig.dependents.at(cur).begin(), ig.dependents.at(cur).end());
                for (uint64_t nxt : nexts)
                    if (ig.instrs.at(nxt)->kind() == InstrKind::Pointwise && ig.can_fuse(cur, nxt)) {
                        ig.fuse(cur, nxt);
                        changed = true;
                        break;
                    }
                if (changed) break;  // the map changed under the loop
            }
        }
    }

    // generate_plan_from_graph (:275-321): Kahn levels
    auto plan = std::make_shared<Plan>();
    {
        const size_t total = ig.instrs.size();
        std::map<uint64_t, size_t> indeg;
        std::vector<uint64_t> stack;
        for (auto& kv : ig.instrs) {
            indeg[kv.first] = ig.dependencies.at(kv.first).size();
            if (indeg[kv.first] == 0) stack.push_back(kv.first);
        }
        size_t placed = 0;
        while (!stack.empty()) {
            std::vector<uint64_t> step;
            step.swap(stack);
            for (uint64_t id : step)
                for (uint64_t nxt : ig.dependents.at(id)) {
                    HE_REQUIRE(indeg[nxt] > 0, HE_ERR_INTERNAL, "indegree underflow");
                    if (--indeg[nxt] == 0) stack.push_back(nxt);
                }
            Step s;
            for (uint64_t id : step) s.instrs.push_back(ig.instrs.at(id));
            placed += s.instrs.size();
            plan->steps.push_back(std::move(s));
        }
        HE_REQUIRE(placed == total, HE_ERR_INTERNAL, "cycle detected in instruction graph?");
    }

    // delay_computations (:325-353): push every instruction to the step before its first reader
    for (int i = (int)plan->steps.size() - 1; i >= 0; i--) {
        std::vector<std::shared_ptr<Instr>> kept;
        std::vector<std::shared_ptr<Instr>> here;
        here.swap(plan->steps[i].instrs);
        for (auto& instr : here) {
            const auto outs = instr->outputs();
            int target = -1;
            for (size_t j = i + 1; j < plan->steps.size(); j++) {
                bool reads = false;
                for (auto& other : plan->steps[j].instrs) reads = reads || intersects(other->inputs(), outs);
                if (reads) {
                    target = (int)j - 1;
                    break;
                }
            }
            if (target >= 0 && target != i) plan->steps[target].instrs.push_back(instr);
            else kept.push_back(instr);
        }
        plan->steps[i].instrs = kept;
    }

    // Beyond the reference: small pointwise kernels of one step that walk the same index space run as one kernel. They
    // are independent by construction (one step), each costs a launch of several microseconds for a few hundred
    // elements (per-channel arithmetic of a batch norm's backward pass next to the optimizer's update of its scale and
    // shift), and one launch computes all of them in the same time.
    if (rematerialize()) {
        auto small_space = [&](const Instr& instr, int64_t* numel) {
            if (instr.kind() != InstrKind::Pointwise) return false;
            *numel = -1;
            for (NodeId leaf : instr.subgraph().leafs()) {
                const ir::Node& n = g->get(leaf);
                if (n.op.kind == ir::OpKind::Reduce) return false;
                const int64_t e = ir::num_elements(n.desc.shape);
                if (*numel >= 0 && e != *numel) return false;
                *numel = e;
            }
            return *numel >= 0 && *numel <= (1 << 16);
        };
        for (Step& step : plan->steps) {
            for (size_t i = 0; i < step.instrs.size(); i++) {
                int64_t ni = 0;
                if (!small_space(*step.instrs[i], &ni)) continue;
                for (size_t j = i + 1; j < step.instrs.size();) {
                    int64_t nj = 0;
                    const Instr &a = *step.instrs[i], &b = *step.instrs[j];
                    if (small_space(b, &nj) && nj == ni && a.outputs().size() + b.outputs().size() <= 24 &&
                        a.subgraph().nodes().size() + b.subgraph().nodes().size() <= 160 && a.can_fuse_with(b)) {
                        step.instrs[i] = std::make_shared<Instr>(a.fuse_with(b));
                        step.instrs.erase(step.instrs.begin() + j);
                    } else {
                        j++;
                    }
                }
            }
        }
    }

    // Beyond the reference: a small pointwise instruction that reads column reductions of a large pointwise instruction
    // (a batch norm's per-channel arithmetic behind its sums) rides on the launch that folds those reductions instead of
    // being a launch of its own, when everything else it reads exists by then. The plan keeps both instructions where
    // they are; the large one carries the small one (Instr::carry).
    if (rematerialize() && !tuning::get("HELIUM_HIP_NO_CARRY")) {
        std::map<NodeId, std::pair<size_t, size_t>> made_at;  // leaf -> (step, position in the step)
        size_t carried_count = 0;
        std::map<std::string, int> why;
        for (size_t i = 0; i < plan->steps.size(); i++)
            for (size_t j = 0; j < plan->steps[i].instrs.size(); j++)
                for (NodeId leaf : plan->steps[i].instrs[j]->outputs()) made_at[leaf] = {i, j};
        for (size_t i2 = 0; i2 < plan->steps.size(); i2++) {
            for (auto& small : plan->steps[i2].instrs) {
                if (small->kind() != InstrKind::Pointwise || small->carried() || small->absorbed()) continue;
                bool is_small = true;
                for (NodeId n : small->subgraph().nodes()) is_small = is_small && ir::num_elements(g->get(n).desc.shape) <= (1 << 16);
                if (!is_small) continue;
                // the producer that runs last must be the one whose reductions are read (the others are done before it: earlier
                // steps, or earlier in a step that then runs in order)
                bool have = false, reads_reduction = false;
                std::pair<size_t, size_t> last{0, 0};
                for (NodeId in : small->inputs()) {
                    auto it = made_at.find(in);
                    if (it == made_at.end()) continue;  // an input of the graph
                    if (!have || it->second > last) last = it->second;
                    have = true;
                }
                if (!have || last.first >= i2) { why["no producer before"]++; continue; }
                Instr& large = *plan->steps[last.first].instrs[last.second];
                if (large.kind() == InstrKind::Permute || large.carried() || large.absorbed()) { why["last producer taken"]++; continue; }
                bool same_step = false;  // another producer in the large one's step (ahead of it, `last` being the last)
                for (NodeId in : small->inputs()) {
                    auto it = made_at.find(in);
                    if (it == made_at.end()) continue;
                    if (it->second == last) reads_reduction = reads_reduction || g->get(in).op.kind == ir::OpKind::Reduce;
                    else same_step = same_step || it->second.first == last.first;
                }
                if (!reads_reduction) { why["reads no reduction of it"]++; continue; }
                try {
                    if (large.kind() == InstrKind::Gemm) {
                        if (!gemm_can_carry(large.subgraph(), small->subgraph())) { why["does not attach to the product"]++; continue; }
                        large.carry(small);
                        if (same_step) plan->steps[last.first].in_order = true;
                        carried_count++;
                        continue;
                    }
                    tp::Program prog = tp::lower_pointwise(large.subgraph());
                    if (!tp::attach_post(&prog, tp::lower_pointwise(small->subgraph()))) { why["does not attach"]++; continue; }
                    if (!tp::emit_pointwise(prog, "pointwise_kernel").post_carried) { why["no fold launch"]++; continue; }
                } catch (const Error&) {
                    continue;
                }
                large.carry(small);
                if (same_step) plan->steps[last.first].in_order = true;
                carried_count++;
            }
        }
        if (getenv("HELIUM_HIP_PLAN_DEBUG") && carried_count) {
            fprintf(stderr, "[plan] %zu small instructions ride on fold launches", carried_count);
            for (auto& kv : why) fprintf(stderr, "; %s: %d", kv.first.c_str(), kv.second);
            fprintf(stderr, "\n");
        }
    }

    // analyze_tensor_lifetimes (:360-416)
    {
        std::vector<std::vector<NodeId>> releases;
        releases.emplace_back();  // nothing is freed at the first step
        for (size_t i = 0; i < plan->steps.size(); i++) {
            std::vector<NodeId> used;
            for (auto& instr : plan->steps[i].instrs)
                for (NodeId in : instr->inputs()) used.push_back(in);
            std::sort(used.begin(), used.end());
            used.erase(std::unique(used.begin(), used.end()), used.end());
            std::vector<NodeId> rel;
            for (NodeId t : used) {
                if (g->feeds_output(t)) continue;
                bool later = false;
                for (size_t j = i + 1; j < plan->steps.size() && !later; j++)
                    for (auto& instr : plan->steps[j].instrs) {
                        const auto ins = instr->inputs();
                        if (std::find(ins.begin(), ins.end(), t) != ins.end()) {
                            later = true;
                            break;
                        }
                    }
                if (!later) rel.push_back(t);
            }
            releases.push_back(std::move(rel));
        }
        plan->steps.emplace_back();  // a last, empty step that frees the final temporaries
        for (size_t i = 0; i < plan->steps.size(); i++) plan->steps[i].tensors_to_release = releases[i];
    }
    return plan;
}

std::string Plan::describe(bool origins) const {
    std::ostringstream s;
    const ir::OpGraph* g = nullptr;
    for (auto& st : steps)
        for (auto& instr : st.instrs) g = instr->subgraph().graph().get();
    for (size_t i = 0; i < steps.size(); i++) {
        s << "step " << i << ":";
        for (auto& instr : steps[i].instrs) s << " " << instr->describe(origins);
        s << " | release";
        for (NodeId t : steps[i].tensors_to_release)
            if (!(g && origins) || g->origin(t) != ir::kNoNode) s << " " << (g && origins ? g->origin(t) : t);
        s << "\n";
    }
    return s.str();
}

int64_t plan_traffic_bytes(const Plan& plan) {
    int64_t bytes = 0;
    for (auto& st : plan.steps)
        for (auto& instr : st.instrs) {
            const ir::OpGraph& g = *instr->subgraph().graph();
            for (NodeId n : instr->inputs()) bytes += (int64_t)storage_bytes(g.get(n).desc.dtype, (size_t)ir::num_elements(g.get(n).desc.shape));
            for (NodeId n : instr->outputs()) bytes += (int64_t)storage_bytes(g.get(n).desc.dtype, (size_t)ir::num_elements(g.get(n).desc.shape));
        }
    return bytes;
}

std::shared_ptr<const ir::OpGraph> graph_for_execution(const std::shared_ptr<const ir::OpGraph>& g) {
    const bool debug = getenv("HELIUM_HIP_PLAN_DEBUG") != nullptr;
    // 1. transpositions that undo each other go - when the plan then moves no more bytes (the kernels walk their tensors
    //    in memory order instead)
    std::shared_ptr<const ir::OpGraph> base = g;
    const int64_t recorded = plan_traffic_bytes(*generate_cached_plan(g));
    int64_t base_bytes = recorded;
    if (cancel_transposes())
        if (auto untransposed = ir::transposes_cancelled(*g)) {
            const int64_t bytes = plan_traffic_bytes(*generate_cached_plan(untransposed));
            if (debug) fprintf(stderr, "[plan] transpositions cancelled: %zu -> %zu nodes, %lld -> %lld bytes\n", g->num_nodes(), untransposed->num_nodes(), (long long)recorded, (long long)bytes);
            if (bytes <= base_bytes) {
                base = untransposed;
                base_bytes = bytes;
            }
        }
    // ... and pointwise ops on broadcasts alone are applied before the broadcast: less arithmetic for about the same
    // bytes (the small results are tensors of their own)
    if (hoist_broadcasts())
        if (auto hoisted = ir::broadcasts_hoisted(*base)) {
            if (base != g) hoisted->rebase_origins(*base);
            const int64_t bytes = plan_traffic_bytes(*generate_cached_plan(hoisted));
            if (debug) fprintf(stderr, "[plan] broadcasts hoisted: %zu -> %zu nodes, %lld -> %lld bytes\n", base->num_nodes(), hoisted->num_nodes(), (long long)base_bytes, (long long)bytes);
            if (bytes <= base_bytes + base_bytes / 20 + (64 << 10)) {
                base = hoisted;
                base_bytes = bytes;
            }
        }
    // 2. cheap values are computed where they are used
    std::shared_ptr<ir::OpGraph> other = rematerialize() ? ir::rematerialized(*base) : nullptr;
    if (other) {
        // Copies that the fusion rules keep out of their consumers' kernels are written out, each on its own: where one
        // kernel ends up with several copies of a value among its outputs, that value goes back to being computed once,
        // and the graph is planned again.
        std::set<ir::NodeId> keep_single;
        std::shared_ptr<ir::OpGraph> best;
        int64_t best_bytes = 0;
        for (int round = 0; round < 3 && other; round++) {
            const size_t known = keep_single.size();
            const auto plan = generate_plan(other);
            const int64_t bytes = plan_traffic_bytes(*plan);
            if (debug) fprintf(stderr, "[plan] round %d: %zu -> %zu nodes, %zu kept single, %lld bytes\n", round, base->num_nodes(), other->num_nodes(), known, (long long)bytes);
            if (!best || bytes < best_bytes) {
                best = other;
                best_bytes = bytes;
            }
            for (auto& st : plan->steps)
                for (auto& instr : st.instrs) {
                    std::set<ir::NodeId> origins;
                    for (ir::NodeId leaf : instr->outputs())
                        if (!origins.insert(other->origin(leaf)).second) keep_single.insert(other->origin(leaf));
                }
            if (keep_single.size() == known) break;
            other = ir::rematerialized(*base, keep_single);
        }
        other = best;  // (a round that takes copies back usually moves fewer bytes, not always)
        // A value that depends on two tensors of its size is written once and read back - unless the kernel that reads
        // it reads those two tensors anyway, or all but one of them: then it computes the value itself, the kernel that
        // made it (a batch norm's backward sums, which need it too) no longer writes it, and a pass or two over a
        // full-size tensor goes. The plan tells which values those are; the graph is rewritten with their source
        // pairs admitted, planned again, and kept when it moves fewer bytes.
        if (other && !tuning::get("HELIUM_HIP_NO_TWO_SOURCE_REMAT")) {
            std::set<std::vector<ir::NodeId>> two_sources;
            for (int round = 0; round < 3; round++) {
                const auto plan = generate_plan(other);
                const size_t known = two_sources.size();
                auto large_inputs = [&](const Instr& instr, int64_t numel) {
                    std::vector<ir::NodeId> v;
                    for (ir::NodeId in : instr.inputs())
                        if (ir::num_elements(other->get(in).desc.shape) * 8 >= numel) v.push_back(in);
                    return v;
                };
                std::map<ir::NodeId, std::vector<const Instr*>> readers;
                for (auto& st : plan->steps)
                    for (auto& instr : st.instrs)
                        for (ir::NodeId in : instr->inputs()) readers[in].push_back(instr.get());
                for (auto& st : plan->steps)
                    for (auto& maker : st.instrs) {
                        if (maker->kind() != InstrKind::Pointwise) continue;
                        for (ir::NodeId x : maker->outputs()) {
                            const ir::Node& xn = other->get(x);
                            const int64_t numel = ir::num_elements(xn.desc.shape);
                            if (numel < (1 << 16) || xn.op.kind == ir::OpKind::Reduce || other->feeds_output(x)) continue;
                            auto rd = readers.find(x);
                            if (rd == readers.end() || rd->second.size() != 1 || rd->second[0]->kind() != InstrKind::Pointwise) continue;
                            std::vector<ir::NodeId> sources = large_inputs(*maker, numel);
                            if (sources.size() != 2) continue;
                            const std::vector<ir::NodeId> theirs = large_inputs(*rd->second[0], numel);
                            int fresh = 0;
                            for (ir::NodeId s : sources) fresh += std::find(theirs.begin(), theirs.end(), s) == theirs.end();
                            if (fresh > 1) continue;
                            std::vector<ir::NodeId> pair{other->origin(sources[0]), other->origin(sources[1])};
                            std::sort(pair.begin(), pair.end());
                            two_sources.insert(pair);
                        }
                    }
                if (two_sources.size() == known) break;
                auto again = ir::rematerialized(*base, keep_single, two_sources);
                if (!again) break;
                const int64_t bytes = plan_traffic_bytes(*generate_plan(again));
                if (debug) fprintf(stderr, "[plan] two-source round %d: %zu pairs, %lld -> %lld bytes\n", round, two_sources.size(), (long long)best_bytes, (long long)bytes);
                if (bytes >= best_bytes) break;
                other = again;
                best_bytes = bytes;
            }
        }
    }
    if (!other) return base;
    if (base != g) other->rebase_origins(*base);
    const int64_t after = plan_traffic_bytes(*generate_cached_plan(other));
    if (debug) fprintf(stderr, "[plan] ... %lld bytes with cheap values computed where they are used\n", (long long)after);
    return after < base_bytes ? std::shared_ptr<const ir::OpGraph>(other) : base;
}

// ---------------------------------------------------------------------------------------------------------
// Plan cache (plan_generation.rs:29-50)
// ---------------------------------------------------------------------------------------------------------
namespace {
struct CacheEntry {
    uint64_t options;
    uint64_t hash;
    std::shared_ptr<const ir::OpGraph> graph;
    std::shared_ptr<const Plan> plan;
};
std::mutex g_plan_mu;
std::list<CacheEntry> g_plans;  // most recently used first
uint64_t g_plan_hits = 0, g_plan_misses = 0;
constexpr size_t kPlanCacheCapacity = 256;
}  // namespace

std::shared_ptr<const Plan> generate_cached_plan(const std::shared_ptr<const ir::OpGraph>& g) {
    const uint64_t h = g->structural_hash();
    {
        std::lock_guard<std::mutex> lk(g_plan_mu);
        for (auto it = g_plans.begin(); it != g_plans.end(); ++it)
            if (it->hash == h && it->options == option_mask() && it->graph->structurally_equal(*g)) {
                g_plans.splice(g_plans.begin(), g_plans, it);
                g_plan_hits++;
                return g_plans.front().plan;
            }
        g_plan_misses++;
    }
    // The cached plan refers to the graph object it was generated from; node ids are equal by construction.
    std::shared_ptr<const Plan> plan = generate_plan(g);
    std::lock_guard<std::mutex> lk(g_plan_mu);
    g_plans.push_front({option_mask(), h, g, plan});
    if (g_plans.size() > kPlanCacheCapacity) g_plans.pop_back();
    return plan;
}

void plan_cache_stats(uint64_t* hits, uint64_t* misses) {
    std::lock_guard<std::mutex> lk(g_plan_mu);
    *hits = g_plan_hits;
    *misses = g_plan_misses;
}

// ---------------------------------------------------------------------------------------------------------
// helium-ir Matmul -> GEMM problem
// ---------------------------------------------------------------------------------------------------------
namespace {
// Op::Conv as a GEMM: rows = output pixels (n, p, q), columns = output channels, k = filter taps (r, s, c). The
// filter [out_channels, kh, kw, in_channels] is B with k contiguous; A is gathered from the NHWC image on the fly.
GemmProblem conv_problem(const ir::OpSubgraph& sg, NodeId conv) {
    const ir::OpGraph& g = *sg.graph();
    const ir::Op& op = g.get(conv).op;
    HE_REQUIRE(sg.is_input(op.inputs[0]) && sg.is_input(op.inputs[1]), HE_ERR_UNSUPPORTED, "a convolution reads materialised operands");
    const ir::Descriptor &image = g.get(op.inputs[0]).desc, &filter = g.get(op.inputs[1]).desc, &out = g.get(conv).desc;
    HE_REQUIRE(dtype_class(image.dtype) == DataClass::Float && filter.dtype == image.dtype, HE_ERR_UNSUPPORTED,
               "conv takes a float image and a filter of the same type");
    HE_REQUIRE(filter.shape[0] == op.conv.out_channels && filter.shape[3] == op.conv.in_channels && image.shape[3] == op.conv.in_channels &&
                   filter.shape[1] == op.conv.kernel[0] && filter.shape[2] == op.conv.kernel[1],
               HE_ERR_INVALID, "conv filter / image shapes do not match the parameters");
    GemmProblem pr;
    auto& cv = pr.conv_a;
    cv.on = true;
    cv.N = image.shape[0]; cv.H = image.shape[1]; cv.W = image.shape[2]; cv.C = image.shape[3];
    cv.R = filter.shape[1]; cv.S = filter.shape[2];
    cv.P = out.shape[1]; cv.Q = out.shape[2];
    cv.sh = op.conv.stride[0]; cv.sw = op.conv.stride[1];
    cv.dh = op.conv.dilation[0]; cv.dw = op.conv.dilation[1];
    int64_t pad[2];
    op.conv.padding(pad);
    cv.ph = pad[0]; cv.pw = pad[1];
    pr.batch = 1;
    pr.M = cv.N * cv.P * cv.Q;
    pr.N = op.conv.out_channels;
    pr.K = cv.R * cv.S * cv.C;
    pr.split_k = choose_split_k(pr.M, pr.N, pr.K, 1);
    HE_REQUIRE(pr.M > 0 && pr.M < (1ll << 31) && ir::num_elements(image.shape) < (1ll << 32), HE_ERR_UNSUPPORTED, "conv too large for 32-bit tile indices");
    pr.mma_dtype = image.dtype == HE_F32 ? HE_F32 : image.dtype == HE_F16 ? HE_F16 : HE_BF16;
    auto operand = [&](tp::Program& p, const ir::Descriptor& d, NodeId node, int64_t rows, int64_t cols) {
        p.dims = {1, rows, cols};
        p.args.push_back({d.dtype, ir::num_elements(d.shape), false, node});
        tp::Expr e;
        e.kind = tp::Expr::Load;
        e.cls = tp::Cls::F;
        e.access.arg = 0;
        e.access.dtype = d.dtype;
        e.access.stride = ir::packed_strides(p.dims);
        p.exprs.push_back(e);
    };
    operand(pr.op_a, image, op.inputs[0], pr.M, pr.K);   // stands for the gathered matrix; only its argument is used
    operand(pr.op_b, filter, op.inputs[1], pr.N, pr.K);  // [n][k]: k contiguous
    pr.b_nk = true;
    pr.root_a = pr.root_b = 0;
    if (sg.nodes().size() > 1) {
        // Conv + the pointwise / reduce ops after it (beyond the reference, whose convolution instruction never
        // fuses): the epilogue runs on the accumulators, over [n, p, q, channels] with (n, p, q) as the rows. The
        // partial tiles of a split k range could not run it, so the k range stays whole.
        pr.split_k = 1;
        pr.epi = tp::lower_ir_epilogue(sg, conv, 3);
        validate_gemm_epilogue(pr.epi);
        assemble_gemm_args(pr);
        return pr;
    }
    pr.epi.dims = {1, pr.M, pr.N};
    pr.epi.fast_math = true;
    tp::Expr acc;
    acc.kind = tp::Expr::Acc;
    acc.cls = tp::Cls::F;
    pr.epi.exprs.push_back(acc);
    pr.epi.acc_expr = 0;
    tp::Out o;
    o.expr = 0;
    o.arg = 0;
    o.dtype = out.dtype;
    pr.epi.outs.push_back(o);
    pr.epi.args.push_back({out.dtype, ir::num_elements(out.shape), true, conv});
    validate_gemm_epilogue(pr.epi);
    assemble_gemm_args(pr);
    return pr;
}
}  // namespace

namespace {
// Op::ConvBackwardData as a GEMM: rows = pixels (n, h, w) of the image gradient, columns = input channels,
// k = (r, s, o). A is gathered from the flow (the gradient of the forward output): tap (r, s) of pixel (h, w) reads
// flow[n][(h + ph - r*dh) / sh][(w + pw - s*dw) / sw][o] where that pixel exists; B's row (r, s, o) is the filter's
// [o][r][s][:] row of input channels, picked out of the [out, kh, kw, in] tensor where it lies.
// `cls` < 0: the whole gradient as one product, every row testing every tap for divisibility by the stride. Otherwise
// class cls = a * stride_w + b: the pixels (h, w) with h % stride_h == a and w % stride_w == b. Of the taps only
// r = r0 + stride_h * r' (r0 = (a + pad) % stride_h) reach such a row, and with h = stride_h * i + a the flow row is
// i + (a + pad - r0) / stride_h - r': a stride-1 data gradient over the class's own grid of pixels with every
// stride-th tap of the filter, whose rows land on every stride-th pixel of the output. `empty` (if given) tells that
// no tap reaches the class: those pixels of the gradient are zero.
GemmProblem conv_backward_data_problem(const ir::OpSubgraph& sg, NodeId node, int cls = -1, bool* empty = nullptr) {
    const ir::OpGraph& g = *sg.graph();
    HE_REQUIRE(sg.nodes().size() == 1, HE_ERR_UNSUPPORTED, "a convolution instruction holds the op alone");
    const ir::Op& op = g.get(node).op;
    const ir::Descriptor &flow = g.get(op.inputs[0]).desc, &filter = g.get(op.inputs[1]).desc, &out = g.get(node).desc;
    HE_REQUIRE(flow.shape.size() == 4 && filter.shape.size() == 4, HE_ERR_INVALID, "conv backward takes rank-4 tensors");
    HE_REQUIRE(dtype_class(flow.dtype) == DataClass::Float && filter.dtype == flow.dtype, HE_ERR_UNSUPPORTED,
               "conv backward takes a float flow and a filter of the same type");
    HE_REQUIRE(filter.shape[0] == op.conv.out_channels && filter.shape[3] == op.conv.in_channels && flow.shape[3] == op.conv.out_channels &&
                   filter.shape[1] == op.conv.kernel[0] && filter.shape[2] == op.conv.kernel[1],
               HE_ERR_INVALID, "conv backward filter / flow shapes do not match the parameters");
    GemmProblem pr;
    auto& cv = pr.conv_a;
    cv.on = cv.bwd = true;
    cv.N = flow.shape[0]; cv.H = flow.shape[1]; cv.W = flow.shape[2]; cv.C = flow.shape[3];
    cv.R = filter.shape[1]; cv.S = filter.shape[2];
    cv.P = out.shape[1]; cv.Q = out.shape[2];
    cv.sh = op.conv.stride[0]; cv.sw = op.conv.stride[1];
    cv.dh = op.conv.dilation[0]; cv.dw = op.conv.dilation[1];
    int64_t pad[2];
    op.conv.padding(pad);
    cv.ph = pad[0]; cv.pw = pad[1];
    const int64_t in_channels = op.conv.in_channels;
    pr.batch = 1;
    int64_t r0 = 0, s0 = 0;
    const int64_t full_r = cv.R, full_s = cv.S, image_h = cv.P, image_w = cv.Q, stride_h = cv.sh, stride_w = cv.sw;
    if (cls >= 0) {
        const int64_t a = cls / stride_w, b = cls % stride_w;
        r0 = (a + cv.ph) % stride_h;
        s0 = (b + cv.pw) % stride_w;
        cv.R = r0 < full_r ? (full_r - r0 + stride_h - 1) / stride_h : 0;
        cv.S = s0 < full_s ? (full_s - s0 + stride_w - 1) / stride_w : 0;
        cv.P = a < image_h ? (image_h - a + stride_h - 1) / stride_h : 0;
        cv.Q = b < image_w ? (image_w - b + stride_w - 1) / stride_w : 0;
        cv.ph = (a + cv.ph - r0) / stride_h;
        cv.pw = (b + cv.pw - s0) / stride_w;
        cv.sh = cv.sw = 1;
        pr.out_rows.on = true;
        pr.out_rows.P = cv.P; pr.out_rows.Q = cv.Q;
        pr.out_rows.H = image_h; pr.out_rows.W = image_w;
        pr.out_rows.sh = stride_h; pr.out_rows.sw = stride_w;
        pr.out_rows.a = a; pr.out_rows.b = b;
        if (empty) *empty = cv.R == 0 || cv.S == 0 || cv.P == 0 || cv.Q == 0;
        if (cv.R == 0 || cv.S == 0 || cv.P == 0 || cv.Q == 0) return pr;
    }
    pr.M = cv.N * cv.P * cv.Q;
    pr.N = in_channels;
    pr.K = cv.R * cv.S * cv.C;
    pr.split_k = cls >= 0 ? 1 : choose_split_k(pr.M, pr.N, pr.K, 1);
    HE_REQUIRE(pr.M > 0 && pr.M < (1ll << 31) && ir::num_elements(flow.shape) < (1ll << 32), HE_ERR_UNSUPPORTED, "conv too large for 32-bit tile indices");
    pr.mma_dtype = flow.dtype == HE_F32 ? HE_F32 : flow.dtype == HE_F16 ? HE_F16 : HE_BF16;
    HE_REQUIRE(in_channels % (pr.mma_dtype == HE_F32 ? 4 : 8) == 0, HE_ERR_UNSUPPORTED,
               "conv backward data needs an input-channel count that fills 16-byte chunks");
    pr.b_rows.on = true;
    pr.b_rows.group = cv.C;                                 // k = (r*S + s) * out_channels + o
    pr.b_rows.o_stride = full_r * full_s * in_channels;     // filter[o][..]
    pr.b_rows.rs_stride = in_channels;                      // filter[.][r][s][..]
    if (cls >= 0) {                                         // filter[.][r0 + stride_h * r'][s0 + stride_w * s'][..]
        pr.b_rows.s_count = cv.S;
        pr.b_rows.base = (r0 * full_s + s0) * in_channels;
        pr.b_rows.r_stride = stride_h * full_s * in_channels;
        pr.b_rows.s_stride = stride_w * in_channels;
    }
    auto operand = [&](tp::Program& p, const ir::Descriptor& d, NodeId n, int64_t rows, int64_t cols) {
        p.dims = {1, rows, cols};
        p.args.push_back({d.dtype, ir::num_elements(d.shape), false, n});
        tp::Expr e;
        e.kind = tp::Expr::Load;
        e.cls = tp::Cls::F;
        e.access.arg = 0;
        e.access.dtype = d.dtype;
        e.access.stride = ir::packed_strides(p.dims);
        p.exprs.push_back(e);
    };
    operand(pr.op_a, flow, op.inputs[0], pr.M, pr.K);    // stand-ins: only the arguments are used
    operand(pr.op_b, filter, op.inputs[1], pr.K, pr.N);
    pr.root_a = pr.root_b = 0;
    pr.epi.dims = {1, pr.M, pr.N};
    pr.epi.fast_math = true;
    tp::Expr acc;
    acc.kind = tp::Expr::Acc;
    acc.cls = tp::Cls::F;
    pr.epi.exprs.push_back(acc);
    pr.epi.acc_expr = 0;
    tp::Out o;
    o.expr = 0;
    o.arg = 0;
    o.dtype = out.dtype;
    pr.epi.outs.push_back(o);
    pr.epi.args.push_back({out.dtype, ir::num_elements(out.shape), true, node});
    validate_gemm_epilogue(pr.epi);
    assemble_gemm_args(pr);
    return pr;
}
}  // namespace

namespace {
int filter_gradient_split_k(const GemmProblem& pr, bool element_gather);
// Op::ConvBackwardFilter as a GEMM: rows = output channels o, columns = filter taps (r, s, c), k = output pixels
// (n, p, q). A is the flow read as [k][m] (its own memory order: m contiguous); B[k][(r, s, c)] is gathered from the
// image with the forward convolution's map. The product has few output tiles and a very long k, so the k range is
// split over many workgroups whose partial tiles a second launch adds up.
GemmProblem conv_backward_filter_problem(const ir::OpSubgraph& sg, NodeId node) {
    const ir::OpGraph& g = *sg.graph();
    HE_REQUIRE(sg.nodes().size() == 1, HE_ERR_UNSUPPORTED, "a convolution instruction holds the op alone");
    const ir::Op& op = g.get(node).op;
    const ir::Descriptor &flow = g.get(op.inputs[0]).desc, &image = g.get(op.inputs[1]).desc, &out = g.get(node).desc;
    HE_REQUIRE(flow.shape.size() == 4 && image.shape.size() == 4, HE_ERR_INVALID, "conv backward takes rank-4 tensors");
    HE_REQUIRE(dtype_class(flow.dtype) == DataClass::Float && image.dtype == flow.dtype, HE_ERR_UNSUPPORTED,
               "conv backward takes a float flow and an image of the same type");
    HE_REQUIRE(flow.shape[3] == op.conv.out_channels && image.shape[3] == op.conv.in_channels && flow.shape[0] == image.shape[0],
               HE_ERR_INVALID, "conv backward filter: flow / image shapes do not match the parameters");
    GemmProblem pr;
    auto& cv = pr.conv_b;
    cv.on = true;
    cv.N = image.shape[0]; cv.H = image.shape[1]; cv.W = image.shape[2]; cv.C = image.shape[3];
    cv.R = op.conv.kernel[0]; cv.S = op.conv.kernel[1];
    cv.P = flow.shape[1]; cv.Q = flow.shape[2];
    cv.sh = op.conv.stride[0]; cv.sw = op.conv.stride[1];
    cv.dh = op.conv.dilation[0]; cv.dw = op.conv.dilation[1];
    int64_t pad[2];
    op.conv.padding(pad);
    cv.ph = pad[0]; cv.pw = pad[1];
    pr.batch = 1;
    pr.M = op.conv.out_channels;
    pr.N = cv.R * cv.S * cv.C;
    pr.K = cv.N * cv.P * cv.Q;
    HE_REQUIRE(pr.K > 0 && pr.K < (1ll << 31) && ir::num_elements(image.shape) < (1ll << 32), HE_ERR_UNSUPPORTED, "conv too large for 32-bit tile indices");
    pr.mma_dtype = flow.dtype == HE_F32 ? HE_F32 : flow.dtype == HE_F16 ? HE_F16 : HE_BF16;
    auto operand = [&](tp::Program& p, const ir::Descriptor& d, NodeId n, int64_t rows, int64_t cols) {
        p.dims = {1, rows, cols};
        p.args.push_back({d.dtype, ir::num_elements(d.shape), false, n});
        tp::Expr e;
        e.kind = tp::Expr::Load;
        e.cls = tp::Cls::F;
        e.access.arg = 0;
        e.access.dtype = d.dtype;
        e.access.stride = ir::packed_strides(p.dims);
        p.exprs.push_back(e);
    };
    operand(pr.op_a, flow, op.inputs[0], pr.K, pr.M);   // [k][m] as stored
    pr.a_km = true;
    operand(pr.op_b, image, op.inputs[1], pr.K, pr.N);  // stand-in: only the argument is used
    pr.root_a = pr.root_b = 0;
    pr.split_k = filter_gradient_split_k(pr, image.dtype != HE_F32 && cv.C % 8 != 0);
    pr.epi.dims = {1, pr.M, pr.N};
    pr.epi.fast_math = true;
    tp::Expr acc;
    acc.kind = tp::Expr::Acc;
    acc.cls = tp::Cls::F;
    pr.epi.exprs.push_back(acc);
    pr.epi.acc_expr = 0;
    tp::Out o;
    o.expr = 0;
    o.arg = 0;
    o.dtype = out.dtype;
    pr.epi.outs.push_back(o);
    pr.epi.args.push_back({out.dtype, ir::num_elements(out.shape), true, node});
    validate_gemm_epilogue(pr.epi);
    assemble_gemm_args(pr);
    return pr;
}
}  // namespace

std::vector<GemmProblem> strided_data_gradient_classes(const ir::OpSubgraph& sg, bool* any_empty) {
    const ir::OpGraph& g = *sg.graph();
    *any_empty = false;
    if (sg.nodes().size() != 1 || tuning::get("HELIUM_HIP_GEMM_NO_STRIDE_CLASSES")) return {};
    const ir::Op& op = g.get(sg.nodes()[0]).op;
    if (op.kind != ir::OpKind::ConvBackwardData || (op.conv.stride[0] == 1 && op.conv.stride[1] == 1) || op.conv.dilation[0] != 1 ||
        op.conv.dilation[1] != 1 || op.conv.stride[0] > 4 || op.conv.stride[1] > 4)
        return {};
    std::vector<GemmProblem> out;
    for (int cls = 0; cls < (int)(op.conv.stride[0] * op.conv.stride[1]); cls++) {
        bool empty = false;
        GemmProblem pr = conv_backward_data_problem(sg, sg.nodes()[0], cls, &empty);
        if (empty) *any_empty = true;
        else out.push_back(std::move(pr));
    }
    return out;
}

namespace {
int filter_gradient_split_k(const GemmProblem& pr, bool element_gather) {
    // about two workgroups per CU, each with at least four 64-wide k-tiles (128x128 output tiles)
    const int64_t tiles = ((pr.M + 127) / 128) * ((pr.N + 127) / 128), k_tiles = (pr.K + 63) / 64;
    // (many shares are rounded down: a few workgroups more than fit at once make a second round of the whole launch -
    // the 56x56x64 layer 102 -> 87 us; few shares are rounded up: 3 instead of 4 leave a quarter of the chip idle)
    const int64_t shares = 512 / tiles >= 32 ? 512 / tiles : (512 + tiles - 1) / tiles;
    int split = (int)std::max<int64_t>(1, std::min<int64_t>({shares, k_tiles / 4, 1024}));
    // Measured at batch 128 on the resnet-train layers (us per graph, fold launch included), and kept where batch 64 and the
    // stride-2 layers do not lose:
    //  - 128 output channels take 128x256 tiles (gemm.cpp), one workgroup per CU: the 28x28x128 layer 73.7 -> 61.8
    //    (5 tiles x 50 shares against 9 x 56 of 128x128), at batch 64 45.8 -> 43.6, the stride-2 56x56x64 -> 128 layer 50.8 -> 44.5;
    //  - 512 output channels keep 256x256 tiles, whose count, not that of 128x128 tiles, decides the shares as long as a
    //    share keeps 12 k-tiles: the 7x7x512 layer 36 x 4 = 144 workgroups 77.4 us, 36 x 7 = 252 workgroups 70.3.
    if (tuning::get("HELIUM_HIP_GEMM_NO_WIDE_CONV_TILES")) {
        // (the shares as they were, for comparison)
    } else if (!element_gather && pr.M > 64 && pr.M <= 128 && pr.N >= 512) {
        const int64_t wide = (pr.N + 255) / 256;
        split = (int)std::max<int64_t>(1, std::min<int64_t>({256 / wide, k_tiles / 4, 1024}));
    } else if (!element_gather && pr.M >= 512 && pr.N >= 512) {
        const int64_t large = ((pr.M + 255) / 256) * ((pr.N + 255) / 256);
        const int64_t s256 = std::min<int64_t>(256 / large, k_tiles / 12);
        if (s256 * large >= 192) split = (int)s256;
    }
    // (an image whose channels do not fill 16-byte chunks is gathered element by element, by 32x64 tiles of two waves: six
    // workgroups per CU, one round of them over the chip)
    if (element_gather && pr.M <= 32 && pr.M > 16 && pr.N >= 128)
        split = (int)std::max<int64_t>(1, std::min<int64_t>({1536 / ((pr.N + 63) / 64), k_tiles / 4, 1024}));
    if (const char* env = tuning::get("HELIUM_HIP_GEMM_SPLIT_K")) split = std::max(1, atoi(env));
    return split;
}

// A forward convolution or a filter gradient over a 16-bit image of 3 or 4 channels with an even stride along w and no
// dilation along w: the same product over the image repacked to 4 channels with its padding written out, two pixels
// making one 8-channel pixel of an image of half the width (kernels.h: ConvRepack). `packed` is that product: the image
// argument stands for the copy [N, Hp, Wp / 2, 8], the filter argument (the output, for a filter gradient) for
// [O, R, ceil(S / 2), 8].
bool over_repacked_image(const GemmProblem& pr, GemmProblem* packed, ConvRepack* geo) {
    const bool fwd = pr.conv_a.on && !pr.conv_a.bwd, grad = pr.conv_b.on;
    if ((!fwd && !grad) || pr.mma_dtype == HE_F32 || tuning::get("HELIUM_HIP_GEMM_NO_REPACK")) return false;
    const GemmProblem::ConvGather& cv = fwd ? pr.conv_a : pr.conv_b;
    if (cv.C < 3 || cv.C > 4 || cv.dw != 1 || cv.sw % 2 != 0 || cv.S < 2) return false;
    const int image_arg = fwd ? pr.map_a[0] : pr.map_b[0];
    const int filter_arg = fwd ? pr.map_b[0] : pr.map_e[pr.epi.outs[0].arg];
    // (an epilogue that reads the image or the filter itself would see the copies)
    for (size_t i = 0; i < pr.epi.args.size(); i++)
        if (!pr.epi.args[i].is_output && (pr.map_e[i] == image_arg || pr.map_e[i] == filter_arg)) return false;
    ConvRepack g;
    g.filter_gradient = grad;
    g.N = cv.N; g.H = cv.H; g.W = cv.W; g.C = cv.C;
    g.O = fwd ? pr.N : pr.M; g.R = cv.R; g.S = cv.S;
    g.Sp = (cv.S + 1) / 2 * 2;
    g.Hp = (cv.P - 1) * cv.sh + (cv.R - 1) * cv.dh + 1;
    g.Wp = (cv.Q - 1) * cv.sw + g.Sp;
    g.ph = cv.ph; g.pw = cv.pw;
    g.image_arg = image_arg; g.filter_arg = filter_arg;
    g.elem_bytes = grad ? dtype_bits(pr.args[filter_arg].dtype) / 8 : 2;
    if (g.N * g.Hp * g.Wp * 4 >= (1ll << 31)) return false;
    *packed = pr;
    GemmProblem::ConvGather& pv = fwd ? packed->conv_a : packed->conv_b;
    pv.H = g.Hp; pv.W = g.Wp / 2; pv.C = 8; pv.S = g.Sp / 2; pv.sw = cv.sw / 2; pv.ph = 0; pv.pw = 0;
    const int64_t taps = pv.R * pv.S * pv.C;
    auto resize = [](tp::Program& p, int64_t rows, int64_t cols, int64_t numel) {
        p.dims = {1, rows, cols};
        p.args[0].numel = numel;
        p.exprs[0].access.stride = ir::packed_strides(p.dims);
    };
    if (fwd) {
        packed->K = taps;
        resize(packed->op_a, packed->M, packed->K, g.N * g.Hp * g.Wp * 4);
        resize(packed->op_b, packed->N, packed->K, g.O * taps);
        if (pr.split_k > 1) packed->split_k = choose_split_k(packed->M, packed->N, packed->K, 1);
    } else {
        packed->N = taps;
        resize(packed->op_b, packed->K, packed->N, g.N * g.Hp * g.Wp * 4);
        packed->epi.dims = {1, packed->M, packed->N};
        packed->epi.args[0].numel = g.O * taps;
        packed->split_k = filter_gradient_split_k(*packed, false);
    }
    assemble_gemm_args(*packed);
    *geo = g;
    return true;
}
}  // namespace

// Whether the launch that folds the epilogue reductions of the product `large` can also evaluate the small pointwise
// instruction `small` (tp::attach_post): a plain product (no classes of a strided data gradient, no repacked image, a
// whole k range) whose column sums the small program reads.
bool gemm_can_carry(const ir::OpSubgraph& large, const ir::OpSubgraph& small) {
    bool any_empty = false;
    if (!strided_data_gradient_classes(large, &any_empty).empty()) return false;
    GemmProblem pr = gemm_problem_from_ir(large);
    ConvRepack geometry;
    GemmProblem packed;
    if (over_repacked_image(pr, &packed, &geometry) || pr.split_k != 1 || pr.batch != 1) return false;
    return tp::attach_post(&pr.epi, tp::lower_pointwise(small));
}

std::unique_ptr<KernelBase> make_gemm_kernel(const ir::OpSubgraph& sg, const ir::OpSubgraph* carried, bool beside_main_chain) {
    if (carried) {
        GemmProblem pr = gemm_problem_from_ir(sg);
        HE_REQUIRE(tp::attach_post(&pr.epi, tp::lower_pointwise(*carried)), HE_ERR_INTERNAL, "the carried instruction does not fit the fold launch any more");
        assemble_gemm_args(pr);
        return std::unique_ptr<KernelBase>(new GemmKernel(std::move(pr)));
    }
    // The data gradient of a strided convolution is one product per class of pixels (row and column modulo the
    // stride): each multiplies only the taps that reach its pixels.
    bool any_empty = false;
    std::vector<GemmProblem> classes = strided_data_gradient_classes(sg, &any_empty);
    if (!classes.empty()) {
        std::vector<std::unique_ptr<KernelBase>> parts;
        for (auto& pr : classes) parts.emplace_back(new GemmKernel(std::move(pr)));
        return std::unique_ptr<KernelBase>(new CompositeKernel(std::move(parts), any_empty));
    }
    GemmProblem pr = gemm_problem_from_ir(sg);
    // A filter gradient that runs beside the main chain takes 0.4 of the workgroups it would take alone: four in ten of
    // the CUs are then busy with it and the main chain's kernels keep the rest, where a launch that fills the chip
    // holds every main-chain kernel back until its workgroups retire. Measured on the training step at batch 128
    // (shares of 1 / 0.5 / 0.4 / 0.33 / 0.25 / 0.2: 4.49 / 4.42 / 4.39 / 4.40 / 4.39 / 4.67 ms - below a quarter the side
    // stream becomes the longer chain); fewer shares also write and re-read fewer partial tiles.
    if (beside_main_chain && pr.conv_b.on && pr.split_k > 1) {
        const double share = tuning::get("HELIUM_HIP_SIDE_SPLIT_SCALE") ? atof(tuning::get("HELIUM_HIP_SIDE_SPLIT_SCALE")) : 0.4;
        pr.split_k = std::max(1, (int)(pr.split_k * share + 0.5));
    }
    ConvRepack geometry;
    GemmProblem packed;
    if (over_repacked_image(pr, &packed, &geometry)) {
        std::vector<tp::Arg> args = pr.args;
        return std::unique_ptr<KernelBase>(new RepackedConvKernel(std::move(args), geometry, std::unique_ptr<KernelBase>(new GemmKernel(std::move(packed)))));
    }
    return std::unique_ptr<KernelBase>(new GemmKernel(std::move(pr)));
}

GemmProblem gemm_problem_from_ir(const ir::OpSubgraph& sg) {
    const ir::OpGraph& g = *sg.graph();
    for (NodeId n : sg.nodes()) {
        if (g.get(n).op.kind == ir::OpKind::ConvBackwardFilter) return conv_backward_filter_problem(sg, n);
        if (g.get(n).op.kind == ir::OpKind::Conv) return conv_problem(sg, n);
        if (g.get(n).op.kind == ir::OpKind::ConvBackwardData) return conv_backward_data_problem(sg, n);
    }
    NodeId mm = ir::kNoNode;
    for (NodeId n : sg.nodes())
        if (g.get(n).op.kind == ir::OpKind::Matmul) {
            HE_REQUIRE(mm == ir::kNoNode, HE_ERR_UNSUPPORTED, "a GEMM fusion holds one Matmul");
            mm = n;
        }
    HE_REQUIRE(mm != ir::kNoNode, HE_ERR_UNSUPPORTED, "no Matmul in the subgraph");  // find_matmul (matmul.rs:222-233)
    const ir::Op& op = g.get(mm).op;
    const ir::Descriptor &da = g.get(op.inputs[0]).desc, &db = g.get(op.inputs[1]).desc, &dc = g.get(mm).desc;
    HE_REQUIRE(da.shape.size() >= 2 && da.shape.size() == db.shape.size(), HE_ERR_UNSUPPORTED, "matmul operand ranks differ");
    const size_t r = da.shape.size();
    int64_t batch = 1;
    for (size_t i = 0; i + 2 < r; i++) {
        HE_REQUIRE(da.shape[i] == db.shape[i], HE_ERR_UNSUPPORTED, "matmul batch extents differ");
        batch *= da.shape[i];
    }
    HE_REQUIRE(da.shape[r - 1] == db.shape[r - 2], HE_ERR_INVALID, "matmul inner extents differ");
    HE_REQUIRE(dtype_class(da.dtype) == DataClass::Float && dtype_class(db.dtype) == DataClass::Float, HE_ERR_UNSUPPORTED,
               "matmul takes float operands");
    GemmProblem pr;
    pr.batch = batch;
    pr.M = da.shape[r - 2];
    pr.K = da.shape[r - 1];
    pr.N = db.shape[r - 1];
    // Multiplicand type by Precision (precision.rs:36-81): never less precise than asked for. TF32 and F8 have no
    // matrix-core form here; TF32 runs as f32, F8 as bf16.
    switch (op.precision) {
        case ir::Precision::MulF32AccumF32:
        case ir::Precision::MulTf32AccumF32: pr.mma_dtype = HE_F32; break;
        case ir::Precision::MulF16AccumF32:
        case ir::Precision::MulF16AccumF16: pr.mma_dtype = HE_F16; break;
        default: pr.mma_dtype = HE_BF16; break;
    }
    // An operand is a subgraph input, or (beyond the reference, whose matmul takes materialised operands only) a
    // SwapDims of the two matrix dims of one: `x.transpose().matmul(dy)`, `dy.matmul(w.transpose())` of a linear
    // layer's backward pass. The transposed tensor is then never written: the kernel reads the source as it lies.
    size_t operand_swaps = 0;
    auto operand = [&](tp::Program& p, NodeId node, int64_t rows, int64_t cols) -> bool {
        bool swapped = false;
        if (!sg.is_input(node)) {
            const ir::Node& sn = g.get(node);
            const int64_t rank = (int64_t)sn.desc.shape.size();
            const bool last_two = sn.kind == ir::Node::Intermediate && sn.op.kind == ir::OpKind::SwapDims &&
                                  std::min(sn.op.axis_a, sn.op.axis_b) == rank - 2 && std::max(sn.op.axis_a, sn.op.axis_b) == rank - 1;
            HE_REQUIRE(last_two && sg.contains(node) && sg.is_input(sn.op.inputs[0]) && g.outbound(node).size() == 1, HE_ERR_UNSUPPORTED,
                       "ops that feed a Matmul operand are fused through the fusion IR only (a transposition of the matrix dims aside)");
            swapped = true;
            operand_swaps++;
            node = sn.op.inputs[0];
        }
        const ir::Descriptor& d = g.get(node).desc;
        p.dims = swapped ? ir::Shape{batch, cols, rows} : ir::Shape{batch, rows, cols};
        p.args.push_back({d.dtype, ir::num_elements(d.shape), false, node});
        tp::Expr e;
        e.kind = tp::Expr::Load;
        e.cls = tp::Cls::F;
        e.access.arg = 0;
        e.access.dtype = d.dtype;
        e.access.stride = ir::packed_strides(p.dims);
        p.exprs.push_back(e);
        return swapped;
    };
    pr.a_km = operand(pr.op_a, op.inputs[0], pr.M, pr.K);
    pr.b_nk = operand(pr.op_b, op.inputs[1], pr.K, pr.N);
    pr.root_a = pr.root_b = 0;
    if (sg.nodes().size() == 1 + operand_swaps) {
        pr.epi.dims = {batch, pr.M, pr.N};
        pr.epi.fast_math = true;
        tp::Expr acc;
        acc.kind = tp::Expr::Acc;
        acc.cls = tp::Cls::F;
        pr.epi.exprs.push_back(acc);
        pr.epi.acc_expr = 0;
        tp::Out o;
        o.expr = 0;
        o.arg = 0;
        o.dtype = dc.dtype;  // the accumulator type (op.rs:61-73)
        pr.epi.outs.push_back(o);
        pr.epi.args.push_back({dc.dtype, ir::num_elements(dc.shape), true, mm});
    } else {
        // Matmul + the pointwise / reduce ops after it: the epilogue runs on the accumulators
        // (MatmulGenerator's leaves, matmul.rs:88-130).
        pr.epi = tp::lower_ir_epilogue(sg, mm);
    }
    validate_gemm_epilogue(pr.epi);
    assemble_gemm_args(pr);
    return pr;
}

}  // namespace he::plan
