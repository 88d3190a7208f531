// C ABI of the fusion search: a whole fusion-IR graph -> Core / Aux fusions -> one kernel per fusion, run in
// dependency order.
#include <sstream>

#include "capi_types.h"
#include "exec.h"
#include "fused_graph.h"

namespace {
using namespace he;
using fsearch::FusionId;
using fir::OpNode;

struct FusionKernel {
    std::unique_ptr<KernelBase> kernel;
    // per kernel argument: the (provider fusion, node) whose buffer it binds
    std::vector<std::pair<FusionId, OpNode>> bindings;
};
}  // namespace

struct he_fusion_plan_s {
    std::shared_ptr<const fir::OpGraph> g;
    fsearch::FusedGraph fg = fsearch::FusedGraph::identity(std::make_shared<fir::OpGraph>());
    double cost = 0;
    size_t states = 0;
    std::vector<FusionId> order;  // fusions that become kernels, in dependency order
    std::map<FusionId, FusionKernel> kernels;
    std::string text;
    std::mutex mu;
};

namespace {
// Storage type of a value that crosses a kernel boundary: what its Producer / Consumer declares, f32 for
// reductions, bf16 otherwise (the reference's generated kernels pass every tensor as bf16).
int boundary_dtype(const fir::OpGraph& g, OpNode n) {
    const fir::Op& op = g.get(n);
    if (op.kind == fir::OpKind::Producer) return op.dtype;
    for (OpNode c : g.outbound(n))
        if (g.get(c).kind == fir::OpKind::Consumer) return g.get(c).dtype;
    return op.kind == fir::OpKind::Reduction ? HE_F32 : HE_BF16;
}

FusionKernel& kernel_of(he_fusion_plan_s& plan, FusionId id) {
    std::lock_guard<std::mutex> lk(plan.mu);
    auto it = plan.kernels.find(id);
    if (it != plan.kernels.end()) return it->second;
    const fsearch::Fusion& f = plan.fg.fusions().at(id);
    const fir::OpGraph& g = *plan.g;
    fir::OpGraph sub;
    FusionKernel fk;
    // producers stand for the values other fusions provide, under the provided node's own id
    for (auto& [dep, provider] : f.dependencies) {
        fir::Op p;
        p.kind = fir::OpKind::Producer;
        p.shape = g.shape(dep);
        p.dtype = boundary_dtype(g, dep);
        sub.insert_with_id(dep, p);
        fk.bindings.push_back({provider, dep});
    }
    // members go in after what they read (ids need not follow the dataflow: the README numbers its mainloop ops
    // above their anchor)
    std::vector<OpNode> members = f.nodes();
    std::sort(members.begin(), members.end());
    std::set<OpNode> placed;
    while (placed.size() < members.size()) {
        bool progressed = false;
        for (OpNode n : members) {
            if (placed.count(n)) continue;
            bool ready = true;
            for (OpNode in : g.get(n).inputs()) ready = ready && (sub.has(in) || !f.contains(in));
            if (!ready) continue;
            sub.insert_with_id(n, g.get(n));
            placed.insert(n);
            progressed = true;
        }
        HE_REQUIRE(progressed, HE_ERR_INTERNAL, "fusion %llu has a cycle", (unsigned long long)id);
    }
    // one consumer per distinct value this fusion provides
    std::set<OpNode> provided;
    for (auto& d : f.dependents) provided.insert(d.first);
    HE_REQUIRE(!provided.empty(), HE_ERR_INVALID, "fusion %llu provides nothing", (unsigned long long)id);
    OpNode next_id = g.nodes().back() + 1;
    for (OpNode n : provided) {
        fir::Op c;
        c.kind = fir::OpKind::Consumer;
        c.a = n;
        c.dtype = boundary_dtype(g, n);
        sub.insert_with_id(next_id++, c);
        fk.bindings.push_back({id, n});
    }
    if (f.core) fk.kernel.reset(new GemmKernel(gemm_problem_from_fusion(sub)));
    else fk.kernel.reset(new TileKernel(tp::lower_aux(sub), "fused_auxiliary"));
    HE_REQUIRE(fk.kernel->args().size() == fk.bindings.size(), HE_ERR_INTERNAL, "fusion %llu: %zu kernel arguments for %zu bindings",
               (unsigned long long)id, fk.kernel->args().size(), fk.bindings.size());
    return plan.kernels.emplace(id, std::move(fk)).first->second;
}
}  // namespace

extern "C" {

namespace {
void fusion_search(he_fgraph_t graph, int objective, bool subdivided, he_fusion_plan_t* plan) {
    HE_REQUIRE(graph && plan && objective >= 0 && objective <= 3, HE_ERR_INVALID, "bad argument");
    {
        // he_fusion_plan_execute hands every value to one caller buffer: a value that two Consumers read is refused here,
        // before anything is compiled or launched
        std::set<OpNode> consumed;
        for (OpNode n : graph->g.nodes()) {
            const fir::Op& op = graph->g.get(n);
            if (op.kind != fir::OpKind::Consumer) continue;
            HE_REQUIRE(consumed.insert(op.a).second, HE_ERR_UNSUPPORTED, "value %llu is read by two Consumers: a plan writes each value to one buffer",
                       (unsigned long long)op.a);
        }
    }
    auto p = std::make_unique<he_fusion_plan_s>();
    p->g = std::make_shared<fir::OpGraph>(graph->g);
    const auto params = fsearch::CostParams::mi355x();
    fsearch::SearchResult r = subdivided ? fsearch::minimize_cost_with_subdivision(p->g, (fsearch::Objective)objective, params)
                                         : fsearch::minimize_cost(p->g, (fsearch::Objective)objective, params);
    r.graph.assert_invariants(false);
    p->fg = r.graph;
    p->cost = r.cost;
    p->states = r.states_visited;
    for (FusionId id : p->fg.topo_sort())
        if (!p->fg.fusions().at(id).is_input_output(*p->g)) p->order.push_back(id);
    p->text = p->fg.describe();
    *plan = p.release();
}
}  // namespace

int he_fusion_search(he_fgraph_t graph, int objective, he_fusion_plan_t* plan) {
    return he::guard([&] { fusion_search(graph, objective, false, plan); });
}

int he_fusion_search_subdivided(he_fgraph_t graph, int objective, he_fusion_plan_t* plan) {
    return he::guard([&] { fusion_search(graph, objective, true, plan); });
}

int he_fusion_plan_num_fusions(he_fusion_plan_t plan, int* count) {
    return he::guard([&] { *count = (int)plan->order.size(); });
}

int he_fusion_plan_fusion_info(he_fusion_plan_t plan, int index, int32_t* is_core, uint64_t* anchor, uint64_t* nodes,
                               int32_t* roles, int capacity, int* count) {
    return he::guard([&] {
        HE_REQUIRE(plan && index >= 0 && index < (int)plan->order.size() && count, HE_ERR_INVALID, "bad argument");
        const fsearch::Fusion& f = plan->fg.fusions().at(plan->order[index]);
        if (is_core) *is_core = f.core;
        if (anchor) *anchor = f.core ? f.anchor : 0;
        std::vector<std::pair<OpNode, int>> all;
        for (OpNode n : f.mainloop) all.push_back({n, HE_FUSION_ROLE_MAINLOOP});
        for (OpNode n : f.epilogue) all.push_back({n, HE_FUSION_ROLE_EPILOGUE});
        if (f.core) all.push_back({f.anchor, HE_FUSION_ROLE_ANCHOR});
        for (OpNode n : f.fused) all.push_back({n, HE_FUSION_ROLE_AUX});
        HE_REQUIRE((int)all.size() <= capacity, HE_ERR_INVALID, "fusion has %zu nodes, room for %d", all.size(), capacity);
        for (size_t i = 0; i < all.size(); i++) {
            nodes[i] = all[i].first;
            roles[i] = all[i].second;
        }
        *count = (int)all.size();
    });
}

const char* he_fusion_plan_describe(he_fusion_plan_t plan) { return plan ? plan->text.c_str() : ""; }

int he_fusion_plan_cost(he_fusion_plan_t plan, int objective, int reference_constants, double* cost, uint64_t* states_visited) {
    return he::guard([&] {
        HE_REQUIRE(plan && cost, HE_ERR_INVALID, "bad argument");
        const fsearch::CostParams p = reference_constants ? fsearch::CostParams::reference() : fsearch::CostParams::mi355x();
        *cost = objective == 3 ? fsearch::mi355x_cost(plan->fg) : objective == 2 ? fsearch::analytical_cost(plan->fg) : fsearch::naive_cost(plan->fg, p);
        if (states_visited) *states_visited = plan->states;
    });
}

int he_fusion_plan_cost_terms(he_fusion_plan_t plan, double* terms, int capacity, int* count) {
    return he::guard([&] {
        HE_REQUIRE(plan && terms && count && capacity >= fsearch::CostTerms::kCount, HE_ERR_INVALID, "bad argument");
        double v[fsearch::CostTerms::kCount];
        fsearch::mi355x_cost_terms(plan->fg).to_array(v);
        for (int i = 0; i < fsearch::CostTerms::kCount; i++) terms[i] = v[i];
        *count = fsearch::CostTerms::kCount;
    });
}

int he_fusion_plan_precompile(he_fusion_plan_t plan) {
    return he::guard([&] {
        for (FusionId id : plan->order) (void)kernel_of(*plan, id);
    });
}

int he_fusion_plan_execute(he_fusion_plan_t plan, const uint64_t* producer_nodes, void* const* producer_ptrs, int num_producers,
                           const uint64_t* consumer_nodes, void* const* consumer_ptrs, int num_consumers, he_stream_t stream) {
    return he::guard([&] {
        HE_REQUIRE(plan, HE_ERR_INVALID, "null plan");
        const fir::OpGraph& g = *plan->g;
        hipStream_t s = stream ? stream->s : nullptr;
        std::map<std::pair<FusionId, OpNode>, void*> buffers;
        std::vector<std::pair<void*, void*>> copies;  // further Consumers of a value that already has a buffer
        // graph inputs
        for (int i = 0; i < num_producers; i++) {
            HE_REQUIRE(g.has(producer_nodes[i]) && g.get(producer_nodes[i]).kind == fir::OpKind::Producer, HE_ERR_INVALID,
                       "node %llu is not a Producer", (unsigned long long)producer_nodes[i]);
            buffers[{plan->fg.fusions_of(producer_nodes[i])[0], producer_nodes[i]}] = producer_ptrs[i];
        }
        // graph outputs: the value a Consumer reads lives in the caller's buffer
        std::map<OpNode, void*> out_ptr;
        for (int i = 0; i < num_consumers; i++) out_ptr[consumer_nodes[i]] = consumer_ptrs[i];
        for (auto& [id, f] : plan->fg.fusions()) {
            if (!f.is_input_output(g)) continue;
            const OpNode n = f.nodes()[0];
            if (g.get(n).kind == fir::OpKind::Producer) {
                HE_REQUIRE(f.dependents.empty() || buffers.count({id, n}), HE_ERR_INVALID, "no buffer given for Producer %llu", (unsigned long long)n);
                continue;
            }
            auto it = out_ptr.find(n);
            HE_REQUIRE(it != out_ptr.end(), HE_ERR_INVALID, "no buffer given for Consumer %llu", (unsigned long long)n);
            const OpNode x = g.get(n).a;
            const auto key = std::make_pair(f.dependencies.at(x), x);
            if (!buffers.count(key)) buffers[key] = it->second;
            else copies.push_back({it->second, buffers[key]});
        }
        HE_REQUIRE(copies.empty(), HE_ERR_INTERNAL, "a value with two Consumers passed the check of he_fusion_search");
        exec::DevicePool& pool = exec::DevicePool::global();
        const uint64_t scope = pool.begin_scope();
        std::vector<exec::TensorRef> temporaries;
        for (FusionId id : plan->order) {
            FusionKernel& fk = kernel_of(*plan, id);
            const auto& args = fk.kernel->args();
            std::vector<void*> ptrs(args.size());
            for (size_t a = 0; a < args.size(); a++) {
                auto it = buffers.find(fk.bindings[a]);
                if (it == buffers.end()) {
                    HE_REQUIRE(args[a].is_output, HE_ERR_INTERNAL, "fusion %llu reads node %llu before it was produced", (unsigned long long)id,
                               (unsigned long long)fk.bindings[a].second);
                    exec::TensorRef t = exec::allocate_tensor(args[a].dtype, (size_t)args[a].numel, scope);
                    temporaries.push_back(t);
                    it = buffers.emplace(fk.bindings[a], t->ptr).first;
                }
                ptrs[a] = it->second;
            }
            fk.kernel->execute(ptrs.data(), s);
        }
        exec::EventRef done = pool.take_event();
        HE_HIP(hipEventRecord(done->e, s));
        temporaries.clear();  // blocks return to the scope; the pool frees them for others when `done` has passed
        pool.end_scope_after(scope, std::move(done));
    });
}

int he_fusion_plan_destroy(he_fusion_plan_t plan) {
    delete plan;
    return HE_OK;
}

int he_fgraph_subdivide(he_fgraph_t graph, uint64_t* nodes, int32_t* portions, int32_t* subdivision_of, int capacity, int* count) {
    return he::guard([&] {
        HE_REQUIRE(graph && count, HE_ERR_INVALID, "bad argument");
        auto subs = fsearch::subdivide(graph->g);
        int k = 0;
        for (size_t s = 0; s < subs.size(); s++)
            for (auto& [n, p] : subs[s]) {
                HE_REQUIRE(k < capacity, HE_ERR_INVALID, "room for %d entries is not enough", capacity);
                nodes[k] = n;
                portions[k] = (int)p;
                subdivision_of[k] = (int)s;
                k++;
            }
        *count = k;
    });
}

}  // extern "C"
