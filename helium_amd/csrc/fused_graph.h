// Fusion search over a fusion-IR graph: which ops share a kernel, as Core(mainloop, anchor, epilogue) and Aux
// fusions with recomputation allowed — helium-playground/src/fused_graph.rs (FusedGraph, Fusion, Action),
// cost_model.rs (naive / analytical cost, minimize_cost_function) and subdivision.rs (subdivide).
#pragma once
#include <map>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "fusion_ir.h"

namespace he::fsearch {

using fir::OpNode;
using FusionId = uint64_t;
enum class NodePortion : int { Mainloop = 0, Epilogue = 1, Full = 2 };  // subdivision.rs:9-14

// fused_graph.rs:1082-1235
struct Fusion {
    bool core = false;
    OpNode anchor = fir::kNoOpNode;
    std::vector<OpNode> mainloop, epilogue;  // Core; sorted
    std::vector<OpNode> fused;               // Aux; sorted
    std::map<OpNode, FusionId> dependencies;               // node read from outside -> fusion that provides it
    std::set<std::pair<OpNode, FusionId>> dependents;      // (node of this fusion, fusion that reads it)

    std::vector<OpNode> nodes() const;  // mainloop, epilogue, anchor | fused (fused_graph.rs:1138-1150)
    bool contains(OpNode n) const;
    void remove_node(OpNode n);
    bool is_input_output(const fir::OpGraph& g) const;
    std::string key() const;  // canonical text of kind, members and edges (state identity)
};

// fused_graph.rs:1237-1263
struct Action {
    enum Kind { CoreFuseIntoEpilogue, CoreFuseIntoMainloop, AuxFuse, TransitionEdge } kind = AuxFuse;
    OpNode node = 0;        // the node fused / the transitioned input
    FusionId fusion = 0;    // the fusion that grows / whose edge moves
    std::map<OpNode, FusionId> providers;  // fuse actions: who provides each dependency the node brings along
    FusionId new_provider = 0;             // TransitionEdge
    bool operator==(const Action& o) const {
        return kind == o.kind && node == o.node && fusion == o.fusion && providers == o.providers && new_provider == o.new_provider;
    }
    std::string describe() const;
};

class FusedGraph {
public:
    // fused_graph.rs:62-111. Fusion ids count up from `first_id` (the reference draws them from one process-wide
    // counter, which is what lets graphs of several subdivisions be merged).
    static FusedGraph identity(std::shared_ptr<const fir::OpGraph> g, FusionId first_id = 0);
    void produce_maximal_fusions();                                      // :113-223
    void clean();                                                        // :237-282
    std::vector<Action> enumerate_possible_actions() const;              // :285-358
    void apply_action(const Action& a);                                  // :596-769
    std::vector<FusionId> topo_sort() const;                             // :878-908
    // :834-876. clean() drops what no Consumer reads, after which those nodes are in no fusion: pass false then.
    void assert_invariants(bool every_node_placed = true) const;
    uint64_t state_hash() const;  // order-independent over the fusions (:51-55)
    std::string describe() const; // the printed form (:1060-1068, :1152-1183)

    // fused_graph.rs:910-1058: one graph over `original` from the separately fused subdivisions (fusion ids must
    // not repeat between them). An anchor's fusion takes its epilogue from the subdivision that holds its epilogue
    // portion and its mainloop from the one that holds its mainloop portion.
    static FusedGraph merge_from_subdivisions(const std::vector<std::set<std::pair<OpNode, NodePortion>>>& subdivisions,
                                              const std::vector<FusedGraph>& fused, std::shared_ptr<const fir::OpGraph> original);

    const std::map<FusionId, Fusion>& fusions() const { return fusions_; }
    const fir::OpGraph& opgraph() const { return *g_; }
    const std::vector<FusionId>& fusions_of(OpNode n) const { return node_fusions_.at(n); }

private:
    bool would_create_cycle(FusionId from, FusionId to) const;  // :567-590
    std::vector<FusionId> dependency_providers(OpNode dep, FusionId fusion, std::map<std::pair<FusionId, FusionId>, bool>& cache) const;
    void epilogue_expansions(FusionId id, bool has_core, OpNode core, const std::vector<OpNode>& existing_epilogue,
                             const std::vector<OpNode>& existing_mainloop, std::vector<Action>& out,
                             std::map<std::pair<FusionId, FusionId>, bool>& cache) const;
    void mainloop_expansions(FusionId id, OpNode core, const std::vector<OpNode>& existing_mainloop, std::vector<Action>& out,
                             std::map<std::pair<FusionId, FusionId>, bool>& cache) const;
    void remove_edge(OpNode node, FusionId provider, FusionId consumer);  // :771-815
    void maybe_remove_collapsed(FusionId id);                             // :817-832
    bool try_fuse_singletons(Action::Kind kind);

    std::shared_ptr<const fir::OpGraph> g_;
    std::map<FusionId, Fusion> fusions_;
    std::map<OpNode, std::vector<FusionId>> node_fusions_;
};

// cost_model.rs:9-16: element rate of memory, matrix and vector FLOP rates.
struct CostParams {
    double memory_elements_per_s, tensor_flops, regular_flops;
    static CostParams reference() { return {2.4e11, 950.0e12, 67.0e12}; }
    // MI355X as measured by this backend: 5.9 TB/s of 2-byte elements, 1.0 PFLOP/s fused GEMM, 256 CUs x 64 lanes x
    // ~1.9 GHz of plain FP32 issue (packed FP32 is not used).
    static CostParams mi355x() { return {2.95e12, 1.0e15, 3.1e13}; }
};
double naive_cost(const FusedGraph& fg, const CostParams& p);  // cost_model.rs:9-89
double analytical_cost(const FusedGraph& fg);                   // cost_model.rs:91-231 (coefficients as published there)

// A cost model of the same purpose as the analytical one, for this backend's kernels on MI355X: the time of a plan
// is a sum over its kernels, linear in seven terms whose coefficients are fitted to measured kernels
// (harness/cost_fit.py measures and fits; profiles/cost_model_fit.txt holds the data). The terms say what the
// hardware bounds: matrix-core work, the bytes a kernel moves to and from HBM, the vector work of epilogue / anchor-less
// kernels, and - what makes a mainloop fusion lose on this chip - the operand traffic from L2 to the CUs, which every
// tile column (for A) or tile row (for B) of a product repeats: a fused `relu(A0) * T` makes 16 workgroups per tile row
// stream T next to A0, 1.5x the plain k-loop's bytes on a loop that is bound by exactly that stream.
struct CostTerms {
    double launches = 0;           // kernels, plus one fold launch per kernel that ends in reductions
    double mma_flops = 0;          // 2 b M N K of every anchor
    double mainloop_l2_bytes = 0;  // operand bytes streamed to the CUs beyond the two plain operands
    double mainloop_ops = 0;       // weighted vector ops on operand elements, times the tiles that repeat them
    double hbm_bytes = 0;          // tensors read from and written to memory by epilogues and anchor-less kernels
    double epilogue_ops = 0;       // weighted vector ops on accumulator elements
    double aux_ops = 0;            // weighted vector ops of anchor-less kernels
    static constexpr int kCount = 7;
    void to_array(double (&out)[kCount]) const;
};
struct Mi355xCoefficients {
    double c[CostTerms::kCount];
    static Mi355xCoefficients fitted();
};
CostTerms mi355x_cost_terms(const FusedGraph& fg);
double mi355x_cost(const FusedGraph& fg, const Mi355xCoefficients& k = Mi355xCoefficients::fitted());

// cost_model.rs:256-343: maximal fusions, then depth-7 searches from the best state until none improves.
// `max_states` bounds the states visited per search (the reference has no bound).
struct SearchResult {
    FusedGraph graph;
    double cost;
    size_t states_visited;
};
enum class Objective : int { Maximal = 0, Naive = 1, Analytical = 2, Mi355x = 3 };
SearchResult minimize_cost(std::shared_ptr<const fir::OpGraph> g, Objective objective, const CostParams& p, size_t max_states = 200000,
                           FusionId first_id = 0);
// cost_model.rs:241-259: subdivide, search every subdivision's subgraph on its own, merge. The search is exponential
// in the graph's size; the subdivisions are what keeps large graphs searchable.
SearchResult minimize_cost_with_subdivision(std::shared_ptr<const fir::OpGraph> g, Objective objective, const CostParams& p,
                                            size_t max_states = 200000);

// subdivision.rs:24-113
std::vector<std::set<std::pair<OpNode, NodePortion>>> subdivide(const fir::OpGraph& g);

}  // namespace he::fsearch
