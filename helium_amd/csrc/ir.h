// The helium-ir operation graph (helium-ir/src/opgraph.rs, opgraph/op.rs, opgraph/subgraph.rs, shape.rs),
// restated in C++ so that plan generation and the kernel generators consume the same structure the Rust
// front-end records.
#pragma once
#include <algorithm>
#include <cstdint>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "common.h"

namespace he::ir {

using NodeId = uint32_t;  // index into the graph's node table; ids are never reused within a graph
constexpr NodeId kNoNode = 0xffffffffu;

using Shape = std::vector<int64_t>;
int64_t num_elements(const Shape& s);
Shape packed_strides(const Shape& s);

enum class OpKind : int {
    Matmul = 0, UnaryPointwise, BinaryPointwise, ChangeDataType, Reduce, Broadcast, Reshape, SwapDims, Compare,
    Select, Conv, ConvBackwardData, ConvBackwardFilter, Constant
};
// opgraph/op.rs:291-304
enum class UnaryOp : int { Recip = 0, Neg, Exp, Sin, Cos, Tan, Sigmoid, Tanh, Relu, Sqrt, Log };
// opgraph/op.rs:315-328
enum class BinaryOp : int { Add = 0, Mul, Pow, Min, Max, And, Or, Xor };
// opgraph/op.rs:360-367
enum class ReduceOp : int { Sum = 0, Mean, Max, Min };
// opgraph/op.rs:429-437
enum class CompareOp : int { Equal = 0, NotEqual, LessThan, LessThanOrEqual, GreaterThan, GreaterThanOrEqual };
// opgraph/op/precision.rs:36-81 (the two FP8 variants carry their modes in `f8_modes`)
enum class Precision : int { MulF32AccumF32 = 0, MulTf32AccumF32, MulBf16AccumF32, MulF16AccumF32, MulF16AccumF16,
                             MulF8AccumF32, MulF8AccumF16 };
int accumulator_type(Precision p);  // precision.rs:87-96

struct BroadcastAxis {
    int64_t axis, new_size;
    bool operator==(const BroadcastAxis& o) const { return axis == o.axis && new_size == o.new_size; }
};

// Conv2dParams (opgraph/op/conv.rs:5-12) and ConvBackwardData::input_size (op.rs:462-468).
struct ConvParams {
    int64_t in_channels = 0, out_channels = 0;
    int64_t kernel[2] = {1, 1}, stride[2] = {1, 1}, dilation[2] = {1, 1};
    int padding_mode = 0;            // 0 Same, 1 Valid, 2 Full
    int64_t input_size[2] = {0, 0};  // ConvBackwardData only
    bool operator==(const ConvParams& o) const;
    // compute_output_size (conv.rs:51-73) and compute_padding_amount (conv.rs:85-91)
    void output_size(const int64_t in[2], const int64_t kernel_size[2], int64_t out[2]) const;
    void padding(int64_t pad[2]) const;
};

struct Op {
    OpKind kind = OpKind::Constant;
    std::vector<NodeId> inputs;  // Matmul: a,b; Binary/Compare: lhs,rhs; Select: lhs,rhs,selector
    int sub_op = 0;              // UnaryOp / BinaryOp / ReduceOp / CompareOp
    Precision precision = Precision::MulBf16AccumF32;
    int f8_modes = 0;
    int target_type = HE_F32;    // ChangeDataType
    uint32_t depth = 0;          // Reduce
    int64_t new_dim_count = 0;   // Broadcast
    std::vector<BroadcastAxis> broadcast_axes;
    Shape shape;                 // Reshape target / Constant shape
    int64_t axis_a = 0, axis_b = 0;
    uint32_t const_bits = 0;     // Constant scalar, bit pattern in its own dtype
    int const_dtype = HE_F32;
    ConvParams conv;             // Conv (image, filter), ConvBackwardData (flow, filter), ConvBackwardFilter (flow, image)
    bool operator==(const Op& o) const;
    uint64_t hash() const;
};

struct Descriptor {
    Shape shape;
    int dtype = HE_F32;
    bool operator==(const Descriptor& o) const { return shape == o.shape && dtype == o.dtype; }
};

struct Node {
    enum Kind { Input, Intermediate, Output, Removed } kind = Removed;
    Descriptor desc;
    Op op;  // Intermediate only
};

class OpGraph {
public:
    NodeId new_input(const Descriptor& d);
    NodeId new_op(Op op);  // infers the output descriptor (op.rs:52-179)
    NodeId new_output(NodeId from);
    void remove(NodeId id);
    void optimize();  // prune_unused (opgraph.rs:165-191)

    const Node& get(NodeId id) const;
    bool alive(NodeId id) const { return id < nodes_.size() && nodes_[id].kind != Node::Removed; }
    std::vector<NodeId> nodes() const;  // live nodes in id order
    size_t capacity() const { return nodes_.size(); }
    size_t num_nodes() const;
    const std::vector<NodeId>& inputs() const { return inputs_; }
    const std::vector<NodeId>& outputs() const { return outputs_; }
    const std::vector<NodeId>& inbound(NodeId id) const { return in_[id]; }
    const std::vector<NodeId>& outbound(NodeId id) const { return out_[id]; }
    bool feeds_output(NodeId id) const;
    uint64_t structural_hash() const;
    bool structurally_equal(const OpGraph& o) const;

    static Descriptor infer(const Op& op, const OpGraph& g);
    static Shape broadcast_output_shape(const Op& op, const Shape& in);

    // For a graph that `rematerialized` built: the node of the graph it was built from that a node stands for (several
    // nodes may stand for the same one; kNoNode for a helper node that stands for none); the node itself in any other graph.
    NodeId origin(NodeId id) const { return id < origin_.size() ? origin_[id] : id; }
    bool has_origins() const { return !origin_.empty(); }
    // When the graph this one was built from was itself built from another: origins then name that one's nodes.
    void rebase_origins(const OpGraph& through);
    // For a graph that `rematerialized` built: whether the node is a copy made for one consumer, to be computed in that
    // consumer's kernel. A kernel that would write such a copy to memory has the wrong one.
    bool made_for_consumer(NodeId id) const { return id < for_consumer_.size() && for_consumer_[id]; }

private:
    NodeId push(Node n);
    std::vector<Node> nodes_;
    std::vector<NodeId> inputs_, outputs_;
    std::vector<std::vector<NodeId>> in_, out_;
    std::vector<NodeId> origin_;
    std::vector<uint8_t> for_consumer_;
    friend std::shared_ptr<OpGraph> rematerialized(const OpGraph& g, const std::set<NodeId>& keep_single,
                                                   const std::set<std::vector<NodeId>>& two_sources);
    friend std::shared_ptr<OpGraph> transposes_cancelled(const OpGraph& g);
    friend std::shared_ptr<OpGraph> broadcasts_hoisted(const OpGraph& g);
};

// A copy of `g` in which values that are cheap to compute again are computed once per use instead of once: every
// pointwise / shape op whose value depends on at most one tensor of its own size (the rest being broadcasts of small
// tensors) is duplicated for each of its consumers, so that plan generation can fuse every copy into the kernel that
// uses it and the value never travels through memory. A batch norm's forward pass is the case in point: as recorded
// (batch_norm.rs:53-71) it leaves eight full-size intermediates for the backward pass to read - the broadcast scale,
// the broadcast reciprocal of the deviation, x minus the mean, ... - each a few instructions away from x and four
// per-channel vectors. Ops that compute the same thing are merged first (the reference's tape records a forward op again
// when the backward pass needs its value). A consumer that reads its operands from memory whatever happens (a product, a
// large permute, an Output) shares one copy. `keep_single`: nodes of `g` that are not to be duplicated. Node ids are new
// (in dataflow order); `origin` maps them back to `g`. Returns null when nothing changes.
// `two_sources`: sorted pairs of tensors (nodes of `g`) from which a value may be recomputed by every kernel that uses
// it, although a value that depends on two tensors of its size is otherwise written once and read back.
std::shared_ptr<OpGraph> rematerialized(const OpGraph& g, const std::set<NodeId>& keep_single = {},
                                        const std::set<std::vector<NodeId>>& two_sources = {});

// A copy of `g` without the transpositions that undo each other. The reference's front end writes a reduction over
// leading dims as SwapDims + Reduce and its gradient rules answer a SwapDims with a SwapDims (tensor.rs), so a recorded
// backward pass computes whole chains of pointwise ops on the transposed tensor and transposes the result back (batch
// norm: the statistics over N, H, W of an NHWC activation). Here a SwapDims is moved towards the producers of its
// operand - through pointwise ops (the same op on transposed operands), into broadcasts (whose axes are renamed) and
// constants - and is dropped when on every path it meets the SwapDims it undoes; the ops in between are then computed
// in the layout of the tensors in memory. A chain of SwapDims in front of a Reduce is replaced by the shortest chain that
// reduces the same dims (their order does not matter to a Sum / Mean / Min / Max beyond rounding). Node ids are new;
// `origin` names the node of `g` whose value, possibly transposed, a node computes. Returns null when nothing changes.
std::shared_ptr<OpGraph> transposes_cancelled(const OpGraph& g);

// A copy of `g` in which a pointwise op whose operands all are the same broadcast of small tensors (or constants) is
// applied to the small tensors, and its result broadcast: the front end writes `(variance.broadcast_to(x.shape) +
// 1e-3).sqrt()` (batch_norm.rs:56), a square root per element of x where one per channel does. Element by element the
// values are the same. Node ids are new; `origin` as above. Returns null when nothing changes.
std::shared_ptr<OpGraph> broadcasts_hoisted(const OpGraph& g);

// Subset of an OpGraph (opgraph/subgraph.rs): nodes sorted by id; `inputs` = outside producers feeding it,
// `roots` = members with an outside input, `leafs` = members with an outside consumer.
class OpSubgraph {
public:
    OpSubgraph() = default;
    OpSubgraph(std::shared_ptr<const OpGraph> g, std::vector<NodeId> nodes);
    OpSubgraph merge_with(const OpSubgraph& o) const;
    const std::shared_ptr<const OpGraph>& graph() const { return graph_; }
    const std::vector<NodeId>& nodes() const { return nodes_; }
    const std::vector<NodeId>& inputs() const { return inputs_; }
    const std::vector<NodeId>& roots() const { return roots_; }
    const std::vector<NodeId>& leafs() const { return leafs_; }
    bool contains(NodeId id) const { return std::binary_search(nodes_.begin(), nodes_.end(), id); }
    bool is_input(NodeId id) const { return std::find(inputs_.begin(), inputs_.end(), id) != inputs_.end(); }
    bool is_leaf(NodeId id) const { return std::find(leafs_.begin(), leafs_.end(), id) != leafs_.end(); }
    // Structural key used by the kernel caches (subgraph.rs:203-233): ops, descriptors and input descriptors.
    std::string cache_key() const;

private:
    std::shared_ptr<const OpGraph> graph_;
    std::vector<NodeId> nodes_, inputs_, roots_, leafs_;
};

}  // namespace he::ir
