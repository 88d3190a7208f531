#include "fusion_ir.h"

#include <set>

namespace he::fir {

std::vector<OpNode> Op::inputs() const {
    switch (kind) {
        case OpKind::Producer:
        case OpKind::Constant: return {};
        case OpKind::Matmul:
        case OpKind::BinaryPointwise: return {a, b};
        default: return {a};
    }
}

Shape3 OpGraph::shape_given_inputs(const Op& op, const OpGraph& g) {
    switch (op.kind) {
        case OpKind::Producer:
        case OpKind::Constant: return op.shape;
        case OpKind::Matmul: {
            const Shape3 &sa = g.shape(op.a), &sb = g.shape(op.b);
            HE_REQUIRE(sa[2] == sb[1], HE_ERR_INVALID, "matmul inner extents differ: %u vs %u", sa[2], sb[1]);
            HE_REQUIRE(sa[0] == sb[0], HE_ERR_INVALID, "matmul batch extents differ: %u vs %u", sa[0], sb[0]);
            return {sa[0], sa[1], sb[2]};
        }
        case OpKind::UnaryPointwise:
        case OpKind::Consumer: return g.shape(op.a);
        case OpKind::BinaryPointwise:
            HE_REQUIRE(g.shape(op.a) == g.shape(op.b), HE_ERR_INVALID, "binary pointwise operands differ in shape");
            return g.shape(op.a);
        case OpKind::Reduction: {
            Shape3 s = g.shape(op.a);
            switch (op.depth) {
                case ReductionDepth::Rows: s[2] = 1; break;
                case ReductionDepth::Columns: s[1] = 1; break;
                case ReductionDepth::Item: s[1] = s[2] = 1; break;
                case ReductionDepth::Batch: s[0] = s[1] = s[2] = 1; break;
            }
            return s;
        }
        case OpKind::Broadcast: {
            Shape3 s = g.shape(op.a);
            HE_REQUIRE(op.axis < 3, HE_ERR_INVALID, "broadcast axis %u out of range", op.axis);
            HE_REQUIRE(s[op.axis] == 1 || s[op.axis] == op.amount, HE_ERR_INVALID,
                       "broadcast of an axis of extent %u", s[op.axis]);
            s[op.axis] = op.amount;
            return s;
        }
        case OpKind::Transpose: {
            Shape3 s = g.shape(op.a);
            std::swap(s[1], s[2]);
            return s;
        }
    }
    fail(HE_ERR_INVALID, "bad fusion-IR op kind");
}

OpNode OpGraph::insert(const Op& op) { return insert_with_id(next_, op); }

OpNode OpGraph::insert_with_id(OpNode id, const Op& op) {
    HE_REQUIRE(!nodes_.count(id), HE_ERR_INVALID, "fusion-IR node %llu already exists", (unsigned long long)id);
    std::vector<OpNode> inputs = op.inputs();
    for (OpNode i : inputs)
        HE_REQUIRE(nodes_.count(i), HE_ERR_INVALID, "fusion-IR node %llu does not exist", (unsigned long long)i);
    Shape3 s = shape_given_inputs(op, *this);
    nodes_[id] = op;
    shapes_[id] = s;
    for (OpNode i : inputs) out_[i].push_back(id);
    if (inputs.empty()) roots_.push_back(id);
    in_[id] = inputs;
    out_[id];
    if (id >= next_) next_ = id + 1;
    return id;
}

OpGraph OpGraph::subgraph(const std::vector<OpNode>& nodes) const {
    std::set<OpNode> keep(nodes.begin(), nodes.end());
    OpGraph out;
    for (OpNode n : keep)
        for (OpNode dep : inbound(n)) {
            if (keep.count(dep) || out.has(dep)) continue;
            Op producer;
            producer.kind = OpKind::Producer;
            producer.shape = shape(dep);
            // what a kernel boundary stores: the declared type of a Producer, f32 for a reduction, bf16 otherwise
            const Op& src = get(dep);
            producer.dtype = src.kind == OpKind::Producer ? src.dtype : src.kind == OpKind::Reduction ? HE_F32 : HE_BF16;
            out.insert_with_id(dep, producer);
        }
    for (OpNode n : keep) out.insert_with_id(n, get(n));  // ids grow along every edge, so this order is topological
    OpNode fresh = next_;
    for (OpNode n : keep)
        for (OpNode user : outbound(n)) {
            if (keep.count(user)) continue;
            Op consumer;
            consumer.kind = OpKind::Consumer;
            consumer.a = n;
            consumer.dtype = get(n).kind == OpKind::Reduction ? HE_F32 : HE_BF16;
            // The reference files the Consumer under the reader's id even when that id is taken (a reader of two of
            // the nodes, or one that feeds the set again), which loses the earlier entry; an id beyond the graph's
            // keeps both.
            out.insert_with_id(out.has(user) ? fresh++ : user, consumer);
            break;
        }
    return out;
}

const Op& OpGraph::get(OpNode n) const {
    auto it = nodes_.find(n);
    HE_REQUIRE(it != nodes_.end(), HE_ERR_INVALID, "fusion-IR node %llu does not exist", (unsigned long long)n);
    return it->second;
}
const Shape3& OpGraph::shape(OpNode n) const {
    auto it = shapes_.find(n);
    HE_REQUIRE(it != shapes_.end(), HE_ERR_INVALID, "fusion-IR node %llu does not exist", (unsigned long long)n);
    return it->second;
}
std::vector<OpNode> OpGraph::nodes() const {
    std::vector<OpNode> v;
    for (auto& kv : nodes_) v.push_back(kv.first);
    return v;
}
std::vector<OpNode> OpGraph::leaves() const {
    std::vector<OpNode> v;
    for (auto& kv : nodes_)
        if (out_.at(kv.first).empty()) v.push_back(kv.first);
    return v;
}
const std::vector<OpNode>& OpGraph::inbound(OpNode n) const { return in_.at(n); }
const std::vector<OpNode>& OpGraph::outbound(OpNode n) const { return out_.at(n); }
OpNode OpGraph::anchor() const {
    for (auto& kv : nodes_)
        if (kv.second.is_anchor()) return kv.first;
    return kNoOpNode;
}

}  // namespace he::fir
