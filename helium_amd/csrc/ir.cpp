#include "ir.h"

#include <cstring>
#include <functional>
#include <map>
#include <set>
#include <sstream>
#include <unordered_map>

namespace he::ir {

int64_t num_elements(const Shape& s) {
    int64_t n = 1;
    for (int64_t d : s) n *= d;
    return n;
}

Shape packed_strides(const Shape& s) {
    Shape st(s.size(), 1);
    for (int i = (int)s.size() - 2; i >= 0; i--) st[i] = st[i + 1] * s[i + 1];
    return st;
}

int accumulator_type(Precision p) {
    switch (p) {
        case Precision::MulF16AccumF16:
        case Precision::MulF8AccumF16: return HE_F16;
        default: return HE_F32;
    }
}

bool ConvParams::operator==(const ConvParams& o) const {
    return in_channels == o.in_channels && out_channels == o.out_channels && kernel[0] == o.kernel[0] && kernel[1] == o.kernel[1] &&
           stride[0] == o.stride[0] && stride[1] == o.stride[1] && dilation[0] == o.dilation[0] && dilation[1] == o.dilation[1] &&
           padding_mode == o.padding_mode && input_size[0] == o.input_size[0] && input_size[1] == o.input_size[1];
}
void ConvParams::output_size(const int64_t in[2], const int64_t kernel_size[2], int64_t out[2]) const {
    for (int d = 0; d < 2; d++) {
        int64_t v = in[d];
        if (padding_mode == 2) v += kernel_size[d] / 2;
        else if (padding_mode == 1) v = std::max<int64_t>(0, v - kernel_size[d] / 2);
        out[d] = v / stride[d];
    }
}
void ConvParams::padding(int64_t pad[2]) const {
    for (int d = 0; d < 2; d++) pad[d] = padding_mode == 0 ? kernel[d] / 2 : padding_mode == 1 ? 0 : kernel[d] - 1;
}

bool Op::operator==(const Op& o) const {
    return conv == o.conv && kind == o.kind && inputs == o.inputs && sub_op == o.sub_op && precision == o.precision &&
           f8_modes == o.f8_modes && target_type == o.target_type && depth == o.depth &&
           new_dim_count == o.new_dim_count && broadcast_axes == o.broadcast_axes && shape == o.shape &&
           axis_a == o.axis_a && axis_b == o.axis_b && const_bits == o.const_bits && const_dtype == o.const_dtype;
}

uint64_t Op::hash() const {
    uint64_t h = fnv1a(&kind, sizeof kind);
    auto mix = [&](const void* p, size_t n) { h = fnv1a(p, n, h); };
    if (!inputs.empty()) mix(inputs.data(), inputs.size() * sizeof(NodeId));
    mix(&sub_op, sizeof sub_op);
    mix(&precision, sizeof precision);
    mix(&target_type, sizeof target_type);
    mix(&depth, sizeof depth);
    mix(&new_dim_count, sizeof new_dim_count);
    for (auto& a : broadcast_axes) mix(&a, sizeof a);
    if (!shape.empty()) mix(shape.data(), shape.size() * sizeof(int64_t));
    mix(&axis_a, sizeof axis_a);
    mix(&axis_b, sizeof axis_b);
    mix(&const_bits, sizeof const_bits);
    mix(&const_dtype, sizeof const_dtype);
    if (kind == OpKind::Conv || kind == OpKind::ConvBackwardData || kind == OpKind::ConvBackwardFilter) {
        const int64_t c[] = {conv.in_channels, conv.out_channels, conv.kernel[0], conv.kernel[1], conv.stride[0], conv.stride[1],
                             conv.dilation[0], conv.dilation[1], conv.padding_mode, conv.input_size[0], conv.input_size[1]};
        mix(c, sizeof c);
    }
    return h;
}

NodeId OpGraph::push(Node n) {
    nodes_.push_back(std::move(n));
    in_.emplace_back();
    out_.emplace_back();
    return (NodeId)(nodes_.size() - 1);
}

static void push_if_absent(std::vector<NodeId>& v, NodeId x) {
    if (std::find(v.begin(), v.end(), x) == v.end()) v.push_back(x);
}
static void remove_element(std::vector<NodeId>& v, NodeId x) {
    auto it = std::find(v.begin(), v.end(), x);
    if (it != v.end()) v.erase(it);
}

NodeId OpGraph::new_input(const Descriptor& d) {
    for (int64_t e : d.shape) HE_REQUIRE(e >= 0, HE_ERR_INVALID, "negative extent in input shape");
    Node n;
    n.kind = Node::Input;
    n.desc = d;
    NodeId id = push(std::move(n));
    inputs_.push_back(id);
    return id;
}

Shape OpGraph::broadcast_output_shape(const Op& op, const Shape& in) {
    // op.rs:376-390: left-pad with 1s up to new_dim_count, then overwrite every listed axis.
    Shape s = in;
    while ((int64_t)s.size() < op.new_dim_count) s.insert(s.begin(), 1);
    for (auto& a : op.broadcast_axes) {
        HE_REQUIRE(a.axis >= 0 && a.axis < (int64_t)s.size(), HE_ERR_INVALID, "broadcast axis %lld out of range",
                   (long long)a.axis);
        s[a.axis] = a.new_size;
    }
    return s;
}

Descriptor OpGraph::infer(const Op& op, const OpGraph& g) {
    auto in = [&](size_t i) -> const Descriptor& {
        HE_REQUIRE(i < op.inputs.size(), HE_ERR_INVALID, "op is missing input %zu", i);
        return g.get(op.inputs[i]).desc;
    };
    switch (op.kind) {
        case OpKind::ChangeDataType: return {in(0).shape, op.target_type};
        case OpKind::Matmul: {
            // op.rs:61-73: A's shape with the last extent replaced by B's last extent; accumulator dtype.
            Descriptor d{in(0).shape, accumulator_type(op.precision)};
            HE_REQUIRE(d.shape.size() >= 2 && in(1).shape.size() >= 2, HE_ERR_INVALID, "matmul needs rank >= 2");
            d.shape.back() = in(1).shape.back();
            return d;
        }
        case OpKind::UnaryPointwise:
        case OpKind::BinaryPointwise: return in(0);
        case OpKind::Reduce: {
            // op.rs:78-89: drop the last `depth` dims, append a single 1; always F32.
            Shape s = in(0).shape;
            HE_REQUIRE(op.depth >= 1 && op.depth <= s.size(), HE_ERR_INVALID, "reduce depth %u for rank %zu", op.depth,
                       s.size());
            s.resize(s.size() - op.depth + 1);
            s.back() = 1;
            return {s, HE_F32};
        }
        case OpKind::Reshape:
            HE_REQUIRE(num_elements(op.shape) == num_elements(in(0).shape), HE_ERR_INVALID,
                       "reshape changes the element count");
            return {op.shape, in(0).dtype};
        case OpKind::Broadcast: return {broadcast_output_shape(op, in(0).shape), in(0).dtype};
        case OpKind::SwapDims: {
            Shape s = in(0).shape;
            HE_REQUIRE(op.axis_a >= 0 && op.axis_b >= 0 && op.axis_a < (int64_t)s.size() && op.axis_b < (int64_t)s.size(),
                       HE_ERR_INVALID, "swap axis out of range");
            std::swap(s[op.axis_a], s[op.axis_b]);
            return {s, in(0).dtype};
        }
        case OpKind::Compare: return {in(0).shape, HE_BOOL};
        case OpKind::Select: return in(0);
        case OpKind::Constant: return {op.shape, op.const_dtype};
        case OpKind::Conv: {
            // op.rs:123-142: NHWC image, [out_channels, kh, kw, in_channels] filter; the image's dtype
            const Descriptor &image = in(0), &filter = in(1);
            HE_REQUIRE(image.shape.size() == 4 && filter.shape.size() == 4, HE_ERR_INVALID, "conv takes rank-4 image and filter");
            HE_REQUIRE(op.conv.in_channels > 0 && op.conv.out_channels > 0 && op.conv.kernel[0] > 0 && op.conv.kernel[1] > 0 &&
                           op.conv.stride[0] > 0 && op.conv.stride[1] > 0 && op.conv.dilation[0] > 0 && op.conv.dilation[1] > 0,
                       HE_ERR_INVALID, "conv parameters must be positive (Conv2dParams::validate)");
            const int64_t in_size[2] = {image.shape[1], image.shape[2]}, k_size[2] = {filter.shape[1], filter.shape[2]};
            int64_t out[2];
            op.conv.output_size(in_size, k_size, out);
            return {{image.shape[0], out[0], out[1], op.conv.out_channels}, image.dtype};
        }
        case OpKind::ConvBackwardData:  // op.rs:143-158
            return {{in(0).shape.at(0), op.conv.input_size[0], op.conv.input_size[1], op.conv.in_channels}, in(0).dtype};
        case OpKind::ConvBackwardFilter:  // op.rs:159-173
            return {{op.conv.out_channels, op.conv.kernel[0], op.conv.kernel[1], op.conv.in_channels}, in(0).dtype};
    }
    fail(HE_ERR_INVALID, "bad op kind");
}

NodeId OpGraph::new_op(Op op) {
    for (NodeId i : op.inputs) HE_REQUIRE(alive(i) && get(i).kind != Node::Output, HE_ERR_INVALID, "bad input node %u", i);
    Node n;
    n.kind = Node::Intermediate;
    n.desc = infer(op, *this);
    std::vector<NodeId> inputs = op.inputs;
    n.op = std::move(op);
    NodeId id = push(std::move(n));
    for (NodeId i : inputs) push_if_absent(out_[i], id);
    in_[id] = inputs;
    return id;
}

NodeId OpGraph::new_output(NodeId from) {
    HE_REQUIRE(alive(from), HE_ERR_INVALID, "bad node %u", from);
    Node n;
    n.kind = Node::Output;
    n.desc = get(from).desc;
    NodeId id = push(std::move(n));
    outputs_.push_back(id);
    in_[id] = {from};
    push_if_absent(out_[from], id);
    return id;
}

void OpGraph::remove(NodeId id) {
    HE_REQUIRE(alive(id), HE_ERR_INVALID, "bad node %u", id);
    for (NodeId p : in_[id]) remove_element(out_[p], id);
    for (NodeId s : out_[id]) remove_element(in_[s], id);
    in_[id].clear();
    out_[id].clear();
    remove_element(inputs_, id);
    remove_element(outputs_, id);
    nodes_[id] = Node{};
}

void OpGraph::optimize() {
    std::vector<char> visited(nodes_.size(), 0);
    std::vector<NodeId> stack = outputs_;
    while (!stack.empty()) {
        NodeId n = stack.back();
        stack.pop_back();
        visited[n] = 1;
        for (NodeId p : in_[n])
            if (!visited[p]) stack.push_back(p);
    }
    for (NodeId id = 0; id < nodes_.size(); id++)
        if (nodes_[id].kind != Node::Removed && !visited[id]) remove(id);
}

const Node& OpGraph::get(NodeId id) const {
    HE_REQUIRE(alive(id), HE_ERR_INVALID, "node %u does not exist", id);
    return nodes_[id];
}

std::vector<NodeId> OpGraph::nodes() const {
    std::vector<NodeId> v;
    for (NodeId id = 0; id < nodes_.size(); id++)
        if (nodes_[id].kind != Node::Removed) v.push_back(id);
    return v;
}

size_t OpGraph::num_nodes() const {
    size_t n = 0;
    for (auto& x : nodes_) n += x.kind != Node::Removed;
    return n;
}

bool OpGraph::feeds_output(NodeId id) const {
    for (NodeId s : out_[id])
        if (nodes_[s].kind == Node::Output) return true;
    return false;
}

uint64_t OpGraph::structural_hash() const {
    uint64_t h = 1469598103934665603ull;
    for (NodeId id = 0; id < nodes_.size(); id++) {
        const Node& n = nodes_[id];
        if (n.kind == Node::Removed) continue;
        h = fnv1a(&id, sizeof id, h);
        h = fnv1a(&n.kind, sizeof n.kind, h);
        h = fnv1a(&n.desc.dtype, sizeof n.desc.dtype, h);
        if (!n.desc.shape.empty()) h = fnv1a(n.desc.shape.data(), n.desc.shape.size() * 8, h);
        if (n.kind == Node::Intermediate) {
            uint64_t oh = n.op.hash();
            h = fnv1a(&oh, sizeof oh, h);
        }
    }
    return h;
}

bool OpGraph::structurally_equal(const OpGraph& o) const {
    // opgraph.rs:205-216: same nodes in the same slots with the same edges.
    if (nodes_.size() != o.nodes_.size()) return false;
    for (NodeId id = 0; id < nodes_.size(); id++) {
        const Node &a = nodes_[id], &b = o.nodes_[id];
        if (a.kind != b.kind) return false;
        if (a.kind == Node::Removed) continue;
        if (!(a.desc == b.desc)) return false;
        if (a.kind == Node::Intermediate && !(a.op == b.op)) return false;
        if (in_[id] != o.in_[id] || out_[id] != o.out_[id]) return false;
    }
    return true;
}

OpSubgraph::OpSubgraph(std::shared_ptr<const OpGraph> g, std::vector<NodeId> nodes) : graph_(std::move(g)) {
    std::sort(nodes.begin(), nodes.end());
    nodes.erase(std::unique(nodes.begin(), nodes.end()), nodes.end());
    nodes_ = std::move(nodes);
    for (NodeId n : nodes_) {
        HE_REQUIRE(graph_->alive(n) && graph_->get(n).kind == Node::Intermediate, HE_ERR_INVALID,
                   "subgraph node %u is not an intermediate node", n);
        bool root = false;
        for (NodeId i : graph_->inbound(n))
            if (!contains(i)) {
                push_if_absent(inputs_, i);
                root = true;
            }
        if (root) roots_.push_back(n);
        for (NodeId s : graph_->outbound(n))
            if (!contains(s)) {
                leafs_.push_back(n);
                break;
            }
    }
    std::sort(inputs_.begin(), inputs_.end());
}

OpSubgraph OpSubgraph::merge_with(const OpSubgraph& o) const {
    HE_REQUIRE(graph_ == o.graph_, HE_ERR_INVALID, "subgraphs of different graphs");
    std::vector<NodeId> n = nodes_;
    n.insert(n.end(), o.nodes_.begin(), o.nodes_.end());
    return OpSubgraph(graph_, std::move(n));
}

std::string OpSubgraph::cache_key() const {
    std::ostringstream s;
    for (NodeId n : nodes_) {
        const Node& node = graph_->get(n);
        s << n << ':' << node.op.hash() << ':' << node.desc.dtype << '[';
        for (int64_t d : node.desc.shape) s << d << ',';
        s << "];";
    }
    s << '|';
    for (NodeId n : inputs_) {
        const Node& node = graph_->get(n);
        s << n << ':' << node.desc.dtype << '[';
        for (int64_t d : node.desc.shape) s << d << ',';
        s << "];";
    }
    // which values leave the kernel depends on the consumers outside the node set
    s << "|L";
    for (NodeId n : leafs_) s << n << ',';
    return s.str();
}

}  // namespace he::ir

namespace he::ir {

std::shared_ptr<OpGraph> rematerialized(const OpGraph& g, const std::set<NodeId>& keep_single,
                                        const std::set<std::vector<NodeId>>& two_sources) {
    const size_t cap = g.capacity();
    // 1. Ops that compute the same thing are one op. The reference's tape records a forward op again when the backward
    //    pass needs its value (tensor/tape.rs:93-158 recomputes from the last checkpoint), so every batch norm's
    //    normalisation chain is in the graph twice.
    std::vector<NodeId> canon(cap, kNoNode);
    {
        std::unordered_map<uint64_t, std::vector<NodeId>> seen;
        for (NodeId id : g.nodes()) {
            const Node& n = g.get(id);
            canon[id] = id;
            if (n.kind != Node::Intermediate) continue;
            Op op = n.op;
            for (NodeId& in : op.inputs) in = canon[in];
            auto& bucket = seen[op.hash()];
            for (NodeId other : bucket) {
                Op theirs = g.get(other).op;
                for (NodeId& in : theirs.inputs) in = canon[in];
                if (theirs == op && g.get(other).desc == n.desc) {
                    canon[id] = other;
                    break;
                }
            }
            if (canon[id] == id) bucket.push_back(id);
        }
    }
    std::vector<std::vector<NodeId>> users(cap);  // consumers of a canonical node, themselves canonical
    bool merged_any = false;
    for (NodeId id : g.nodes()) {
        if (canon[id] != id) {
            merged_any = true;
            continue;
        }
        for (NodeId in : g.inbound(id)) users[canon[in]].push_back(id);
    }

    // 2. What a node's value depends on once the cheap ops in between are looked through: the tensors that exist in
    //    memory anyway (`anchors`: inputs, products, reductions, permutes - listed only when they are not small next to
    //    the node), and how many ops a recomputation takes.
    struct Info {
        bool cheap = false;          // an op that may be duplicated
        bool remat = false;          // ... and is, once per use by a kernel that can take it in
        bool remat_for_reduction = false;  // ... or at least once per use by a kernel that only reduces it
        int cost = 0;
        std::vector<NodeId> anchors; // sorted, at most kMaxAnchors + 1 entries
    };
    constexpr int kMaxCost = 64, kMaxCopies = 1024;
    constexpr int64_t kMinElements = 1 << 16;
    constexpr size_t kMaxAnchors = 1;
    std::vector<Info> info(cap);
    bool any = false;
    for (NodeId id : g.nodes()) {
        if (canon[id] != id) continue;
        const Node& n = g.get(id);
        Info& I = info[id];
        if (n.kind != Node::Intermediate) continue;
        switch (n.op.kind) {
            case OpKind::UnaryPointwise:
            case OpKind::BinaryPointwise:
            case OpKind::ChangeDataType:
            case OpKind::Broadcast:
            case OpKind::Reshape:
            case OpKind::Compare:
            case OpKind::Select:
            case OpKind::Constant: I.cheap = true; break;
            default: break;
        }
        if (!I.cheap) continue;
        const int64_t numel = num_elements(n.desc.shape);
        I.cost = 1;
        for (NodeId raw : n.op.inputs) {
            const NodeId in = canon[raw];
            const Info& J = info[in];
            // (a cheap op that is not copied exists once, in memory like a product: its consumers start from it)
            if (J.cheap && (J.remat || num_elements(g.get(in).desc.shape) < kMinElements)) {
                I.cost += J.cost;
                for (NodeId a : J.anchors) I.anchors.push_back(a);
            } else if (num_elements(g.get(in).desc.shape) * 8 >= numel) {
                I.anchors.push_back(in);
            }
        }
        std::sort(I.anchors.begin(), I.anchors.end());
        I.anchors.erase(std::unique(I.anchors.begin(), I.anchors.end()), I.anchors.end());
        // a tensor that is small next to this node may still have been an anchor of an input: keep what is not small
        std::vector<NodeId> kept;
        for (NodeId a : I.anchors)
            if (num_elements(g.get(a).desc.shape) * 8 >= numel) kept.push_back(a);
        I.anchors = kept;
        if (I.anchors.size() > kMaxAnchors + 2) I.anchors.resize(kMaxAnchors + 2);
        I.cost = std::min(I.cost, kMaxCost + 1);
        // (a node with one consumer is copied as well when that consumer is: its copies' inputs must not meet in one
        // shared node, which would then have several consumers and travel through memory after all)
        I.remat = numel >= kMinElements && (I.anchors.size() <= kMaxAnchors || (I.anchors.size() == 2 && two_sources.count(I.anchors))) &&
                  I.cost <= kMaxCost && !keep_single.count(id);
        // A value that only reductions read (through transpositions and pointwise ops) may depend on one tensor more:
        // written out and read back it moves as many bytes as its two operands do, and the reductions of one backward
        // pass (a batch norm's four) then share one pass over those operands instead of reading a tensor each.
        I.remat_for_reduction = numel >= kMinElements && I.anchors.size() <= kMaxAnchors + 1 && I.cost <= kMaxCost && !keep_single.count(id);
        any = any || (I.remat && users[id].size() > 1) || (I.remat_for_reduction && !I.remat);
    }
    if (!any && !merged_any) return nullptr;
    // nodes whose value ends in reductions only (a SwapDims and pointwise ops may lie in between)
    std::vector<char> reduced_only(cap, 0);
    {
        std::vector<NodeId> order = g.nodes();
        for (auto it = order.rbegin(); it != order.rend(); ++it) {
            const NodeId id = *it;
            if (canon[id] != id || g.get(id).kind != Node::Intermediate) continue;
            if (g.get(id).op.kind == OpKind::Reduce) {
                reduced_only[id] = 1;
                continue;
            }
            if (!info[id].cheap && g.get(id).op.kind != OpKind::SwapDims) continue;
            bool all = !users[id].empty();
            for (NodeId u : users[id]) all = all && reduced_only[u];
            reduced_only[id] = all;
        }
    }

    auto out = std::make_shared<OpGraph>();
    std::vector<NodeId> placed(cap, kNoNode);  // node of `g` -> its one node in `out` (what is not duplicated)
    std::vector<int> copies(cap, 0);
    auto note_origin = [&](NodeId fresh, NodeId old) {
        if (out->origin_.size() <= fresh) out->origin_.resize(fresh + 1, kNoNode);
        out->origin_[fresh] = old;
    };
    // A kernel that cannot take a producer in (a product reads operands from memory, so does a permute, and an Output is
    // memory) reads the one shared copy; every other consumer gets a copy of its own.
    auto takes_producers_in = [&](const Node& consumer) {
        if (consumer.kind != Node::Intermediate) return false;
        switch (consumer.op.kind) {
            case OpKind::Matmul:
            case OpKind::Conv:
            case OpKind::ConvBackwardData:
            case OpKind::ConvBackwardFilter: return false;
            case OpKind::SwapDims: return num_elements(consumer.desc.shape) <= 1000000;
            default: return true;
        }
    };
    // for_fusing_consumer: 0 a consumer that reads from memory, 1 one that can compute the value itself, 2 one that does
    // and ends in reductions only
    // A value that a product, a permute or the caller reads is written to memory whatever happens: a reduction that could
    // recompute it from two tensors of its size reads the one tensor instead (the input gradient of a batch norm goes on
    // to a convolution's gradients and, through the residual connection, into the next batch norm's sums: those sums read
    // 2 tensors per element instead of 3, and the training step's plan moves 12.5 GB instead of 13.4).
    std::vector<char> written_anyway(cap, 0);
    for (NodeId id : g.nodes()) {
        if (canon[id] != id) continue;
        for (NodeId u : users[id]) written_anyway[id] = written_anyway[id] || (!takes_producers_in(g.get(u)) && !(g.get(u).kind == Node::Intermediate && reduced_only[canon[u]]));
    }
    std::function<NodeId(NodeId, int)> emit = [&](NodeId raw, int for_fusing_consumer) -> NodeId {
        const NodeId id = canon[raw];
        const Node& n = g.get(id);
        const bool for_reduction = for_fusing_consumer == 2 && info[id].remat_for_reduction && !written_anyway[id];
        const bool dup = (info[id].remat || for_reduction) && for_fusing_consumer && copies[id] < kMaxCopies;
        if (!dup && placed[id] != kNoNode) return placed[id];
        NodeId fresh;
        if (n.kind == Node::Input) {
            fresh = out->new_input(n.desc);
        } else {
            Op op = n.op;
            // (a large SwapDims is a permute, which reads from memory, unless only reductions read it: then it is part
            // of their kernel)
            const int fusing = reduced_only[id] && (info[id].cheap || n.op.kind == OpKind::SwapDims) ? 2 : takes_producers_in(n) ? 1 : 0;
            for (NodeId& in : op.inputs) in = emit(in, fusing);
            fresh = out->new_op(std::move(op));
        }
        note_origin(fresh, id);
        if (dup) {
            copies[id]++;
            if (out->for_consumer_.size() <= fresh) out->for_consumer_.resize(fresh + 1, 0);
            out->for_consumer_[fresh] = 1;
        } else {
            placed[id] = fresh;
        }
        return fresh;
    };
    // inputs first, in their own order
    for (NodeId id : g.inputs()) emit(id, 0);
    for (NodeId id : g.nodes()) {
        const Node& n = g.get(id);
        if (n.kind == Node::Output) {
            NodeId fresh = out->new_output(emit(g.inbound(id)[0], 0));
            note_origin(fresh, id);
        } else if (n.kind == Node::Intermediate && canon[id] == id && !info[id].remat) {
            emit(id, 0);
        }
    }
    out->optimize();
    return out;
}

// ---------------------------------------------------------------------------------------------------------
// Transpositions that cancel
// ---------------------------------------------------------------------------------------------------------
namespace {
using Perm = std::vector<int>;  // transposed.shape[i] = source.shape[perm[i]]

bool is_identity(const Perm& p) {
    for (size_t i = 0; i < p.size(); i++)
        if (p[i] != (int)i) return false;
    return true;
}
// transposing by `first`, then by `second`
Perm compose(const Perm& first, const Perm& second) {
    Perm out(second.size());
    for (size_t i = 0; i < second.size(); i++) out[i] = first[second[i]];
    return out;
}
Perm swap_perm(size_t rank, int64_t a, int64_t b) {
    Perm p(rank);
    for (size_t i = 0; i < rank; i++) p[i] = (int)i;
    std::swap(p[a], p[b]);
    return p;
}
// swaps (applied in order) that turn the identity into `p`
std::vector<std::pair<int, int>> swaps_for(const Perm& p) {
    std::vector<std::pair<int, int>> out;
    Perm cur(p.size());
    for (size_t i = 0; i < p.size(); i++) cur[i] = (int)i;
    for (size_t i = 0; i < p.size(); i++) {
        if (cur[i] == p[i]) continue;
        size_t j = i + 1;
        while (cur[j] != p[i]) j++;
        out.push_back({(int)i, (int)j});
        std::swap(cur[i], cur[j]);
    }
    return out;
}
}  // namespace

std::shared_ptr<OpGraph> transposes_cancelled(const OpGraph& g) {
    const size_t cap = g.capacity();
    constexpr int kStop = 1000;  // a transposition that would have to stay, somewhere further up
    // What is left of a transposition by `p` of `node`'s value once it has been moved towards the producers: 0 when it
    // disappears (it meets its inverse, a broadcast, or a constant on every path), the number of transpositions
    // that remain otherwise.
    std::map<std::pair<NodeId, Perm>, int> left_memo;
    std::function<int(NodeId, const Perm&)> left = [&](NodeId node, const Perm& p) -> int {
        if (is_identity(p)) return 0;
        auto key = std::make_pair(node, p);
        auto it = left_memo.find(key);
        if (it != left_memo.end()) return it->second;
        left_memo[key] = kStop;  // (no cycles in a graph; the entry is overwritten below)
        const Node& n = g.get(node);
        int cost = kStop;
        if (n.kind == Node::Intermediate && n.desc.shape.size() == p.size()) {
            switch (n.op.kind) {
                case OpKind::SwapDims: cost = left(n.op.inputs[0], compose(swap_perm(p.size(), n.op.axis_a, n.op.axis_b), p)); break;
                case OpKind::UnaryPointwise:
                case OpKind::ChangeDataType:
                case OpKind::BinaryPointwise:
                case OpKind::Compare:
                case OpKind::Select: {
                    cost = 0;
                    for (NodeId in : n.op.inputs) {
                        if (g.get(in).desc.shape != g.get(n.op.inputs[0]).desc.shape) cost = kStop;
                        cost = std::min(kStop, cost + left(in, p));
                    }
                    break;
                }
                case OpKind::Constant: cost = 0; break;
                case OpKind::Broadcast: {
                    // the listed axes must be extents of 1 in the source, and the source small next to the result
                    Shape padded = g.get(n.op.inputs[0]).desc.shape;
                    while ((int64_t)padded.size() < n.op.new_dim_count) padded.insert(padded.begin(), 1);
                    bool plain = padded.size() == p.size() && num_elements(padded) * 8 <= num_elements(n.desc.shape);
                    for (auto& a : n.op.broadcast_axes) plain = plain && padded[a.axis] == 1;
                    if (plain) cost = 0;
                    break;
                }
                default: break;
            }
        }
        left_memo[key] = cost;
        return cost;
    };

    auto out = std::make_shared<OpGraph>();
    std::vector<NodeId> placed(cap, kNoNode);
    auto note_origin = [&](NodeId fresh, NodeId old) {
        if (out->origin_.size() <= fresh) out->origin_.resize(fresh + 1, kNoNode);
        out->origin_[fresh] = old;
    };
    auto swapped = [&](NodeId fresh, const Perm& p, NodeId origin) {
        for (auto [a, b] : swaps_for(p)) {
            Op op;
            op.kind = OpKind::SwapDims;
            op.inputs = {fresh};
            op.axis_a = a;
            op.axis_b = b;
            fresh = out->new_op(std::move(op));
            note_origin(fresh, origin);
        }
        return fresh;
    };
    bool changed = false;
    // `node`'s value transposed by `p`, as a node of `out`. `recorded`: a SwapDims of `g` that SwapDims nodes made here
    // stand for (an origin has to be a node that only moves data: whoever evaluates the plan on `g` reads such nodes
    // through, and would otherwise recompute a value that the plan keeps in memory).
    std::map<std::pair<NodeId, Perm>, NodeId> built;
    std::function<NodeId(NodeId, const Perm&, NodeId)> build = [&](NodeId node, const Perm& p, NodeId recorded) -> NodeId {
        if (is_identity(p)) return placed[node];
        auto key = std::make_pair(node, p);
        auto it = built.find(key);
        if (it != built.end()) return it->second;
        const Node& n = g.get(node);
        NodeId fresh = kNoNode;
        if (left(node, p) != 0) {
            fresh = swapped(placed[node], p, recorded);
        } else {
            switch (n.op.kind) {
                case OpKind::SwapDims: fresh = build(n.op.inputs[0], compose(swap_perm(p.size(), n.op.axis_a, n.op.axis_b), p), recorded); break;
                case OpKind::Constant: {
                    Op op = n.op;
                    for (size_t i = 0; i < p.size(); i++) op.shape[i] = n.op.shape[p[i]];
                    fresh = out->new_op(std::move(op));
                    note_origin(fresh, node);
                    break;
                }
                case OpKind::Broadcast: {
                    const Shape& src = g.get(n.op.inputs[0]).desc.shape;
                    Shape padded = src;
                    while (padded.size() < p.size()) padded.insert(padded.begin(), 1);
                    Shape moved(p.size());
                    for (size_t i = 0; i < p.size(); i++) moved[i] = padded[p[i]];
                    // extents of 1 do not count: when the others keep their order the source is only given a new shape
                    std::vector<int64_t> before, after;
                    for (size_t i = 0; i < p.size(); i++) {
                        if (padded[i] != 1) before.push_back((int64_t)i);
                        if (moved[i] != 1) after.push_back(p[i]);
                    }
                    // (the nodes that bring the small source into shape stand for no node of `g`: the broadcast as recorded
                    // reads the recorded source)
                    NodeId source = placed[n.op.inputs[0]];
                    if (before == after) {
                        if (moved != src) {
                            Op r;
                            r.kind = OpKind::Reshape;
                            r.inputs = {source};
                            r.shape = moved;
                            source = out->new_op(std::move(r));
                            note_origin(source, kNoNode);
                        }
                    } else {
                        if (padded != src) {
                            Op r;
                            r.kind = OpKind::Reshape;
                            r.inputs = {source};
                            r.shape = padded;
                            source = out->new_op(std::move(r));
                            note_origin(source, kNoNode);
                        }
                        source = swapped(source, p, kNoNode);
                    }
                    Op op = n.op;
                    op.inputs = {source};
                    op.new_dim_count = (int64_t)p.size();
                    for (auto& a : op.broadcast_axes)
                        for (size_t i = 0; i < p.size(); i++)
                            if (p[i] == a.axis) {
                                a.axis = (int64_t)i;
                                break;
                            }
                    std::sort(op.broadcast_axes.begin(), op.broadcast_axes.end(), [](const BroadcastAxis& x, const BroadcastAxis& y) { return x.axis < y.axis; });
                    fresh = out->new_op(std::move(op));
                    note_origin(fresh, node);
                    break;
                }
                default: {  // pointwise: the same op on transposed operands
                    Op op = n.op;
                    for (NodeId& in : op.inputs) in = build(in, p, recorded);
                    fresh = out->new_op(std::move(op));
                    note_origin(fresh, node);
                    break;
                }
            }
        }
        built[key] = fresh;
        return fresh;
    };

    for (NodeId id : g.inputs()) {
        placed[id] = out->new_input(g.get(id).desc);
        note_origin(placed[id], id);
    }
    for (NodeId id : g.nodes()) {
        const Node& n = g.get(id);
        if (n.kind == Node::Input) continue;
        if (n.kind == Node::Output) {
            placed[id] = out->new_output(placed[g.inbound(id)[0]]);
            note_origin(placed[id], id);
            continue;
        }
        const size_t rank = n.op.inputs.empty() ? 0 : g.get(n.op.inputs[0]).desc.shape.size();
        if (n.op.kind == OpKind::SwapDims) {
            const Perm p = swap_perm(rank, n.op.axis_a, n.op.axis_b);
            if (left(n.op.inputs[0], p) == 0) {
                placed[id] = build(n.op.inputs[0], p, id);
                changed = true;
                continue;
            }
        }
        if (n.op.kind == OpKind::Reduce && g.get(n.op.inputs[0]).kind == Node::Intermediate && g.get(n.op.inputs[0]).op.kind == OpKind::SwapDims) {
            // The reduced dims may come in any order. Of all transpositions that put the kept dims first, in their
            // order, the one with the fewest swaps is taken: a chain of swaps (the gradient of a broadcast is recorded as
            // one, tensor.rs) becomes the single swap that the pointwise kernel folds into its walk over the tensor.
            NodeId base = n.op.inputs[0];
            Perm p(rank);
            for (size_t i = 0; i < rank; i++) p[i] = (int)i;
            size_t chain = 0;
            while (g.get(base).kind == Node::Intermediate && g.get(base).op.kind == OpKind::SwapDims) {
                const Op& s = g.get(base).op;
                p = compose(swap_perm(rank, s.axis_a, s.axis_b), p);
                base = s.inputs[0];
                chain++;
            }
            const size_t kept = rank - n.op.depth;
            Perm q(rank, -1);
            std::vector<bool> used(rank, false);
            for (size_t i = 0; i < kept; i++) {
                q[i] = p[i];
                used[p[i]] = true;
            }
            for (size_t j = kept; j < rank; j++)  // a reduced dim that can stay where it is
                if (!used[j]) {
                    q[j] = (int)j;
                    used[j] = true;
                }
            for (size_t j = kept; j < rank; j++) {
                if (q[j] >= 0) continue;
                // dim j is kept, at position i: dim i coming here closes a cycle of two
                size_t i = 0;
                while (q[i] != (int)j) i++;
                size_t pick = !used[i] ? i : rank;
                for (size_t d = 0; d < rank && pick == rank; d++)
                    if (!used[d]) pick = d;
                q[j] = (int)pick;
                used[pick] = true;
            }
            if (swaps_for(q).size() < chain) {
                Op op = n.op;
                op.inputs = {build(base, q, n.op.inputs[0])};
                const NodeId fresh = out->new_op(std::move(op));
                if (out->get(fresh).desc == n.desc) {
                    placed[id] = fresh;
                    note_origin(fresh, id);
                    changed = true;
                    continue;
                }
                // (a reduction that did not keep its shape is left in place, unused, and pruned below)
            }
        }
        Op op = n.op;
        for (NodeId& in : op.inputs) in = placed[in];
        placed[id] = out->new_op(std::move(op));
        note_origin(placed[id], id);
    }
    if (!changed) return nullptr;
    out->optimize();
    return out;
}

std::shared_ptr<OpGraph> broadcasts_hoisted(const OpGraph& g) {
    const size_t cap = g.capacity();
    auto out = std::make_shared<OpGraph>();
    std::vector<NodeId> placed(cap, kNoNode);
    auto note_origin = [&](NodeId fresh, NodeId old) {
        if (out->origin_.size() <= fresh) out->origin_.resize(fresh + 1, kNoNode);
        out->origin_[fresh] = old;
    };
    // a Broadcast of `out` that only repeats its source: the source's extents at the listed axes are 1
    auto plain_broadcast = [&](NodeId id, Shape* padded) {
        const Node& n = out->get(id);
        if (n.kind != Node::Intermediate || n.op.kind != OpKind::Broadcast) return false;
        *padded = out->get(n.op.inputs[0]).desc.shape;
        while ((int64_t)padded->size() < n.op.new_dim_count) padded->insert(padded->begin(), 1);
        for (auto& a : n.op.broadcast_axes)
            if ((*padded)[a.axis] != 1) return false;
        return num_elements(*padded) < num_elements(n.desc.shape);
    };
    bool changed = false;
    for (NodeId id : g.inputs()) {
        placed[id] = out->new_input(g.get(id).desc);
        note_origin(placed[id], id);
    }
    for (NodeId id : g.nodes()) {
        const Node& n = g.get(id);
        if (n.kind == Node::Input) continue;
        if (n.kind == Node::Output) {
            placed[id] = out->new_output(placed[g.inbound(id)[0]]);
            note_origin(placed[id], id);
            continue;
        }
        Op op = n.op;
        for (NodeId& in : op.inputs) in = placed[in];
        bool pointwise = false;
        switch (op.kind) {
            case OpKind::UnaryPointwise:
            case OpKind::BinaryPointwise:
            case OpKind::ChangeDataType:
            case OpKind::Compare:
            case OpKind::Select: pointwise = true; break;
            default: break;
        }
        // A reduction of a broadcast along reduced dims only: the repeated terms need not be walked. Sum: the small
        // tensor's sum times the number of repeats; Mean, Max, Min: the small tensor's.
        if (op.kind == OpKind::Reduce) {
            Shape padded;
            const Shape full_in = out->get(op.inputs[0]).desc.shape;
            if (plain_broadcast(op.inputs[0], &padded) && padded.size() == full_in.size() && op.depth <= padded.size()) {
                const Op broadcast = out->get(op.inputs[0]).op;
                bool inside = true;
                double repeats = 1;
                for (auto& a : broadcast.broadcast_axes) {
                    inside = inside && (size_t)a.axis >= padded.size() - op.depth;
                    repeats *= (double)full_in[a.axis];
                }
                if (inside && repeats > 1) {
                    NodeId small_in = broadcast.inputs[0];
                    if (out->get(small_in).desc.shape != padded) {
                        Op r;
                        r.kind = OpKind::Reshape;
                        r.inputs = {small_in};
                        r.shape = padded;
                        small_in = out->new_op(std::move(r));
                        note_origin(small_in, kNoNode);
                    }
                    Op red = op;
                    red.inputs = {small_in};
                    NodeId result = out->new_op(std::move(red));
                    if (out->get(result).desc == n.desc) {
                        if ((ReduceOp)op.sub_op == ReduceOp::Sum) {
                            note_origin(result, kNoNode);
                            Op c;
                            c.kind = OpKind::Constant;
                            c.shape = n.desc.shape;
                            c.const_dtype = HE_F32;
                            const float f = (float)repeats;
                            memcpy(&c.const_bits, &f, 4);
                            const NodeId factor = out->new_op(std::move(c));
                            note_origin(factor, kNoNode);
                            Op mul;
                            mul.kind = OpKind::BinaryPointwise;
                            mul.sub_op = (int)BinaryOp::Mul;
                            mul.inputs = {result, factor};
                            result = out->new_op(std::move(mul));
                        }
                        placed[id] = result;
                        note_origin(result, id);
                        changed = true;
                        continue;
                    }
                }
            }
        }
        // Every operand a broadcast of a small tensor (or a constant): the op is applied to the small tensors, brought
        // to the smallest shape that holds them all ([C] and [1] meet in [C]), and its result is broadcast.
        const Shape& full = n.desc.shape;
        Shape small(full.size(), 1);
        std::vector<Shape> padded(op.inputs.size());
        bool hoist = pointwise, any_broadcast = false;
        for (size_t i = 0; i < op.inputs.size() && hoist; i++) {
            const Node& in = out->get(op.inputs[i]);
            if (in.kind == Node::Intermediate && in.op.kind == OpKind::Constant) continue;
            if (!plain_broadcast(op.inputs[i], &padded[i]) || padded[i].size() != full.size()) {
                hoist = false;
                break;
            }
            any_broadcast = true;
            for (size_t d = 0; d < full.size(); d++) small[d] = std::max(small[d], padded[i][d]);
        }
        if (hoist && any_broadcast && num_elements(small) * 8 <= num_elements(full)) {
            Op inner = op;
            for (size_t i = 0; i < inner.inputs.size(); i++) {
                NodeId& in = inner.inputs[i];
                const Node src = out->get(in);  // (a copy: new nodes move the node table)
                // (the constants, reshapes and small broadcasts made here stand for no node of `g`)
                if (src.op.kind == OpKind::Constant) {
                    Op c = src.op;
                    c.shape = small;
                    in = out->new_op(std::move(c));
                    note_origin(in, kNoNode);
                    continue;
                }
                in = src.op.inputs[0];
                if (out->get(in).desc.shape != padded[i]) {
                    Op r;
                    r.kind = OpKind::Reshape;
                    r.inputs = {in};
                    r.shape = padded[i];
                    in = out->new_op(std::move(r));
                    note_origin(in, kNoNode);
                }
                if (padded[i] != small) {
                    Op b;
                    b.kind = OpKind::Broadcast;
                    b.inputs = {in};
                    b.new_dim_count = (int64_t)small.size();
                    for (size_t d = 0; d < small.size(); d++)
                        if (padded[i][d] == 1 && small[d] != 1) b.broadcast_axes.push_back({(int64_t)d, small[d]});
                    in = out->new_op(std::move(b));
                    note_origin(in, kNoNode);
                }
            }
            const NodeId computed = out->new_op(std::move(inner));
            note_origin(computed, id);
            Op again;
            again.kind = OpKind::Broadcast;
            again.inputs = {computed};
            again.new_dim_count = (int64_t)full.size();
            for (size_t d = 0; d < full.size(); d++)
                if (small[d] == 1 && full[d] != 1) again.broadcast_axes.push_back({(int64_t)d, full[d]});
            placed[id] = out->new_op(std::move(again));
            // (the broadcast stands for no node of `g`: whoever evaluates the plan on `g` reads `id` from memory there)
            note_origin(placed[id], kNoNode);
            if (out->get(placed[id]).desc == n.desc) {
                changed = true;
                continue;
            }
        }
        placed[id] = out->new_op(std::move(op));
        note_origin(placed[id], id);
    }
    if (!changed) return nullptr;
    out->optimize();
    return out;
}

void OpGraph::rebase_origins(const OpGraph& through) {
    for (NodeId& o : origin_)
        if (o != kNoNode) o = through.origin(o);
}


}  // namespace he::ir
