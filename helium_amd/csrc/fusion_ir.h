// The fusion IR of helium-playground (src/opgraph.rs): 3-d [batch, rows, cols] shapes and the op vocabulary the
// Core(mainloop, anchor, epilogue) / Aux fusions are written in. Kept as the reference defines it, plus a
// storage dtype per Producer / Consumer (the reference's generated kernels hard-code bf16).
#pragma once
#include <array>
#include <map>
#include <vector>

#include "common.h"

namespace he::fir {

using OpNode = uint64_t;
using Shape3 = std::array<uint32_t, 3>;

// opgraph.rs:264-301
enum class OpKind : int { Producer = 0, Constant, Matmul, UnaryPointwise, Reduction, BinaryPointwise, Broadcast,
                          Transpose, Consumer };
// opgraph.rs:317-328; AddConstant/MulConstant/PowConstant carry `constant`
enum class UnaryOp : int { Neg = 0, Relu, Gelu, Tanh, Exp, Ln, Sqrt, AddConstant, MulConstant, PowConstant };
// opgraph.rs:330-338
enum class BinaryOp : int { Add = 0, Sub, Mul, Div, Pow, Drelu };
// opgraph.rs:309-314
enum class ReductionDepth : int { Rows = 0, Columns, Item, Batch };

struct Op {
    OpKind kind = OpKind::Producer;
    Shape3 shape{1, 1, 1};  // Producer / Constant
    float value = 0;        // Constant
    OpNode a = 0, b = 0;    // Matmul a,b; Binary lhs,rhs; unary x in `a`
    int sub_op = 0;         // UnaryOp / BinaryOp
    float constant = 0;     // AddConstant / MulConstant / PowConstant
    ReductionDepth depth = ReductionDepth::Rows;
    uint32_t axis = 0, amount = 0;  // Broadcast
    int dtype = HE_BF16;            // Producer / Consumer storage type
    std::vector<OpNode> inputs() const;
    bool is_anchor() const { return kind == OpKind::Matmul; }
};

class OpGraph {
public:
    OpNode insert(const Op& op);  // opgraph.rs:33-57; node ids are assigned in insertion order
    // Inserts with a caller-chosen id (used to reproduce printed fusions with their original numbering).
    OpNode insert_with_id(OpNode id, const Op& op);
    const Op& get(OpNode n) const;
    const Shape3& shape(OpNode n) const;
    bool has(OpNode n) const { return nodes_.count(n) != 0; }
    std::vector<OpNode> nodes() const;
    std::vector<OpNode> roots() const { return roots_; }
    std::vector<OpNode> leaves() const;
    const std::vector<OpNode>& inbound(OpNode n) const;
    const std::vector<OpNode>& outbound(OpNode n) const;
    OpNode anchor() const;  // the Matmul node, or ~0 when there is none
    static Shape3 shape_given_inputs(const Op& op, const OpGraph& g);  // opgraph.rs:386-426
    // opgraph.rs:96-178: the given nodes with their ids kept; every value they read from outside becomes a
    // Producer under that value's id, and every node read from outside gets one Consumer, under the id of its first
    // outside reader.
    OpGraph subgraph(const std::vector<OpNode>& nodes) const;

private:
    std::map<OpNode, Op> nodes_;
    std::map<OpNode, Shape3> shapes_;
    std::map<OpNode, std::vector<OpNode>> in_, out_;
    std::vector<OpNode> roots_;
    OpNode next_ = 0;
};
constexpr OpNode kNoOpNode = ~0ull;

}  // namespace he::fir
