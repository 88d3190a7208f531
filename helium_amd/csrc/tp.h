// Tile program: the kernel-level form both front-end IRs are lowered to before HIP source is emitted.
//
// A program evaluates a DAG of scalar expressions at every coordinate of an N-d iteration space and writes
// full-size outputs and/or reductions of them. The same expression emitter serves the pointwise/reduction
// instruction (helium/src/cuda/instr/pointwise/jit.rs), the anchor-less "auxiliary" fusions and the epilogue of
// the fused GEMM (helium-playground/src/kernel_generator.rs), which differ only in the loop that drives it.
#pragma once
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "common.h"
#include "fusion_ir.h"
#include "ir.h"

namespace he::tp {

using ir::Shape;

enum class Cls : int { F = 0, I = 1, B = 2 };  // f32 math, uint32 math, bool (jit.rs:917-925)
enum class UOp : int { Recip = 0, Neg, Exp, Sin, Cos, Tan, Sigmoid, Tanh, Relu, Sqrt, Log, Gelu, AddC, MulC, PowC };
enum class BOp : int { Add = 0, Sub, Mul, Div, Pow, Min, Max, And, Or, Xor, Drelu };
enum class COp : int { Eq = 0, Ne, Lt, Le, Gt, Ge };
enum class ROp : int { Sum = 0, Mean, Max, Min };

// One reference-style index map (jit.rs:802-915), kept for the rare accesses that are not affine in the
// iteration coordinates (a Reshape between two index-changing ops).
struct GenericMap {
    enum Kind { Swap, Bcast } kind = Swap;
    Shape in_shape;                 // shape of the op's input
    int64_t axis_a = 0, axis_b = 0; // Swap
    Shape out_shape;                // Bcast: shape of the op's output
    std::vector<char> bcast;        // Bcast: per output dim, 1 when the coordinate is forced to 0
    bool operator==(const GenericMap& o) const {
        return kind == o.kind && in_shape == o.in_shape && axis_a == o.axis_a && axis_b == o.axis_b &&
               out_shape == o.out_shape && bcast == o.bcast;
    }
};

struct Access {
    int arg = -1;
    int dtype = HE_F32;
    std::vector<int64_t> stride;    // per iteration dim; linear index = sum coord[d] * stride[d]
    std::vector<GenericMap> chain;  // then these maps, in order
};

struct Expr {
    enum Kind { Load, Acc, Const, Unary, Binary, Compare, Select, Cast } kind = Const;
    Cls cls = Cls::F;
    int a = -1, b = -1, c = -1;  // operand expression ids (Select: a=lhs, b=rhs, c=selector)
    int op = 0;                  // UOp / BOp / COp
    uint32_t bits = 0;           // Const: f32 / u32 / bool bit pattern; Unary *C ops: f32 bits of the constant
    Access access;               // Load
};

struct Out {
    int expr = -1;
    int arg = -1;
    int dtype = HE_F32;
    bool reduce = false;
    ROp rop = ROp::Sum;
    // Which parts of the canonical [B.., M, N] space the reduction folds. `b_div` folds the trailing part of the
    // flattened B index: the output's leading index is b / b_div.
    bool fold_n = false, fold_m = false;
    int64_t b_div = 1;
    double mean_scale = 1.0;  // Mean multiplies every term by this (as a double, jit.rs:599-604)
    // A full-size output that is not stored in iteration order: per iteration dim, the stride of its coordinate in the
    // output (an untransposed tensor written by a kernel that iterates in the index space of its reductions). Empty:
    // element i of the iteration space is element i of the output.
    std::vector<int64_t> stride;
};

struct Arg {
    int dtype = HE_F32;
    int64_t numel = 0;
    bool is_output = false;
    uint64_t node = 0;  // front-end node id the argument stands for
};

struct Program {
    Shape dims;  // iteration space, row-major; last = N, second to last = M, the rest flatten to B
    std::vector<Expr> exprs;  // topologically ordered
    std::vector<Out> outs;
    std::vector<Arg> args;
    bool fast_math = false;   // GEMM epilogues use the fast intrinsics (helium-kernel-generator/src/pointwise.rs:53-98)
    int acc_expr = -1;        // id of the Acc expression when the program is a GEMM epilogue
    // A second, small program over [columns] that the launch which folds this program's column reductions evaluates once
    // per column (the per-channel arithmetic behind a batch norm's sums, which would otherwise be a launch of its own):
    // its Loads of arguments that are column reductions of this program read the folded values, everything else comes
    // from memory. Its argument indices refer to this program's `args`. Set by attach_post.
    std::shared_ptr<const Program> post;

    int64_t N() const { return dims.empty() ? 1 : dims.back(); }
    int64_t M() const { return dims.size() >= 2 ? dims[dims.size() - 2] : 1; }
    int64_t B() const {
        int64_t b = 1;
        for (size_t i = 0; i + 2 < dims.size(); i++) b *= dims[i];
        return b;
    }
};

// ---- lowering -----------------------------------------------------------------------------------------------
// Pointwise/reduction subgraph of a helium-ir graph → program. Arguments: subgraph inputs in id order, then one
// per leaf in id order (the parameter order of jit.rs:213-221,285-286 is inputs, then outputs as they are stored;
// here outputs are always in leaf order).
Program lower_pointwise(const ir::OpSubgraph& sg);
// A Matmul node (`anchor`) and the pointwise / reduce ops downstream of it -> the GEMM epilogue program over the
// Matmul's output shape. Throws HE_ERR_UNSUPPORTED when the ops cannot run on the accumulator in place.
// `row_dims`: how many leading dims of the anchor's output form the rows of the product (3 for a convolution's
// [n, p, q, channels]); they end up merged into one dim.
Program lower_ir_epilogue(const ir::OpSubgraph& sg, ir::NodeId anchor, size_t row_dims = 1);
// supports_subgraph of helium/src/cuda/instr/pointwise.rs:121-186.
bool pointwise_supports(const ir::OpSubgraph& sg);

// Anchor-less fusion-IR graph (Producer/Consumer at the boundary) → program. Arguments: producers in id order,
// then consumers in id order (kernel_generator.rs:52-63,138-148).
Program lower_aux(const fir::OpGraph& g);
// The epilogue of a Core fusion: everything downstream of `anchor`. Producers that feed only the mainloop are not
// arguments of the program. `arg_nodes` receives the producer / consumer node behind every program argument.
Program lower_epilogue(const fir::OpGraph& g, fir::OpNode anchor);
// One Matmul operand together with the mainloop ops that produce it, evaluated over the operand's own shape
// ([batch, M, K] for a, [batch, K, N] for b). `root_expr` receives the id of the operand's value.
// `transposed`: the same values iterated as [batch, cols, rows] (vector accesses then run along the value's rows).
Program lower_operand(const fir::OpGraph& g, fir::OpNode value, int* root_expr, bool transposed = false);

// Makes `post` (a program over the columns of main's column reductions: no reductions, Bool values or index maps of its
// own) ride on the launch that folds them: its arguments are merged into main->args (shared tensors once, the rest
// appended) and main->post is set. False, with *main untouched, when it cannot.
bool attach_post(Program* main, const Program& post);

// ---- emission -----------------------------------------------------------------------------------------------
struct PointwiseLaunch {
    std::string source, entry;
    uint32_t grid = 1, threads = 256;
    int nv = 1, tx = 1, ty = 1, rpt = 1;
    // Outputs that must be filled before the launch: (argument index, 32-bit fill pattern).
    std::vector<std::pair<int, uint32_t>> fills;
    // Scratch the kernel takes as two trailing arguments (float* then u32*) when nonzero: per-block partial results
    // and arrival counters of the reductions that span several blocks. Counters must be zero before the first
    // launch; the block that arrives last combines the partials in block order and zeroes its counter again.
    uint64_t ws_floats = 0, ws_counters = 0;
    // Long launches fold the partials with a second launch instead: entry `finalize_entry` of the same source, with
    // `finalize_grid` blocks of `threads` threads, taking the kernel's arguments followed by the float scratch.
    std::string finalize_entry;
    uint32_t finalize_grid = 0;
    std::vector<std::string> options;
    std::string describe;
    // Whether the program's `post` is evaluated by the fold launch. False (and `post` ignored) when the column reductions
    // it reads do not all fold in a second launch over the same partial blocks.
    bool post_carried = false;
};
PointwiseLaunch emit_pointwise(const Program& p, const std::string& entry);

// Emits the statements that evaluate every expression for NV consecutive n at the current coordinate.
// The surrounding code must define: `coord[d]` for every iteration dim except the last two as u32 values named
// cB<d>, `m` (u32), `n0` (u32, first of the NV columns), pointer arguments named a<k>, and — for GEMM epilogues —
// float acc[NV]. Results are left in arrays named e<id>[NV].
struct EmitCtx {
    int nv = 1;
    bool guard_vector_loads = false;  // when set, full-width loads are only legal if `vec_ok` is true
    // 0: everything. 1: only the full-vector loads, left undecoded in members raw<expr id> of a struct named `R`.
    // 2: everything else, reading those members. Splitting lets a kernel issue the loads long before it needs them.
    int phase = 0;
    bool defer_row_varying_only = false;  // phases 1/2: loads whose address ignores the row stay in phase 2
    // Pow whose exponent is a launch-uniform operand: written as x * x (the caller has tested the exponents)
    bool uniform_pow_is_square = false;
    // 0: every expression. 1: only those whose value is the same in every row a thread walks (operands that are
    // broadcast along the rows, and what is computed from them alone); their loads are issued only `if (col_ok)`.
    // 2: the others, which read the former from the enclosing scope.
    int row_part = 0;
    // Loads of these arguments take the given expression (a value the surrounding code holds in a register) instead of
    // reading memory.
    const std::map<int, std::string>* arg_values = nullptr;
};
// Per expression: whether its value ignores the row coordinate `m`.
std::vector<char> row_invariant_exprs(const Program& p);
// Whether expression `id` is a Pow whose exponent is a float operand read at one address by the whole launch.
bool is_uniform_pow(const Program& p, int id);
// Members of the struct phase 1 fills: one native vector per deferred Load of the program.
std::string emit_raw_members(const Program& p, int nv, bool row_varying_only = false);
std::string emit_exprs(const Program& p, const EmitCtx& cx);
// Largest vector width (elements) legal for every full-row access and store of the program.
int pick_nv(const Program& p, int max_bytes);
// Whether an output tensor is written with streaming stores (st_vec<NV, true>): 4 MiB or more, i.e. too large to be
// read back out of L2 by whoever comes next.
bool streams_out(const Arg& a);
std::string emit_prelude(const Program& p);
const char* c_type(int dtype);

}  // namespace he::tp
