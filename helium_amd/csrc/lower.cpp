// Lowering of the two front-end IRs to tile programs.
#include <algorithm>
#include <cstring>
#include <map>

#include "tp.h"

namespace he::plan {
bool rematerialize();
bool feeds_only_reductions(const ir::OpGraph& g, ir::NodeId node, int budget);
}
namespace he::tp {

namespace {

// How the linear index of the node being visited depends on the iteration coordinates: an affine part
// (weights per iteration dim, in the node's packed layout) followed by reference-style generic maps.
struct Mapping {
    std::vector<int64_t> w;
    std::vector<GenericMap> chain;
    bool operator==(const Mapping& o) const { return w == o.w && chain == o.chain; }
};

// For every dim of `shape`, the iteration dim its coordinate equals (-1: coordinate 0). Fails when an iteration
// dim does not land on exactly one dim of `shape` (a Reshape regrouped it).
bool try_align(const std::vector<int64_t>& w, const Shape& iter_dims, const Shape& shape, std::vector<int>& src) {
    Shape st = ir::packed_strides(shape);
    src.assign(shape.size(), -1);
    for (size_t d = 0; d < w.size(); d++) {
        if (iter_dims[d] <= 1 || w[d] == 0) continue;
        int found = -1;
        for (size_t j = 0; j < shape.size(); j++)
            if (st[j] == w[d] && shape[j] >= iter_dims[d] && shape[j] > 1) {
                found = (int)j;
                break;
            }
        if (found < 0 || src[found] != -1) return false;
        src[found] = (int)d;
    }
    return true;
}

Mapping through_swap(const Mapping& mp, const Shape& iter_dims, const Shape& out_shape, const Shape& in_shape,
                     int64_t a, int64_t b) {
    Mapping r = mp;
    std::vector<int> src;
    if (mp.chain.empty() && try_align(mp.w, iter_dims, out_shape, src)) {
        Shape st = ir::packed_strides(in_shape);
        std::fill(r.w.begin(), r.w.end(), 0);
        for (size_t j = 0; j < out_shape.size(); j++) {
            if (src[j] < 0) continue;
            size_t k = (int64_t)j == a ? (size_t)b : (int64_t)j == b ? (size_t)a : j;
            r.w[src[j]] += st[k];
        }
        return r;
    }
    GenericMap g;
    g.kind = GenericMap::Swap;
    g.in_shape = in_shape;
    g.axis_a = a;
    g.axis_b = b;
    r.chain.push_back(g);
    return r;
}

Mapping through_broadcast(const Mapping& mp, const Shape& iter_dims, const Shape& out_shape, const Shape& in_shape,
                          const std::vector<char>& bcast) {
    Mapping r = mp;
    std::vector<int> src;
    const size_t pad = out_shape.size() - in_shape.size();
    if (mp.chain.empty() && try_align(mp.w, iter_dims, out_shape, src)) {
        Shape st = ir::packed_strides(in_shape);
        std::fill(r.w.begin(), r.w.end(), 0);
        for (size_t j = pad; j < out_shape.size(); j++) {
            if (src[j] < 0 || bcast[j]) continue;
            r.w[src[j]] += st[j - pad];
        }
        return r;
    }
    GenericMap g;
    g.kind = GenericMap::Bcast;
    g.in_shape = in_shape;
    g.out_shape = out_shape;
    g.bcast = bcast;
    r.chain.push_back(g);
    return r;
}

Cls cls_of(int dtype) {
    switch (dtype_class(dtype)) {
        case DataClass::Float: return Cls::F;
        case DataClass::Int: return Cls::I;
        case DataClass::Bool: return Cls::B;
    }
    return Cls::F;
}

float bf16_bits_to_f32(uint32_t b) {
    uint32_t u = b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
float f16_bits_to_f32(uint32_t h) {
    uint32_t sign = (h >> 15) & 1, exp = (h >> 10) & 0x1f, man = h & 0x3ff, u;
    if (exp == 0) {
        if (man == 0) {
            u = sign << 31;
        } else {
            int e = -1;
            do {
                e++;
                man <<= 1;
            } while (!(man & 0x400));
            u = (sign << 31) | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ff) << 13);
        }
    } else if (exp == 31) {
        u = (sign << 31) | 0x7f800000u | (man << 13);
    } else {
        u = (sign << 31) | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}
uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

// ---------------------------------------------------------------------------------------------------------
// helium-ir pointwise subgraphs
// ---------------------------------------------------------------------------------------------------------
// Element count from which a reduction over leading dims is reordered into a column reduction.
int64_t fold_columns_threshold() {
    if (const char* env = tuning::get("HELIUM_HIP_FOLD_COLUMNS_MIN")) return atoll(env);
    return 1 << 20;
}

class PointwiseLowering {
public:
    // With `anchor` set the subgraph is a Matmul plus the ops that follow it: the program is the epilogue, iterates
    // over the Matmul's output and reads the anchor's value as the accumulator.
    // `row_dims` > 1: the anchor's leading `row_dims` dims together are the rows of the product (the n, p, q of a
    // convolution's NHWC output) and are merged into one dim once the program is built.
    explicit PointwiseLowering(const ir::OpSubgraph& sg, ir::NodeId anchor = ir::kNoNode, size_t row_dims = 1)
        : sg_(sg), g_(*sg.graph()), anchor_(anchor), row_dims_(row_dims) {}

    Program run() {
        HE_REQUIRE(!sg_.leafs().empty(), HE_ERR_INVALID, "pointwise subgraph has no output");
        // Iteration space: the (pre-reduction) shape of the first leaf, as compute_output_shape picks it
        // (jit.rs:350-362) - of the first Reduce leaf when there is one: the reductions of a kernel share one input
        // shape and have to walk it dim by dim, the other outputs only need their element.
        ir::NodeId first = sg_.leafs()[0];
        for (ir::NodeId leaf : sg_.leafs())
            if (g_.get(leaf).op.kind == ir::OpKind::Reduce) {
                first = leaf;
                break;
            }
        const ir::Node& fn = g_.get(first);
        p_.dims = fn.op.kind == ir::OpKind::Reduce ? g_.get(fn.op.inputs[0]).desc.shape : fn.desc.shape;
        if (anchor_ != ir::kNoNode) {
            p_.dims = g_.get(anchor_).desc.shape;
            p_.fast_math = true;
        }
        if (p_.dims.empty()) p_.dims = {1};
        const int64_t numel = ir::num_elements(p_.dims);

        for (ir::NodeId in : sg_.inputs()) {
            const ir::Descriptor& d = g_.get(in).desc;
            input_arg_[in] = (int)p_.args.size();
            p_.args.push_back({d.dtype, ir::num_elements(d.shape), false, in});
        }
        Mapping ident;
        ident.w = ir::packed_strides(p_.dims);
        // Arguments and outputs are in leaf order; the reductions are lowered first, so that a full-size output of another
        // shape (the untransposed tensor next to reductions over its leading dims) can be walked the way they walk it.
        const std::vector<ir::NodeId> leafs = sg_.leafs();
        p_.outs.resize(leafs.size());
        out_depth_.assign(leafs.size(), 0);
        {
            std::vector<Arg> out_args;
            for (ir::NodeId leaf : leafs) {
                const ir::Node& n = g_.get(leaf);
                if (n.op.kind == ir::OpKind::Reduce) out_args.push_back({HE_F32, ir::num_elements(n.desc.shape), true, leaf});
                else out_args.push_back({n.desc.dtype, numel, true, leaf});
            }
            for (size_t k = 0; k < leafs.size(); k++) p_.outs[k].arg = (int)(p_.args.size() + k);
            p_.args.insert(p_.args.end(), out_args.begin(), out_args.end());
        }
        for (int pass = 0; pass < 2; pass++)
        for (size_t leaf_no = 0; leaf_no < leafs.size(); leaf_no++) {
            const ir::NodeId leaf = leafs[leaf_no];
            const ir::Node& n = g_.get(leaf);
            if ((n.op.kind == ir::OpKind::Reduce) != (pass == 0)) continue;
            Out o;
            o.arg = p_.outs[leaf_no].arg;
            cur_out_ = leaf_no;
            if (n.op.kind == ir::OpKind::Reduce) {
                const Shape& rs = g_.get(n.op.inputs[0]).desc.shape;
                HE_REQUIRE(ir::num_elements(rs) == numel, HE_ERR_UNSUPPORTED,
                           "reduction input has a different element count than the other outputs");
                Shape rdims = rs.empty() ? Shape{1} : rs;
                const size_t rank = rdims.size();
                const size_t depth = n.op.depth;
                HE_REQUIRE(depth >= 1 && depth <= rank, HE_ERR_INVALID, "bad reduce depth");
                o.reduce = true;
                o.rop = (ROp)n.op.sub_op;
                int64_t group = 1;
                for (size_t k = rank - depth; k < rank; k++) group *= rdims[k];
                o.mean_scale = 1.0 / (double)group;
                o.dtype = HE_F32;
                // In an epilogue the Reduce's index space may be the product's with its dims permuted (SwapDims + Reduce:
                // column sums, BatchNorm2d statistics of a convolution's output) even where the two shapes are equal
                // (a square product), so the plain reading is only tried first there.
                bool plain = rdims == p_.dims && (row_dims_ <= 1 || depth == 1 || depth == rank);
                if (plain) {
                    o.fold_n = true;
                    o.fold_m = depth >= 2;
                    o.b_div = 1;
                    for (size_t k = rank - depth; k + 2 < rank; k++) o.b_div *= rdims[k];
                    if (row_dims_ > 1) o.b_div = 1;  // all of the rows fold, or none
                    out_depth_[leaf_no] = depth;
                    const size_t exprs = p_.exprs.size(), memo = memo_.size();
                    const int acc = p_.acc_expr;
                    try {
                        o.expr = eval(n.op.inputs[0], ident);
                    } catch (const Error&) {
                        if (anchor_ == ir::kNoNode) throw;
                        p_.exprs.resize(exprs);
                        memo_.resize(memo);
                        p_.acc_expr = acc;
                        plain = false;
                    }
                }
                if (!plain) {
                    HE_REQUIRE(anchor_ != ir::kNoNode, HE_ERR_UNSUPPORTED, "all reductions of a kernel must share one input shape");
                    lower_permuted_reduction(n, rdims, depth, o);
                }
                HE_REQUIRE(p_.exprs[o.expr].cls == Cls::F, HE_ERR_UNSUPPORTED, "reductions take float operands");
            } else {
                HE_REQUIRE(ir::num_elements(n.desc.shape) == numel, HE_ERR_UNSUPPORTED,
                           "all outputs of a pointwise kernel must have the same element count");
                o.dtype = n.desc.dtype;
                // An output whose shape is that of the tensor the reductions' transposition takes is walked through that
                // transposition too: it is then written in the order the reductions read. (Also where the transposed
                // shape is the same - a batch as large as the channel count: the output is a tensor of the untransposed
                // kind, and any one-to-one walk of it is correct.)
                auto nat = natural_.find(n.desc.shape);
                if (anchor_ == ir::kNoNode && n.desc.dtype != HE_BOOL && nat != natural_.end()) {
                    o.stride = nat->second.w;
                    o.expr = eval(leaf, nat->second);
                } else {
                    o.expr = eval(leaf, ident);
                }
            }
            p_.outs[leaf_no] = o;
        }
        if (anchor_ != ir::kNoNode) {
            drop_unused_inputs();
            merge_row_dims();
        } else {
            drop_unit_dims();
            fold_leading_dims_as_columns();
            merge_row_like_dims();
        }
        return std::move(p_);
    }

private:
    bool reads_anchor(ir::NodeId node) const {
        if (node == anchor_) return true;
        if (sg_.is_input(node) || !sg_.contains(node)) return false;
        for (ir::NodeId in : g_.get(node).op.inputs)
            if (reads_anchor(in)) return true;
        return false;
    }

    // Reduce leaf of an epilogue whose input shape `rdims` is a permutation of the iteration dims. Extents may repeat
    // (a square product), so every matching permutation is tried: the right one is the one under which the path back
    // to the anchor arrives with the identity mapping.
    void lower_permuted_reduction(const ir::Node& n, const Shape& rdims, size_t depth, Out& o) {
        const size_t R = p_.dims.size();
        HE_REQUIRE(rdims.size() == R && reads_anchor(n.op.inputs[0]), HE_ERR_UNSUPPORTED,
                   "reduction input is not a permutation of the Matmul result");
        const Shape rst = ir::packed_strides(rdims);
        std::vector<size_t> perm(R);  // perm[j]: the iteration dim that the Reduce's dim j walks
        for (size_t j = 0; j < R; j++) perm[j] = j;
        bool done = false;
        do {
            bool fits = true;
            for (size_t j = 0; j < R; j++) fits = fits && rdims[j] == p_.dims[perm[j]];
            if (!fits) continue;
            Mapping mp;
            mp.w.assign(R, 0);
            for (size_t j = 0; j < R; j++) mp.w[perm[j]] = rst[j];
            const size_t exprs = p_.exprs.size(), memo = memo_.size();
            const int acc = p_.acc_expr;
            try {
                o.expr = eval(n.op.inputs[0], mp);
                done = true;
            } catch (const Error&) {
                p_.exprs.resize(exprs);
                memo_.resize(memo);
                p_.acc_expr = acc;
            }
        } while (!done && std::next_permutation(perm.begin(), perm.end()));
        HE_REQUIRE(done, HE_ERR_UNSUPPORTED, "the reduction reads the Matmul result through more than a permutation of its dims");
        HE_REQUIRE(p_.exprs[o.expr].cls == Cls::F, HE_ERR_UNSUPPORTED, "reductions take float operands");
        // which of [batch.., rows, cols] the folded dims are
        const size_t rows_first = row_dims_ > 1 ? 0 : R - 2, cols = R - 1;
        size_t rows_folded = 0, rows_total = R >= 2 ? cols - rows_first : 0;
        bool cols_folded = false;
        for (size_t j = R - depth; j < R; j++) {
            const size_t d = perm[j];
            if (d == cols) cols_folded = true;
            else if (R >= 2 && d >= rows_first) rows_folded++;
            else fail(HE_ERR_UNSUPPORTED, "a reduction over the batch dim of a product is not fused");
        }
        HE_REQUIRE(rows_folded == 0 || rows_folded == rows_total, HE_ERR_UNSUPPORTED, "the reduction folds part of the product's rows");
        o.fold_n = cols_folded;
        o.fold_m = rows_folded != 0;
        o.b_div = 1;
        // the kept dims keep their order, so that the output is indexed like the product with the folded dims dropped
        size_t last = 0;
        for (size_t j = 0; j + depth < R; j++) {
            HE_REQUIRE(j == 0 || perm[j] > last, HE_ERR_UNSUPPORTED, "the reduction's kept dims are permuted");
            last = perm[j];
        }
    }

    // A kernel without reductions treats every dim but the last as rows: neighbours that every operand walks as one dim
    // (packed tensors; vectors broadcast along all of them) are merged, so that an NHWC activation normalised per
    // channel is [n*h*w, c] — long columns of rows for a block to walk — instead of [n, h][w][c] with w rows per block.
    void merge_row_like_dims() {
        for (auto& o : p_.outs)
            if (o.reduce) return;
        for (auto& e : p_.exprs)
            if (e.kind == Expr::Load && (!e.access.chain.empty() || e.access.stride.size() != p_.dims.size())) return;
        for (auto& o : p_.outs)
            if (!o.stride.empty()) return;  // (only next to reductions, which returned above)
        for (size_t i = 0; i + 2 < p_.dims.size();) {
            bool ok = true;
            for (auto& e : p_.exprs)
                if (e.kind == Expr::Load && e.access.stride[i] != e.access.stride[i + 1] * p_.dims[i + 1]) ok = false;
            if (!ok) {
                i++;
                continue;
            }
            p_.dims[i + 1] *= p_.dims[i];
            p_.dims.erase(p_.dims.begin() + i);
            for (auto& e : p_.exprs)
                if (e.kind == Expr::Load) e.access.stride.erase(e.access.stride.begin() + i);
        }
    }

    // Dims of extent 1 leave the iteration space: the canonical view takes the last dim as the columns and the one
    // before as the rows, and a reduction over [1000, 128, 1, 1] (the gradient of a bias that was broadcast from
    // [1000, 1, 1]) would otherwise run with one element per workgroup. A reduction folds the trailing dims, so its
    // depth counts the remaining ones; one that folded unit dims only is the identity.
    void drop_unit_dims() {
        const size_t R = p_.dims.size();
        for (auto& e : p_.exprs)
            if (e.kind == Expr::Load && e.access.stride.size() != R) return;
        for (auto& o : p_.outs)
            if (!o.stride.empty() && o.stride.size() != R) return;
        out_depth_.resize(p_.outs.size(), 0);
        for (size_t i = 0; i < p_.outs.size(); i++) {
            if (!p_.outs[i].reduce) continue;
            size_t depth = 0;
            for (size_t k = R - out_depth_[i]; k < R; k++) depth += p_.dims[k] != 1;
            out_depth_[i] = depth;
        }
        for (size_t d = R; d-- > 0;) {
            if (p_.dims[d] != 1 || p_.dims.size() == 1) continue;
            p_.dims.erase(p_.dims.begin() + d);
            for (auto& e : p_.exprs)
                if (e.kind == Expr::Load) e.access.stride.erase(e.access.stride.begin() + d);
            for (auto& o : p_.outs)
                if (!o.stride.empty()) o.stride.erase(o.stride.begin() + d);
        }
        const size_t rank = p_.dims.size();
        for (size_t i = 0; i < p_.outs.size(); i++) {
            Out& o = p_.outs[i];
            if (!o.reduce) continue;
            const size_t depth = out_depth_[i];
            if (depth == 0) {
                o.reduce = false;
                continue;
            }
            o.fold_n = true;
            o.fold_m = depth >= 2;
            o.b_div = 1;
            for (size_t k = rank - depth; k + 2 < rank; k++) o.b_div *= p_.dims[k];
        }
    }

    // A convolution's epilogue is lowered over [n, p, q, channels]; the product's rows are (n, p, q) together.
    void merge_row_dims() {
        while (row_dims_ > 1) {
            for (auto& e : p_.exprs)
                if (e.kind == Expr::Load)
                    HE_REQUIRE(e.access.chain.empty() && e.access.stride[0] == e.access.stride[1] * p_.dims[1], HE_ERR_UNSUPPORTED,
                               "an epilogue operand does not walk the product's rows as one dim");
            p_.dims[1] *= p_.dims[0];
            p_.dims.erase(p_.dims.begin());
            for (auto& e : p_.exprs)
                if (e.kind == Expr::Load) e.access.stride.erase(e.access.stride.begin());
            row_dims_--;
        }
    }

    // helium-ir's Reduce folds trailing dims only, so a reduction over leading dims reaches the kernel as
    // SwapDims + Reduce (BatchNorm2d statistics over N, H, W of an NHWC tensor, helium/src/modules/batch_norm.rs:38-46;
    // column sums). Iterated in the Reduce's own index space, the innermost coordinate then strides through memory.
    // When every output is a reduction of one depth and the largest operand is contiguous along the last *kept* dim,
    // the iteration space is reordered to [other kept dims, folded dims by decreasing stride, last kept dim] and
    // mergeable folded dims are merged: the kernel then walks memory in order and folds rows (and part of the batch
    // index) per column, which the emitter does with one pass over the operand.
    void fold_leading_dims_as_columns() {
        const size_t R = p_.dims.size();
        if (p_.outs.empty() || R < 2) return;
        // Small tensors stay as they are: they live in the caches whatever the order, and rows that one wave folds
        // need no exchange between blocks, which at that size costs more than the strided reads.
        if (ir::num_elements(p_.dims) < fold_columns_threshold()) return;
        // (full-size outputs may sit next to the reductions when they are stored by strides of their own)
        size_t depth = 0;
        bool any_reduce = false;
        for (size_t i = 0; i < p_.outs.size(); i++) {
            if (!p_.outs[i].reduce) {
                if (p_.outs[i].stride.size() != R) return;
                continue;
            }
            if (any_reduce && out_depth_[i] != depth) return;
            depth = out_depth_[i];
            any_reduce = true;
        }
        if (!any_reduce) return;
        if (depth >= R) return;
        const size_t K = R - depth, kl = K - 1;
        const Expr* big = nullptr;
        for (auto& e : p_.exprs) {
            if (e.kind != Expr::Load) continue;
            if (!e.access.chain.empty() || e.access.stride.size() != R) return;
            if (!big || p_.args[e.access.arg].numel > p_.args[big->access.arg].numel) big = &e;
        }
        if (!big || big->access.stride[kl] != 1 || p_.dims[kl] < 16 || big->access.stride[R - 1] == 1) return;
        std::vector<size_t> perm;
        for (size_t d = 0; d + 1 < K; d++) perm.push_back(d);
        std::vector<size_t> folded;
        for (size_t d = K; d < R; d++) folded.push_back(d);
        const std::vector<int64_t> key = big->access.stride;
        std::stable_sort(folded.begin(), folded.end(), [&](size_t a, size_t b) { return key[a] > key[b]; });
        perm.insert(perm.end(), folded.begin(), folded.end());
        perm.push_back(kl);
        auto permute = [&](std::vector<int64_t>& v) {
            std::vector<int64_t> r(R);
            for (size_t i = 0; i < R; i++) r[i] = v[perm[i]];
            v = r;
        };
        permute(p_.dims);
        for (auto& e : p_.exprs)
            if (e.kind == Expr::Load) permute(e.access.stride);
        for (auto& o : p_.outs)
            if (!o.reduce) permute(o.stride);
        // merge neighbours among the folded dims (positions K-1 .. size-2) that every operand walks as one dim
        for (size_t i = K - 1; i + 2 < p_.dims.size();) {
            bool ok = true;
            for (auto& e : p_.exprs)
                if (e.kind == Expr::Load && e.access.stride[i] != e.access.stride[i + 1] * p_.dims[i + 1]) ok = false;
            for (auto& o : p_.outs)
                if (!o.reduce && o.stride[i] != o.stride[i + 1] * p_.dims[i + 1]) ok = false;
            if (!ok) {
                i++;
                continue;
            }
            p_.dims[i + 1] *= p_.dims[i];
            p_.dims.erase(p_.dims.begin() + i);
            for (auto& e : p_.exprs)
                if (e.kind == Expr::Load) e.access.stride.erase(e.access.stride.begin() + i);
            for (auto& o : p_.outs)
                if (!o.reduce) o.stride.erase(o.stride.begin() + i);
        }
        int64_t b_div = 1;
        for (size_t i = K - 1; i + 2 < p_.dims.size(); i++) b_div *= p_.dims[i];
        for (auto& o : p_.outs) {
            if (!o.reduce) continue;
            o.fold_n = false;
            o.fold_m = true;
            o.b_div = b_div;
        }
    }

    // The Matmul's own operands are inputs of the subgraph but not of the epilogue unless an epilogue op reads them.
    void drop_unused_inputs() {
        std::vector<char> used(p_.args.size(), 0);
        for (auto& e : p_.exprs)
            if (e.kind == Expr::Load) used[e.access.arg] = 1;
        std::vector<int> remap(p_.args.size(), -1);
        std::vector<Arg> kept;
        for (size_t a = 0; a < p_.args.size(); a++)
            if (p_.args[a].is_output || used[a]) {
                remap[a] = (int)kept.size();
                kept.push_back(p_.args[a]);
            }
        for (auto& e : p_.exprs)
            if (e.kind == Expr::Load) e.access.arg = remap[e.access.arg];
        for (auto& o : p_.outs) o.arg = remap[o.arg];
        p_.args = kept;
    }

    int push(Expr e) {
        p_.exprs.push_back(std::move(e));
        return (int)p_.exprs.size() - 1;
    }

    int eval(ir::NodeId node, const Mapping& mp) {
        for (auto& m : memo_)
            if (m.node == node && m.mp == mp) return m.expr;
        int id = eval_uncached(node, mp);
        memo_.push_back({node, mp, id});
        return id;
    }

    int eval_uncached(ir::NodeId node, const Mapping& mp) {
        const ir::Node& n = g_.get(node);
        if (sg_.is_input(node)) {
            Expr e;
            e.kind = Expr::Load;
            e.cls = cls_of(n.desc.dtype);
            e.access.arg = input_arg_.at(node);
            e.access.dtype = n.desc.dtype;
            e.access.stride = mp.w;
            e.access.chain = mp.chain;
            return push(e);
        }
        HE_REQUIRE(sg_.contains(node) && n.kind == ir::Node::Intermediate, HE_ERR_INVALID,
                   "node %u is outside the subgraph", node);
        if (node == anchor_) {
            // the accumulator exists only at the coordinate a thread owns: the path from the outputs back to the
            // Matmul must not move or repeat elements
            HE_REQUIRE(mp.chain.empty() && mp.w == ir::packed_strides(p_.dims), HE_ERR_UNSUPPORTED,
                       "the epilogue reads the Matmul result through a transposition or broadcast");
            Expr e;
            e.kind = Expr::Acc;
            e.cls = Cls::F;
            p_.acc_expr = push(e);
            return p_.acc_expr;
        }
        const ir::Op& op = n.op;
        auto in_shape = [&](size_t i) -> const Shape& { return g_.get(op.inputs[i]).desc.shape; };
        switch (op.kind) {
            case ir::OpKind::SwapDims: {
                Mapping below = through_swap(mp, p_.dims, n.desc.shape, in_shape(0), op.axis_a, op.axis_b);
                // (how the iteration space walks a tensor of the untransposed shape: kept for full-size outputs of it)
                if (below.chain.empty() && g_.get(op.inputs[0]).op.kind != ir::OpKind::SwapDims) natural_.emplace(in_shape(0), below);
                return eval(op.inputs[0], below);
            }
            case ir::OpKind::Broadcast: {
                std::vector<char> flags(n.desc.shape.size(), 0);
                for (auto& a : op.broadcast_axes) flags[a.axis] = 1;
                return eval(op.inputs[0], through_broadcast(mp, p_.dims, n.desc.shape, in_shape(0), flags));
            }
            case ir::OpKind::Reshape: return eval(op.inputs[0], mp);
            case ir::OpKind::ChangeDataType: {
                int x = eval(op.inputs[0], mp);
                Cls to = cls_of(op.target_type);
                if (p_.exprs[x].cls == to) return x;  // same class: only loads and stores change (jit.rs:674-690)
                Expr e;
                e.kind = Expr::Cast;
                e.cls = to;
                e.a = x;
                return push(e);
            }
            case ir::OpKind::UnaryPointwise: {
                Expr e;
                e.kind = Expr::Unary;
                e.a = eval(op.inputs[0], mp);
                e.cls = p_.exprs[e.a].cls;
                HE_REQUIRE(e.cls == Cls::F, HE_ERR_UNSUPPORTED, "unary pointwise ops take float operands");
                static const UOp map[] = {UOp::Recip, UOp::Neg, UOp::Exp, UOp::Sin, UOp::Cos, UOp::Tan,
                                          UOp::Sigmoid, UOp::Tanh, UOp::Relu, UOp::Sqrt, UOp::Log};
                HE_REQUIRE(op.sub_op >= 0 && op.sub_op < 11, HE_ERR_INVALID, "bad unary op");
                e.op = (int)map[op.sub_op];
                return push(e);
            }
            case ir::OpKind::BinaryPointwise: {
                Expr e;
                e.kind = Expr::Binary;
                e.a = eval(op.inputs[0], mp);
                e.b = eval(op.inputs[1], mp);
                e.cls = p_.exprs[e.a].cls;
                HE_REQUIRE(p_.exprs[e.b].cls == e.cls, HE_ERR_UNSUPPORTED, "binary operands differ in data class");
                static const BOp map[] = {BOp::Add, BOp::Mul, BOp::Pow, BOp::Min, BOp::Max, BOp::And, BOp::Or, BOp::Xor};
                HE_REQUIRE(op.sub_op >= 0 && op.sub_op < 8, HE_ERR_INVALID, "bad binary op");
                e.op = (int)map[op.sub_op];
                return push(e);
            }
            case ir::OpKind::Compare: {
                Expr e;
                e.kind = Expr::Compare;
                e.cls = Cls::B;
                e.a = eval(op.inputs[0], mp);
                e.b = eval(op.inputs[1], mp);
                e.op = op.sub_op;
                return push(e);
            }
            case ir::OpKind::Select: {
                Expr e;
                e.kind = Expr::Select;
                e.a = eval(op.inputs[0], mp);
                e.b = eval(op.inputs[1], mp);
                e.c = eval(op.inputs[2], mp);
                e.cls = p_.exprs[e.a].cls;
                HE_REQUIRE(p_.exprs[e.c].cls == Cls::B, HE_ERR_UNSUPPORTED, "select needs a bool selector");
                return push(e);
            }
            case ir::OpKind::Constant: {
                Expr e;
                e.kind = Expr::Const;
                e.cls = cls_of(op.const_dtype);
                switch (op.const_dtype) {
                    case HE_F32: e.bits = op.const_bits; break;
                    case HE_BF16: e.bits = f32_bits(bf16_bits_to_f32(op.const_bits & 0xffff)); break;
                    case HE_F16: e.bits = f32_bits(f16_bits_to_f32(op.const_bits & 0xffff)); break;
                    case HE_U32: e.bits = op.const_bits; break;
                    case HE_BOOL: e.bits = op.const_bits ? 1 : 0; break;
                }
                return push(e);
            }
            case ir::OpKind::Reduce: fail(HE_ERR_UNSUPPORTED, "a reduction must be an output of its kernel");
            default: fail(HE_ERR_UNSUPPORTED, "op kind is not handled by the pointwise instruction");
        }
    }

    struct Memo {
        ir::NodeId node;
        Mapping mp;
        int expr;
    };
    const ir::OpSubgraph& sg_;
    const ir::OpGraph& g_;
    ir::NodeId anchor_;
    size_t row_dims_ = 1;
    Program p_;
    std::map<ir::NodeId, int> input_arg_;
    std::vector<Memo> memo_;
    std::vector<size_t> out_depth_;  // per output: the Reduce's depth (0 for full-size outputs)
    std::map<Shape, Mapping> natural_;  // shape of a transposition's operand -> the affine mapping the iteration walks it with
    size_t cur_out_ = 0;
};

// ---------------------------------------------------------------------------------------------------------
// fusion-IR graphs (aux fusions and GEMM epilogues)
// ---------------------------------------------------------------------------------------------------------
class FusionLowering {
public:
    FusionLowering(const fir::OpGraph& g, fir::OpNode anchor) : g_(g), anchor_(anchor) {}

    Program run() {
        // Outputs: every leaf; a Consumer stands for the node it reads (kernel_generator.rs:157-167).
        std::vector<std::pair<fir::OpNode, fir::OpNode>> outs;  // (leaf id, value node)
        for (fir::OpNode leaf : g_.leaves()) {
            const fir::Op& op = g_.get(leaf);
            fir::OpNode x = op.kind == fir::OpKind::Consumer ? op.a : leaf;
            if (anchor_ != fir::kNoOpNode && !downstream_of_anchor(x)) continue;
            outs.push_back({leaf, x});
        }
        HE_REQUIRE(!outs.empty(), HE_ERR_INVALID, "fusion has no output");

        // Iteration space: the anchor's output; without an anchor, the (pre-reduction) shape of the first output.
        // (The reference takes M and N from its largest root, kernel_generator.rs:98-106, which only agrees with
        // the outputs when no input is transposed.)
        fir::Shape3 s;
        if (anchor_ != fir::kNoOpNode) {
            s = g_.shape(anchor_);
        } else {
            const fir::Op& vop = g_.get(outs[0].second);
            s = vop.kind == fir::OpKind::Reduction ? g_.shape(vop.a) : g_.shape(outs[0].second);
        }
        p_.dims = {s[0], s[1], s[2]};

        // Arguments: producers reachable from the outputs (in id order), then outputs (in leaf order).
        std::vector<fir::OpNode> producers;
        {
            std::vector<fir::OpNode> stack;
            std::map<fir::OpNode, char> seen;
            for (auto& o : outs) stack.push_back(o.second);
            while (!stack.empty()) {
                fir::OpNode n = stack.back();
                stack.pop_back();
                if (seen[n]++) continue;
                if (n == anchor_) continue;  // the mainloop side is not part of this program
                if (g_.get(n).kind == fir::OpKind::Producer) producers.push_back(n);
                for (fir::OpNode i : g_.inbound(n)) stack.push_back(i);
            }
            std::sort(producers.begin(), producers.end());
        }
        for (fir::OpNode pnode : producers) {
            const fir::Shape3& ps = g_.shape(pnode);
            input_arg_[pnode] = (int)p_.args.size();
            p_.args.push_back({g_.get(pnode).dtype, (int64_t)ps[0] * ps[1] * ps[2], false, pnode});
        }
        Mapping ident;
        ident.w = ir::packed_strides(p_.dims);
        for (auto& [leaf, x] : outs) {
            const fir::Op& vop = g_.get(x);
            Out o;
            o.arg = (int)p_.args.size();
            if (vop.kind == fir::OpKind::Reduction) {
                const fir::Shape3& rs = g_.shape(vop.a);
                HE_REQUIRE(Shape({rs[0], rs[1], rs[2]}) == p_.dims, HE_ERR_UNSUPPORTED,
                           "reduction input shape differs from the fusion's tile space");
                o.reduce = true;
                o.rop = ROp::Sum;
                switch (vop.depth) {
                    case fir::ReductionDepth::Rows: o.fold_n = true; break;
                    case fir::ReductionDepth::Columns: o.fold_m = true; break;
                    case fir::ReductionDepth::Item: o.fold_n = o.fold_m = true; break;
                    case fir::ReductionDepth::Batch:
                        o.fold_n = o.fold_m = true;
                        o.b_div = rs[0];
                        break;
                }
                o.dtype = HE_F32;  // reductions accumulate and are stored in f32
                o.expr = eval(vop.a, ident);
                const fir::Shape3& os = g_.shape(x);
                p_.args.push_back({HE_F32, (int64_t)os[0] * os[1] * os[2], true, leaf});
            } else {
                const fir::Shape3& vs = g_.shape(x);
                HE_REQUIRE(Shape({vs[0], vs[1], vs[2]}) == p_.dims, HE_ERR_UNSUPPORTED,
                           "full-size outputs must have the fusion's tile-space shape (transposed outputs are not fused)");
                o.dtype = g_.get(leaf).kind == fir::OpKind::Consumer ? g_.get(leaf).dtype : HE_BF16;
                o.expr = eval(x, ident);
                p_.args.push_back({o.dtype, ir::num_elements(p_.dims), true, leaf});
            }
            p_.outs.push_back(o);
        }
        return std::move(p_);
    }

    // The value of one node (a Matmul operand with its mainloop ops) over that node's own shape.
    // `transposed`: iterate the value as [batch, cols, rows], so that vectors run along its rows' direction
    Program run_value(fir::OpNode value, int* root, bool transposed = false) {
        const fir::Shape3& s = g_.shape(value);
        p_.dims = {s[0], s[1], s[2]};
        if (transposed) p_.dims = {s[0], s[2], s[1]};
        std::vector<fir::OpNode> producers, stack{value};
        std::map<fir::OpNode, char> seen;
        while (!stack.empty()) {
            fir::OpNode n = stack.back();
            stack.pop_back();
            if (seen[n]++) continue;
            HE_REQUIRE(g_.get(n).kind != fir::OpKind::Matmul && g_.get(n).kind != fir::OpKind::Reduction,
                       HE_ERR_UNSUPPORTED, "a mainloop fusion holds pointwise, broadcast and transpose ops only");
            if (g_.get(n).kind == fir::OpKind::Producer) producers.push_back(n);
            for (fir::OpNode i : g_.inbound(n)) stack.push_back(i);
        }
        std::sort(producers.begin(), producers.end());
        for (fir::OpNode pnode : producers) {
            const fir::Shape3& ps = g_.shape(pnode);
            input_arg_[pnode] = (int)p_.args.size();
            p_.args.push_back({g_.get(pnode).dtype, (int64_t)ps[0] * ps[1] * ps[2], false, pnode});
        }
        Mapping ident;
        ident.w = ir::packed_strides(p_.dims);
        if (transposed) ident.w = {(int64_t)s[1] * s[2], 1, (int64_t)s[2]};  // the value's own packed strides, per iteration dim
        *root = eval(value, ident);
        return std::move(p_);
    }

private:
    bool downstream_of_anchor(fir::OpNode n) {
        auto it = down_.find(n);
        if (it != down_.end()) return it->second;
        bool r = n == anchor_;
        if (!r)
            for (fir::OpNode i : g_.inbound(n)) r = r || downstream_of_anchor(i);
        return down_[n] = r;
    }

    int push(Expr e) {
        p_.exprs.push_back(std::move(e));
        return (int)p_.exprs.size() - 1;
    }

    int eval(fir::OpNode node, const Mapping& mp) {
        for (auto& m : memo_)
            if (m.node == node && m.mp == mp) return m.expr;
        int id = eval_uncached(node, mp);
        memo_.push_back({node, mp, id});
        return id;
    }

    int eval_uncached(fir::OpNode node, const Mapping& mp) {
        const fir::Op& op = g_.get(node);
        auto shape_of = [&](fir::OpNode n) {
            const fir::Shape3& s = g_.shape(n);
            return Shape{s[0], s[1], s[2]};
        };
        if (node == anchor_) {
            HE_REQUIRE(mp.chain.empty() && mp.w == ir::packed_strides(p_.dims), HE_ERR_UNSUPPORTED,
                       "the anchor's tile can only be read in place (no transpose/broadcast of the GEMM result)");
            if (p_.acc_expr < 0) {
                Expr e;
                e.kind = Expr::Acc;
                e.cls = Cls::F;
                p_.acc_expr = push(e);
            }
            return p_.acc_expr;
        }
        switch (op.kind) {
            case fir::OpKind::Producer: {
                Expr e;
                e.kind = Expr::Load;
                e.cls = cls_of(op.dtype);
                HE_REQUIRE(e.cls == Cls::F, HE_ERR_UNSUPPORTED, "fusion-IR tensors are float tensors");
                e.access.arg = input_arg_.at(node);
                e.access.dtype = op.dtype;
                e.access.stride = mp.w;
                e.access.chain = mp.chain;
                return push(e);
            }
            case fir::OpKind::Constant: {
                Expr e;
                e.kind = Expr::Const;
                e.cls = Cls::F;
                e.bits = f32_bits(op.value);
                return push(e);
            }
            case fir::OpKind::UnaryPointwise: {
                Expr e;
                e.kind = Expr::Unary;
                e.cls = Cls::F;
                e.a = eval(op.a, mp);
                static const UOp map[] = {UOp::Neg, UOp::Relu, UOp::Gelu, UOp::Tanh, UOp::Exp, UOp::Log, UOp::Sqrt,
                                          UOp::AddC, UOp::MulC, UOp::PowC};
                HE_REQUIRE(op.sub_op >= 0 && op.sub_op < 10, HE_ERR_INVALID, "bad unary op");
                e.op = (int)map[op.sub_op];
                e.bits = f32_bits(op.constant);
                return push(e);
            }
            case fir::OpKind::BinaryPointwise: {
                Expr e;
                e.kind = Expr::Binary;
                e.cls = Cls::F;
                e.a = eval(op.a, mp);
                e.b = eval(op.b, mp);
                static const BOp map[] = {BOp::Add, BOp::Sub, BOp::Mul, BOp::Div, BOp::Pow, BOp::Drelu};
                HE_REQUIRE(op.sub_op >= 0 && op.sub_op < 6, HE_ERR_INVALID, "bad binary op");
                e.op = (int)map[op.sub_op];
                return push(e);
            }
            case fir::OpKind::Broadcast: {
                std::vector<char> flags(3, 0);
                flags[op.axis] = 1;
                return eval(op.a, through_broadcast(mp, p_.dims, shape_of(node), shape_of(op.a), flags));
            }
            case fir::OpKind::Transpose:
                return eval(op.a, through_swap(mp, p_.dims, shape_of(node), shape_of(op.a), 1, 2));
            case fir::OpKind::Consumer: return eval(op.a, mp);
            case fir::OpKind::Reduction: fail(HE_ERR_UNSUPPORTED, "a reduction terminates its fusion");
            case fir::OpKind::Matmul: fail(HE_ERR_UNSUPPORTED, "a fusion holds at most one Matmul");
        }
        fail(HE_ERR_INVALID, "bad fusion-IR op");
    }

    struct Memo {
        fir::OpNode node;
        Mapping mp;
        int expr;
    };
    const fir::OpGraph& g_;
    fir::OpNode anchor_;
    Program p_;
    std::map<fir::OpNode, int> input_arg_;
    std::map<fir::OpNode, bool> down_;
    std::vector<Memo> memo_;
};

}  // namespace

bool pointwise_supports(const ir::OpSubgraph& sg) {
    // helium/src/cuda/instr/pointwise.rs:121-186, statement for statement: `x` counts Broadcasts as well as
    // SwapDims, and only a SwapDims checks it.
    const ir::OpGraph& g = *sg.graph();
    int64_t output_size = -1;
    bool have_red = false;
    Shape red_shape;
    uint32_t red_depth = 0;
    int x = 0;
    for (ir::NodeId node : sg.nodes()) {
        const ir::Op& op = g.get(node).op;
        ir::NodeId check = op.kind == ir::OpKind::Reduce ? op.inputs[0] : node;
        if (sg.is_leaf(node)) {
            int64_t n = ir::num_elements(g.get(check).desc.shape);
            if (output_size < 0)
                output_size = n;
            else if (output_size != n)
                return false;
        }
        switch (op.kind) {
            case ir::OpKind::Select:
            case ir::OpKind::Reshape:
            case ir::OpKind::Compare:
            case ir::OpKind::UnaryPointwise:
            case ir::OpKind::BinaryPointwise:
            case ir::OpKind::ChangeDataType: continue;
            case ir::OpKind::Broadcast: x += 1; break;
            case ir::OpKind::SwapDims:
                x += 1;
                // (the generator here walks any number of broadcasts and transpositions as strides; the count is the
                // reference's, kept when graphs are planned as recorded)
                if (x > 1 && !plan::rematerialize()) return false;
                break;
            case ir::OpKind::Reduce: {
                if (!sg.is_leaf(node)) return false;
                // (not in the reference's text, which asks for a leaf only: a reduction with one consumer inside and
                // one outside is a leaf, but the inside one cannot read a value that only exists when every thread
                // has finished - that merge is refused as well)
                for (ir::NodeId c : g.outbound(node))
                    if (sg.contains(c)) return false;
                const Shape& s = g.get(op.inputs[0]).desc.shape;
                if (!have_red) {
                    have_red = true;
                    red_shape = s;
                    red_depth = op.depth;
                } else if (red_shape != s || red_depth != op.depth) {
                    return false;
                }
                break;
            }
            case ir::OpKind::Constant:
                // The reference's `_ => return false` includes Constant: a constant is always a kernel of its own that
                // fills a tensor (the zeros and ones of a relu's gradient mask, each as large as the activation). With
                // rematerialisation on it is an immediate of the kernel that uses it.
                if (!plan::rematerialize()) return false;
                continue;
            default: return false;
        }
    }
    // A kernel iterates over one shape: that of its first output, or the input shape of its reductions. Outputs of
    // another shape (the transposed tensor next to the untransposed one) are then written element by element in an
    // order that shares nothing with what the others read, which a large tensor cannot afford: they stay in a kernel
    // of their own. (The reference's rule compares element counts only.)
    // A transposition inside a large kernel is there for reductions over leading dims, which walk the untransposed
    // tensor in memory order when every output of the kernel is such a reduction; any other output next to them (the
    // transposed tensor itself, or a tensor of the same extents in another order - a batch as large as the channel
    // count makes the two shapes equal) would be written element by element.
    if (plan::rematerialize() && output_size >= fold_columns_threshold() && sg.nodes().size() > 1) {
        // The one other output such a kernel may have: a full-size tensor of the shape the transpositions take (the
        // untransposed tensor, or one computed element by element from it), provided every transposition is there for
        // the reductions alone. It is stored through the same walk (tp::Out::stride), in memory order.
        bool transposes = false, swaps_for_reductions = true, one_source_shape = true;
        const Shape* source_shape = nullptr;
        for (ir::NodeId node : sg.nodes()) {
            const ir::Op& op = g.get(node).op;
            if (op.kind != ir::OpKind::SwapDims) continue;
            transposes = true;
            swaps_for_reductions = swaps_for_reductions && plan::feeds_only_reductions(g, node, 64);
            const ir::Node& in = g.get(op.inputs[0]);
            if (in.kind == ir::Node::Intermediate && in.op.kind == ir::OpKind::SwapDims) continue;
            if (source_shape && *source_shape != in.desc.shape) one_source_shape = false;
            source_shape = &in.desc.shape;
        }
        const Shape* shape = nullptr;
        for (ir::NodeId node : sg.leafs()) {
            const ir::Op& op = g.get(node).op;
            // (an output on its way to reductions that have not joined yet is let through: instructions fuse in pairs)
            const bool for_reductions = op.kind == ir::OpKind::Reduce || plan::feeds_only_reductions(g, node, 64);
            const Shape& mine = g.get(op.kind == ir::OpKind::Reduce ? op.inputs[0] : node).desc.shape;
            if (transposes && !for_reductions) {
                if (!(swaps_for_reductions && one_source_shape && source_shape && *source_shape == mine && have_red &&
                      g.get(node).desc.dtype != HE_BOOL))
                    return false;
                continue;
            }
            if (shape && *shape != mine) return false;
            shape = &mine;
        }
    }
    return true;
}

Program lower_pointwise(const ir::OpSubgraph& sg) { return PointwiseLowering(sg).run(); }
Program lower_ir_epilogue(const ir::OpSubgraph& sg, ir::NodeId anchor, size_t row_dims) {
    return PointwiseLowering(sg, anchor, row_dims).run();
}
Program lower_aux(const fir::OpGraph& g) {
    HE_REQUIRE(g.anchor() == fir::kNoOpNode, HE_ERR_INVALID, "an auxiliary fusion holds no Matmul");
    return FusionLowering(g, fir::kNoOpNode).run();
}
Program lower_operand(const fir::OpGraph& g, fir::OpNode value, int* root_expr, bool transposed) {
    return FusionLowering(g, fir::kNoOpNode).run_value(value, root_expr, transposed);
}
Program lower_epilogue(const fir::OpGraph& g, fir::OpNode anchor) {
    Program p = FusionLowering(g, anchor).run();
    p.fast_math = true;
    return p;
}

}  // namespace he::tp
