"""Pointwise / reduction kernel cases shared by the CPU-emulation and GPU parity tests.

Each case builds a helium-ir graph through the C ABI the way helium/src/raw_tensor.rs would, names the subgraph
that forms ONE kernel, and gives seeded inputs. `expected` holds the reference's own known answers where the case
is transcribed from helium/tests/tensor_ops.rs.
"""
import numpy as np

import helium_amd as ha
from oracle import numerics as nm

from helpers import broadcast_to, div, scalar_tensor, sub


class Case:
    def __init__(self, name):
        self.name = name
        self.g = ha.ir.OpGraph()
        self.inputs = {}
        self.nodes = []
        self.leaves = []
        self.expected = {}
        self.reduce_rel = None
        self.admitted_by_fusion_rule = True
        self.env = {}  # environment overrides the kernel is generated under
        self.describes = None  # text the kernel's description has to hold

    def inp(self, shape, dtype, values):
        i = self.g.new_input(list(shape), dtype)
        self.inputs[i] = nm.to_storage(np.asarray(values).reshape(shape), dtype)
        return i

    def op(self, node):
        self.nodes.append(node)
        return node

    def out(self, node, expected=None):
        self.g.new_output(node)
        self.leaves.append(node)
        if expected is not None:
            self.expected[node] = np.asarray(expected, dtype=np.float32)
        return node

    def scalar(self, value, like_shape):
        b, s, host = scalar_tensor(self.g, value, like_shape)
        self.inputs[s] = host
        return self.op(b)


def _ops_between(case, first_new_id):
    """All op nodes created since `first_new_id` (the kernel's subgraph)."""
    return [n["id"] for n in case.g.nodes if n["node"] == "op" and n["id"] >= first_new_id]


def tensor_ops_cases():
    cases = []

    c = Case("add_simple")  # tensor_ops.rs:18-26: f32 + bf16
    a = c.inp([50, 2], "f32", np.full(100, 2.0)); b = c.inp([50, 2], "bf16", np.full(100, 1.0))
    c.out(c.op(c.g.binary(a, b, "add")), np.full(100, 3.0)); cases.append(c)

    c = Case("add_with_broadcast")  # :28-36
    a = c.inp([5, 5], "f32", np.full(25, 3.0)); b = c.inp([1], "f32", [1.0])
    bb = c.op(broadcast_to(c.g, b, [1], [5, 5]))
    c.out(c.op(c.g.binary(a, bb, "add")), np.full(25, 4.0)); cases.append(c)

    c = Case("multiply")  # :38-46
    a = c.inp([50, 2], "f32", np.full(100, 2.0)); b = c.inp([50, 2], "bf16", np.full(100, 3.0))
    c.out(c.op(c.g.binary(a, b, "mul")), np.full(100, 6.0)); cases.append(c)

    c = Case("divide")  # :48-56
    a = c.inp([50, 2], "f32", np.full(100, 6.0)); b = c.inp([50, 2], "bf16", np.full(100, 2.0))
    r = c.op(c.g.unary(b, "recip"))
    c.out(c.op(c.g.binary(a, r, "mul")), np.full(100, 3.0)); cases.append(c)

    c = Case("multiply_by_scalar")  # :58-66
    a = c.inp([50, 2], "f32", np.full(100, 2.0))
    c.out(c.op(c.g.binary(a, c.scalar(3.0, [50, 2]), "mul")), np.full(100, 6.0)); cases.append(c)

    c = Case("divide_by_scalar")  # :68-76: x * (2.0f32).recip()
    a = c.inp([50, 2], "f32", np.full(100, 6.0))
    c.out(c.op(c.g.binary(a, c.scalar(np.float32(1.0) / np.float32(2.0), [50, 2]), "mul")), np.full(100, 3.0)); cases.append(c)

    c = Case("recip")  # :78-85
    a = c.inp([50, 2], "f32", np.full(100, 2.0))
    c.out(c.op(c.g.unary(a, "recip")), np.full(100, 0.5)); cases.append(c)

    c = Case("complex_operation_chain")  # :87-100: (a + b) * (c - d).recip() / 2 + a = 0.4 (epsilon 1e-6)
    a = c.inp([50, 2], "f32", np.full(100, 1.0)); b = c.inp([50, 2], "f32", np.full(100, 2.0))
    cc = c.inp([50, 2], "f32", np.full(100, 0.5)); d = c.inp([50, 2], "f32", np.full(100, 3.0))
    first = len(c.g.nodes)
    ab = c.g.binary(a, b, "add")
    cd = sub(c.g, cc, d)
    t = c.g.binary(ab, c.g.unary(cd, "recip"), "mul")
    half, s, host = scalar_tensor(c.g, np.float32(1.0) / np.float32(2.0), [50, 2]); c.inputs[s] = host
    t = c.g.binary(t, half, "mul")
    r = c.g.binary(t, a, "add")
    c.nodes = [n["id"] for n in c.g.nodes[first:] if n["node"] == "op"]
    c.out(r, np.full(100, 0.4)); cases.append(c)

    for name, fn, exp_all, exp_dim1 in [("reduce_sum", "sum", 1000.0, 40.0), ("reduce_mean", "mean", 10.0, 10.0)]:
        c = Case(name + "_all")  # :102-122
        x = c.inp([25, 4], "f32", np.full(100, 10.0))
        c.out(c.op(c.g.reduce(x, fn, 2)), [exp_all]); cases.append(c)
        c = Case(name + "_dim1")
        x = c.inp([25, 4], "f32", np.full(100, 10.0))
        c.out(c.op(c.g.reduce(x, fn, 1)), np.full(25, exp_dim1)); cases.append(c)

    seq = np.arange(1, 13, dtype=np.float32)
    for name, fn, exp_all, exp_dim1 in [("reduce_max", "max", 12.0, [4, 8, 12]), ("reduce_min", "min", 1.0, [1, 5, 9])]:
        c = Case(name + "_all")  # :124-155
        x = c.inp([3, 4], "f32", seq)
        c.out(c.op(c.g.reduce(x, fn, 2)), [exp_all]); cases.append(c)
        c = Case(name + "_dim1")
        x = c.inp([3, 4], "f32", seq)
        c.out(c.op(c.g.reduce(x, fn, 1)), exp_dim1); cases.append(c)

    big = np.concatenate([np.full(100_000, 1.0), np.full(100_000, 2.0)])
    c = Case("reduce_large_all")  # :157-170
    x = c.inp([2, 1000, 100], "f32", big)
    c.out(c.op(c.g.reduce(x, "sum", 3)), [300_000.0]); cases.append(c)
    c = Case("reduce_large_partial")
    x = c.inp([2, 1000, 100], "f32", big)
    c.out(c.op(c.g.reduce(x, "sum", 2)), [100_000.0, 200_000.0]); cases.append(c)

    c = Case("broadcast")  # :320-332
    x = c.inp([2, 1], "f32", [1.0, 2.0])
    c.out(c.op(broadcast_to(c.g, x, [2, 1], [2, 2, 4])),
          [1, 1, 1, 1, 2, 2, 2, 2, 1, 1, 1, 1, 2, 2, 2, 2]); cases.append(c)

    c = Case("reshape")  # :334-341
    x = c.inp([4], "f32", [1, 2, 3, 4])
    c.out(c.op(c.g.reshape(x, [2, 2])), [1, 2, 3, 4]); cases.append(c)

    c = Case("transpose_pointwise_path")  # :343-358: small tensors swap through the pointwise kernel
    x = c.inp([2, 2, 3], "f32", np.arange(1, 13))
    c.out(c.op(c.g.swap_dims(x, 1, 2)), [1, 4, 2, 5, 3, 6, 7, 10, 8, 11, 9, 12]); cases.append(c)

    c = Case("swap_dims_4d_pointwise_path")  # :360-376
    x = c.inp([2, 2, 2, 2], "f32", np.arange(1, 17))
    c.out(c.op(c.g.swap_dims(x, 1, 2)), [1, 2, 5, 6, 3, 4, 7, 8, 9, 10, 13, 14, 11, 12, 15, 16]); cases.append(c)

    c = Case("relu")  # :399-403
    x = c.inp([4], "f32", [-1.0, -0.5, 1.0, 0.0])
    c.out(c.op(c.g.unary(x, "relu")), [0, 0, 1, 0]); cases.append(c)

    c = Case("constant_f32")  # :474-484
    c.out(c.op(c.g.constant(10.0, "f32", [10, 20])), np.full(200, 10.0)); cases.append(c)

    c = Case("max_with_constant")  # :486-494
    k = c.op(c.g.constant(-1.0, "f32", [3])); b = c.inp([3], "f32", [-3.0, -1.0, 2.0])
    c.out(c.op(c.g.binary(k, b, "max")), [-1, -1, 2]); cases.append(c)

    c = Case("min_with_constant")  # :496-503
    k = c.op(c.g.constant(-1.0, "f32", [3])); b = c.inp([3], "f32", [-3.0, -1.0, 2.0])
    c.out(c.op(c.g.binary(k, b, "min")), [-3, -1, -1]); cases.append(c)
    return cases


def generated_cases():
    """Cases with seeded random data that exercise what the known-answer cases leave open."""
    cases = []
    rng = np.random.default_rng(1234)

    c = Case("snapshot_graph_pow_cos")  # the graph of pointwise/jit.rs:938-989, with a second output of equal size
    a = c.inp([5, 10, 10], "bf16", rng.uniform(0.1, 2.0, 500)); b = c.inp([1, 10], "f16", rng.uniform(-2, 2, 10))
    bb = c.op(c.g.broadcast(b, 3, [(0, 5), (1, 10)]))
    c.out(c.op(c.g.binary(a, bb, "pow")))
    c.out(c.op(c.g.unary(bb, "cos"))); cases.append(c)

    for fn, lo, hi in [("exp", -10, 10), ("sin", -20, 20), ("cos", -20, 20), ("tan", -1.5, 1.5), ("sigmoid", -20, 20),
                       ("tanh", -10, 10), ("sqrt", 0, 100), ("log", 1e-6, 100), ("recip", -4, 4), ("neg", -4, 4)]:
        c = Case(f"unary_{fn}_f32")
        x = c.inp([37, 129], "f32", rng.uniform(lo, hi, 37 * 129))
        c.out(c.op(c.g.unary(x, fn))); cases.append(c)

    c = Case("relu_backward_compare_select_cast")  # helium/src/tensor.rs:374-387
    x = c.inp([16, 48], "bf16", rng.standard_normal(16 * 48)); flow = c.inp([16, 48], "bf16", rng.standard_normal(16 * 48))
    zero = c.op(c.g.constant(0.0, "bf16", [16, 48]))
    mask = c.op(c.g.compare(x, zero, "gt"))
    c.out(c.op(c.g.select(zero, flow, mask)))
    c.out(c.op(c.g.change_data_type(mask, "f32")))
    c.out(mask); cases.append(c)

    c = Case("bool_input_and_logic")
    p = c.inp([7, 45], "bool", rng.integers(0, 2, 7 * 45)); q = c.inp([7, 45], "bool", rng.integers(0, 2, 7 * 45))
    c.out(c.op(c.g.binary(p, q, "xor")))
    c.out(c.op(c.g.change_data_type(c.op(c.g.binary(p, q, "and")), "u32"))); cases.append(c)

    c = Case("u32_arithmetic")
    p = c.inp([33, 20], "u32", rng.integers(0, 1000, 660)); q = c.inp([33, 20], "u32", rng.integers(0, 1000, 660))
    c.out(c.op(c.g.binary(c.op(c.g.binary(p, q, "mul")), q, "add")))
    c.out(c.op(c.g.change_data_type(c.op(c.g.binary(p, q, "max")), "f32"))); cases.append(c)

    c = Case("mixed_dtypes_and_two_reductions")  # every reduction of a kernel shares input shape and depth
    x = c.inp([6, 40, 24], "bf16", rng.standard_normal(6 * 40 * 24)); y = c.inp([6, 40, 24], "f16", rng.standard_normal(6 * 40 * 24))
    s = c.op(c.g.binary(x, y, "mul"))
    c.out(c.op(c.g.reduce(s, "sum", 2)))
    c.out(c.op(c.g.reduce(c.op(c.g.unary(s, "tanh")), "max", 2)))
    c.out(c.op(c.g.change_data_type(s, "f16")))
    c.reduce_rel = 1e-3; cases.append(c)

    for depth in (1, 2, 3, 4):
        c = Case(f"reduce_mean_depth{depth}_rank4")
        x = c.inp([3, 5, 7, 44], "f32", rng.uniform(-1, 1, 3 * 5 * 7 * 44))
        c.out(c.op(c.g.reduce(x, "mean", depth))); c.reduce_rel = 1e-3; cases.append(c)
        c = Case(f"reduce_min_depth{depth}_rank4")
        x = c.inp([3, 5, 7, 44], "f32", rng.uniform(-1, 1, 3 * 5 * 7 * 44))
        c.out(c.op(c.g.reduce(x, "min", depth))); cases.append(c)

    c = Case("wide_rows_sum")  # more columns than one block spans: partial rows meet in atomics
    x = c.inp([3, 5000], "f32", rng.uniform(-1, 1, 15000))
    c.out(c.op(c.g.reduce(x, "sum", 1))); c.reduce_rel = 1e-3; cases.append(c)

    c = Case("broadcast_bias_rows_and_cols")
    x = c.inp([4, 33, 40], "f32", rng.standard_normal(4 * 33 * 40))
    bias_r = c.inp([33, 1], "f32", rng.standard_normal(33)); bias_c = c.inp([40], "bf16", rng.standard_normal(40))
    br = c.op(broadcast_to(c.g, bias_r, [33, 1], [4, 33, 40])); bc = c.op(broadcast_to(c.g, bias_c, [40], [4, 33, 40]))
    c.out(c.op(c.g.unary(c.op(c.g.binary(c.op(c.g.binary(x, br, "add")), bc, "mul")), "relu"))); cases.append(c)

    c = Case("swap_then_pointwise")  # one SwapDims may join a pointwise kernel (pointwise.rs:156-162)
    x = c.inp([6, 10, 12], "f32", rng.standard_normal(720)); y = c.inp([6, 12, 10], "f32", rng.standard_normal(720))
    c.out(c.op(c.g.binary(c.op(c.g.swap_dims(x, 1, 2)), y, "add"))); cases.append(c)

    c = Case("reshape_between_swaps_generic_index_chain")
    x = c.inp([4, 6, 5], "f32", rng.standard_normal(120))
    r = c.op(c.g.reshape(c.op(c.g.swap_dims(x, 0, 2)), [10, 12]))
    c.out(c.op(c.g.unary(c.op(c.g.swap_dims(r, 0, 1)), "neg")))
    c.admitted_by_fusion_rule = False  # two SwapDims: the rule stops at one, the generator does not need to
    cases.append(c)

    c = Case("broadcast_after_reshape")
    x = c.inp([6], "f32", rng.standard_normal(6))
    r = c.op(c.g.reshape(x, [2, 3, 1]))
    c.out(c.op(c.g.broadcast(r, 4, [(3, 5), (0, 4)]))); cases.append(c)

    c = Case("odd_inner_extent_scalar_path")
    x = c.inp([9, 7], "bf16", rng.standard_normal(63)); y = c.inp([9, 7], "bf16", rng.standard_normal(63))
    c.out(c.op(c.g.binary(x, y, "max"))); cases.append(c)

    c = Case("rank1_large")
    x = c.inp([70_001], "f32", rng.standard_normal(70_001))
    c.out(c.op(c.g.unary(x, "sigmoid")))
    cases.append(c)
    # (the reordering starts at 1M elements; the override applies it to shapes the emulation can afford)
    FOLD_SMALL = {"HELIUM_HIP_FOLD_COLUMNS_MIN": "0"}
    # Reductions over leading dims arrive as SwapDims + Reduce; the kernel reorders its iteration space so that the
    # untransposed operand is walked in memory order and rows (and part of the batch index) fold per column.
    c = Case("batch_norm_statistics_nhwc"); c.env = FOLD_SMALL  # helium/src/modules/batch_norm.rs:38-46
    x = c.inp([3, 5, 4, 32], "bf16", rng.standard_normal(3 * 5 * 4 * 32))
    xt = c.op(c.g.swap_dims(x, 0, 3))
    two = c.inp([1], "f32", [2.0])
    c.out(c.op(c.g.reduce(xt, "mean", 3)))
    c.out(c.op(c.g.reduce(c.op(c.g.binary(xt, c.op(c.g.broadcast(two, 4, [(3, 3), (0, 32), (1, 5), (2, 4)])), "pow")), "mean", 3)))
    c.reduce_rel = 1e-3; cases.append(c)

    c = Case("column_sum_via_swap"); c.env = FOLD_SMALL
    x = c.inp([300, 48], "f32", rng.standard_normal(300 * 48))
    c.out(c.op(c.g.reduce(c.op(c.g.swap_dims(x, 0, 1)), "sum", 1))); c.reduce_rel = 1e-3; cases.append(c)

    c = Case("fold_middle_dim_keep_two"); c.env = FOLD_SMALL  # [P,Q,R] -> [P,R,Q], fold Q: outputs [P,R], R contiguous
    x = c.inp([5, 70, 40], "f32", rng.standard_normal(5 * 70 * 40))
    c.out(c.op(c.g.reduce(c.op(c.g.swap_dims(x, 1, 2)), "max", 1))); cases.append(c)

    c = Case("fold_two_dims_keep_two"); c.env = FOLD_SMALL  # [A,B,C,D] -> [A,D,C,B], fold C and B: they merge into one row dim
    x = c.inp([3, 6, 9, 32], "f32", rng.standard_normal(3 * 6 * 9 * 32))
    c.out(c.op(c.g.reduce(c.op(c.g.swap_dims(x, 1, 3)), "sum", 2))); c.reduce_rel = 1e-3; cases.append(c)

    c = Case("fold_leading_dims_second_operand_blocks_merge"); c.env = FOLD_SMALL  # the batch index keeps a folded dim (b_div > 1)
    x = c.inp([6, 5, 4, 32], "f32", rng.standard_normal(6 * 5 * 4 * 32)); y = c.inp([32, 5, 4, 6], "f32", rng.standard_normal(6 * 5 * 4 * 32))
    c.out(c.op(c.g.reduce(c.op(c.g.binary(c.op(c.g.swap_dims(x, 0, 3)), y, "mul")), "sum", 3))); c.reduce_rel = 1e-3; cases.append(c)

    # A full-size output next to reductions over its leading dims (the input gradient of a batch norm and the channel
    # sums of the next one): the untransposed tensor is written through the same walk, in memory order.
    c = Case("full_size_output_next_to_channel_sums"); c.env = FOLD_SMALL; c.admitted_by_fusion_rule = False
    x = c.inp([3, 5, 4, 32], "f32", rng.standard_normal(3 * 5 * 4 * 32)); sc = c.inp([32], "f32", rng.uniform(0.5, 2.0, 32))
    y = c.op(c.g.unary(c.op(c.g.binary(x, c.op(c.g.broadcast(sc, 4, [(0, 3), (1, 5), (2, 4)])), "mul")), "relu"))
    yt = c.op(c.g.swap_dims(y, 0, 3))
    c.out(y)
    c.out(c.op(c.g.reduce(yt, "sum", 3)))
    c.out(c.op(c.g.reduce(c.op(c.g.binary(yt, c.op(c.g.swap_dims(x, 0, 3)), "mul")), "sum", 3)))
    c.reduce_rel = 1e-3; cases.append(c)

    # 16-bit activations seen as [rows, channels] next to f32 per-channel vectors (a batch norm's backward pass): the
    # per-channel operands are loaded once ahead of the rows; with few expressions two rows are in flight.
    TALL = dict(FOLD_SMALL, HELIUM_HIP_POINTWISE_RPT="2")
    c = Case("channel_vectors_hoisted_two_rows_in_flight"); c.env = TALL; c.admitted_by_fusion_rule = False
    x = c.inp([1100, 64], "bf16", rng.standard_normal(1100 * 64)); sc = c.inp([64], "f32", rng.uniform(0.5, 2.0, 64))
    sh = c.inp([64], "f32", rng.standard_normal(64))
    bc = lambda v: c.op(c.g.broadcast(v, 2, [(0, 1100)]))
    y = c.op(c.g.unary(c.op(c.g.binary(c.op(c.g.binary(x, bc(sc), "mul")), bc(sh), "add")), "relu"))
    c.out(c.op(c.g.change_data_type(y, "bf16")))
    c.out(c.op(c.g.reduce(c.op(c.g.swap_dims(y, 0, 1)), "sum", 1)))
    c.reduce_rel = 1e-3; cases.append(c)

    # The same with more than 24 expressions: one row is in flight and the next row's raw vectors are requested ahead of
    # its arithmetic.
    c = Case("many_expressions_rows_requested_ahead"); c.env = TALL; c.admitted_by_fusion_rule = False
    x = c.inp([1100, 64], "bf16", rng.standard_normal(1100 * 64)); f = c.inp([1100, 64], "bf16", rng.standard_normal(1100 * 64))
    sc = c.inp([64], "f32", rng.uniform(0.5, 2.0, 64)); sh = c.inp([64], "f32", rng.standard_normal(64))
    var = c.inp([64], "f32", rng.uniform(0.5, 2.0, 64))
    bc = lambda v: c.op(c.g.broadcast(v, 2, [(0, 1100)]))
    inv = c.op(c.g.unary(c.op(c.g.unary(c.op(c.g.binary(bc(var), c.scalar(1e-3, [1100, 64]), "add")), "sqrt")), "recip"))  # the same in every row
    xh = c.op(c.g.binary(c.op(c.g.binary(x, bc(sh), "add")), inv, "mul"))
    y = c.op(c.g.binary(c.op(c.g.binary(xh, bc(sc), "mul")), bc(sh), "add"))
    zero = c.op(c.g.constant(0.0, "f32", [1100, 64]))
    mask = c.op(c.g.compare(y, zero, "gt"))
    g1 = c.op(c.g.select(zero, f, mask))
    t = g1
    for fn in ("tanh", "neg", "sigmoid", "neg", "relu", "neg", "tanh", "neg"):
        t = c.op(c.g.binary(c.op(c.g.unary(t, fn)), g1, "add"))
    dx = c.op(c.g.binary(c.op(c.g.binary(t, bc(sc), "mul")), inv, "mul"))
    c.out(c.op(c.g.change_data_type(dx, "bf16")))
    c.out(c.op(c.g.change_data_type(mask, "bf16")))
    c.out(c.op(c.g.reduce(c.op(c.g.swap_dims(t, 0, 1)), "sum", 1)))
    c.out(c.op(c.g.reduce(c.op(c.g.swap_dims(c.op(c.g.binary(t, xh, "mul")), 0, 1)), "sum", 1)))
    c.reduce_rel = 1e-3; cases.append(c)

    # A mean over few rows per batch entry (global average pooling: 7 x 7 pixels per image and channel): a block spans
    # all 49 rows, so the kernel writes the means itself - no partial results, no second launch.
    c = Case("pooling_rows_fit_one_block"); c.env = FOLD_SMALL
    x = c.inp([64, 49, 1000], "f32", rng.standard_normal(64 * 49 * 1000))
    c.out(c.op(c.g.reduce(c.op(c.g.swap_dims(x, 1, 2)), "mean", 1))); c.reduce_rel = 1e-3
    c.describes = "grid=256 threads=256 exprs=1 outs=1 ws_floats=0 ws_counters=0 finalize_grid=0"; cases.append(c)

    # Rows that a block spans with four (two) waves: the waves' parts of a row meet in LDS, nothing is accumulated with
    # atomics and nothing has to be filled ahead of the launch (a softmax over 1000 classes).
    for rows, cols, tx in ((37, 1000, 256), (9, 500, 128)):
        c = Case(f"rows_spanning_{tx // 64}_waves")
        x = c.inp([rows, cols], "f32", rng.standard_normal(rows * cols))
        c.out(c.op(c.g.reduce(x, "max", 1)))
        c.out(c.op(c.g.reduce(c.op(c.g.unary(x, "exp")), "sum", 1))); c.reduce_rel = 1e-4
        c.describes = f" TX={tx} TY={256 // tx} RPT=1 grid={(rows + 256 // tx - 1) // (256 // tx)} threads=256 exprs=2 outs=2 ws_floats=0 ws_counters=0 finalize_grid=0 fills=[]"
        cases.append(c)

    return cases


def all_cases():
    return tensor_ops_cases() + generated_cases()
