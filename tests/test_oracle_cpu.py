"""Pins of the CPU oracle itself (no GPU): every function of `oracle/` that a GPU parity test trusts is checked here
against something the oracle did not produce - the vectors the reference's own tests hold (tests/golden/*.json), brute
force written in another form (scalar loops over output elements where the oracle is vectorised over taps), identities
the mathematics fixes (a gradient is the adjoint of its forward map), Python's `math` module for the scalar functions,
and hand-derived closed forms of the README graph. A dropped term, a wrong sign or index, a mirrored operand fails
at least one of them."""
import itertools
import math

import numpy as np
import pytest

from helium_amd import configs
from oracle import fusion_ir as oracle_fir
from oracle import helium_ir as oracle_ir
from oracle import numerics as nm

import reference_cases as rc


# ---- convolution --------------------------------------------------------------------------------------------------
def naive_conv(x, w, stride, dilation, pad, out_hw):
    """Seven nested loops, one output element at a time, float64 (cross-correlation, zero padding)."""
    n, h, wd, c = x.shape
    o, kr, ks, _ = w.shape
    out = np.zeros((n, out_hw[0], out_hw[1], o))
    for b in range(n):
        for p in range(out_hw[0]):
            for q in range(out_hw[1]):
                for k in range(o):
                    acc = 0.0
                    for r in range(kr):
                        for s in range(ks):
                            ih = p * stride[0] + r * dilation[0] - pad[0]
                            iw = q * stride[1] + s * dilation[1] - pad[1]
                            if 0 <= ih < h and 0 <= iw < wd:
                                for ch in range(c):
                                    acc += float(x[b, ih, iw, ch]) * float(w[k, r, s, ch])
                    out[b, p, q, k] = acc
    return out


CONV_GRID = [dict(kernel_size=list(k), stride=list(s), dilation=list(d), padding_mode=m)
             for k in ((3, 3), (1, 1), (3, 2), (5, 3)) for s in ((1, 1), (2, 2), (3, 1)) for d in ((1, 1), (2, 1), (2, 2))
             for m in ("same", "valid", "full")]


def test_conv_output_size_known_answers():
    """Conv2dParams::compute_output_size (helium-ir/src/opgraph/op/conv.rs:51-73), answers worked out by hand:
    Full adds kernel/2, Valid takes kernel/2 away (never below zero), then the stride divides, rounding down."""
    table = [  # mode, input, kernel, stride -> output
        ("same", (7, 9), (3, 3), (1, 1), [7, 9]), ("same", (7, 9), (3, 3), (2, 2), [3, 4]),
        ("same", (8, 8), (7, 7), (2, 2), [4, 4]), ("valid", (7, 9), (3, 3), (1, 1), [6, 8]),
        ("valid", (7, 9), (5, 3), (2, 2), [2, 4]), ("valid", (1, 2), (5, 7), (1, 1), [0, 0]),
        ("full", (7, 9), (3, 3), (1, 1), [8, 10]), ("full", (7, 9), (5, 2), (3, 2), [3, 5]),
        ("same", (256, 256), (7, 7), (2, 2), [128, 128]), ("full", (4, 4), (1, 1), (1, 1), [4, 4]),
    ]
    for mode, size, kernel, stride, want in table:
        assert oracle_ir.conv_output_size({"padding_mode": mode, "stride": stride}, size, kernel) == want
    # PaddingMode::compute_padding_amount (conv.rs:85-91)
    assert oracle_ir.conv_padding({"kernel_size": [5, 3], "padding_mode": "same"}) == [2, 1]
    assert oracle_ir.conv_padding({"kernel_size": [5, 3], "padding_mode": "valid"}) == [0, 0]
    assert oracle_ir.conv_padding({"kernel_size": [5, 3], "padding_mode": "full"}) == [4, 2]


def test_conv_matches_the_reference_known_answer():
    """conv_simple (helium/tests/tensor_ops.rs:379-397): pins NHWC x KRSC layout and which operand index is summed."""
    case = rc.TENSOR_OPS["conv"][0]
    x = np.array(case["image"], dtype=np.float32).reshape(case["image_shape"])
    w = np.array(case["filter"], dtype=np.float32).reshape(case["filter_shape"])
    got = oracle_ir.conv(x, w, case["params"], "f32")
    assert list(got.shape) == case["expected_shape"]
    assert np.array_equal(got.reshape(-1), np.array(case["expected"], dtype=np.float32))
    # the same through the recorded graph (Reshape + Conv) and the graph evaluator
    G, raw = rc.record_conv(case)
    assert np.array_equal(rc.evaluate_on_oracle(G, {"y": raw})["y"], np.array(case["expected"], dtype=np.float32))


@pytest.mark.parametrize("params", CONV_GRID, ids=lambda p: f"k{p['kernel_size']}s{p['stride']}d{p['dilation']}{p['padding_mode']}".replace(" ", ""))
def test_conv_and_its_gradients_against_brute_force(params):
    rng = np.random.default_rng(hash(str(params)) % 2**32)
    params = dict(params, in_channels=3, out_channels=2)
    x = rng.integers(-4, 5, (2, 7, 6, 3)).astype(np.float32)
    w = rng.integers(-3, 4, (2, *params["kernel_size"], 3)).astype(np.float32)
    out_hw = oracle_ir.conv_output_size(params, (7, 6), params["kernel_size"])
    pad = oracle_ir.conv_padding(params)
    want = naive_conv(x, w, params["stride"], params["dilation"], pad, out_hw)
    got = oracle_ir.conv(x, w, params, "f32")
    assert got.shape == want.shape
    assert np.array_equal(got.astype(np.float64), want)  # small integers: exact in both
    if 0 in out_hw:
        return
    # the gradients, as scatter loops over the forward op's products
    dy = rng.integers(-3, 4, want.shape).astype(np.float32)
    dx = np.zeros(x.shape)
    dw = np.zeros(w.shape)
    for b, p, q, k, r, s in itertools.product(range(2), range(out_hw[0]), range(out_hw[1]), range(2),
                                              range(w.shape[1]), range(w.shape[2])):
        ih = p * params["stride"][0] + r * params["dilation"][0] - pad[0]
        iw = q * params["stride"][1] + s * params["dilation"][1] - pad[1]
        if 0 <= ih < 7 and 0 <= iw < 6:
            dx[b, ih, iw, :] += float(dy[b, p, q, k]) * w[k, r, s, :]
            dw[k, r, s, :] += float(dy[b, p, q, k]) * x[b, ih, iw, :]
    assert np.array_equal(oracle_ir.conv_backward_data(dy, w, params, [7, 6]).astype(np.float64), dx)
    assert np.array_equal(oracle_ir.conv_backward_filter(dy, x, params).astype(np.float64), dw)


@pytest.mark.parametrize("mode", ["same", "valid", "full"])
@pytest.mark.parametrize("stride,dilation", [((1, 1), (1, 1)), ((2, 2), (1, 1)), ((1, 2), (2, 1)), ((3, 3), (2, 2))])
def test_conv_gradients_are_the_adjoints_of_the_forward_map(mode, stride, dilation):
    """<conv(x, w), dy> = <x, backward_data(dy, w)> = <w, backward_filter(dy, x)> for random real operands."""
    rng = np.random.default_rng(3)
    params = dict(in_channels=5, out_channels=4, kernel_size=[3, 5], stride=list(stride), dilation=list(dilation),
                  padding_mode=mode)
    x = rng.standard_normal((3, 11, 13, 5)).astype(np.float32)
    w = rng.standard_normal((4, 3, 5, 5)).astype(np.float32)
    y = oracle_ir.conv(x, w, params, "f32").astype(np.float64)
    dy = rng.standard_normal(y.shape).astype(np.float32)
    lhs = float((y * dy).sum())
    dx = oracle_ir.conv_backward_data(dy, w, params, [11, 13]).astype(np.float64)
    dw = oracle_ir.conv_backward_filter(dy, x, params).astype(np.float64)
    assert dx.shape == x.shape and dw.shape == w.shape
    scale = float(np.abs(y * dy).sum()) + 1e-12
    assert abs(lhs - float((dx * x).sum())) <= 1e-5 * scale
    assert abs(lhs - float((dw * w).sum())) <= 1e-5 * scale


# ---- the reference's autodiff / loss / matmul vectors through the graph evaluator ---------------------------------
@pytest.mark.parametrize("case", rc.AUTODIFF, ids=lambda c: c["name"])
def test_oracle_reproduces_the_reference_autodiff_and_loss_vectors(case):
    """helium/tests/autodiff.rs, helium/tests/loss.rs. These graphs go through Compare, Select, Bool -> float casts,
    Broadcast, SwapDims, Reduce (sum / mean / min / max), Reshape, Constant, Pow, Log, Max: a mirrored Select or a
    wrong comparison direction gives a wrong gradient (relu: [1, 0, 5, -10])."""
    G, raws = rc.record_autodiff(case)
    got = rc.evaluate_on_oracle(G, raws)
    for k, want in case["expected"].items():
        want = np.array(want, dtype=np.float32)
        if case.get("exact"):
            assert np.array_equal(got[k], want), (case["name"], k, got[k])
        else:
            assert nm.ulps_close(got[k], want, max_ulps=4).all(), (case["name"], k, got[k], want)


def test_oracle_gradient_descent_converges_on_the_square_root():
    """basic_gradient_descent (autodiff.rs:121-145): one graph per iteration, until sqrt(error) < 1e-3."""
    guess = 1.0
    for _ in range(2000):
        G, error, new_guess = rc.gradient_descent_step(guess)
        got = rc.evaluate_on_oracle(G, {"error": error, "guess": new_guess})
        if math.sqrt(float(got["error"][0])) < 1e-3:
            break
        guess = float(got["guess"][0])
    else:
        pytest.fail("did not converge")
    assert abs(guess - math.sqrt(1001.0)) < 1e-4


@pytest.mark.parametrize("case", rc.TENSOR_OPS["matmul"], ids=lambda c: c["name"])
def test_oracle_reproduces_the_reference_matmul_vectors(case):
    """helium/tests/tensor_ops.rs:172-318: pins operand order, the transposes around a product, batching."""
    G, raw, expected = rc.record_matmul(case)
    got = rc.evaluate_on_oracle(G, {"y": raw})["y"]
    if "expected_shape" in case:
        assert raw.shape == case["expected_shape"]
    assert nm.ulps_close(got, expected, max_ulps=4, epsilon=case["epsilon"]).all(), (got, expected)


def test_compare_select_and_casts_one_element_at_a_time():
    """Compare (op.rs:429-437), Select = rhs where the selector is true (op.rs:439-445, jit.rs:397-400), casts between
    classes (jit.rs:477-485: float -> bool is `!= 0`, bool -> float is 1 / 0), against plain Python."""
    a = np.array([-2.0, -0.0, 0.0, 0.5, 3.0, np.nan], dtype=np.float32)
    b = np.array([-2.0, 0.0, 1.0, 0.25, 3.0, 1.0], dtype=np.float32)
    py = {"eq": lambda x, y: x == y, "ne": lambda x, y: x != y, "lt": lambda x, y: x < y, "le": lambda x, y: x <= y,
          "gt": lambda x, y: x > y, "ge": lambda x, y: x >= y}
    for fn, f in py.items():
        assert oracle_ir.compare(fn, a, b).tolist() == [f(float(x), float(y)) for x, y in zip(a, b)], fn
    nodes = [{"id": 0, "node": "input", "shape": [6], "dtype": "f32"}, {"id": 1, "node": "input", "shape": [6], "dtype": "f32"},
             {"id": 2, "node": "op", "op": "compare", "fn": "lt", "inputs": [0, 1]},
             {"id": 3, "node": "op", "op": "select", "inputs": [0, 1, 2]},
             {"id": 4, "node": "op", "op": "change_dtype", "target": "f32", "inputs": [2]},
             {"id": 5, "node": "op", "op": "change_dtype", "target": "bool", "inputs": [0]},
             {"id": 6, "node": "op", "op": "change_dtype", "target": "u32", "inputs": [1]},
             {"id": 7, "node": "op", "op": "change_dtype", "target": "f32", "inputs": [6]}]
    val, desc = oracle_ir.evaluate(nodes, {0: a, 1: b})
    lt = [float(x) < float(y) for x, y in zip(a, b)]
    want_select = [float(y) if s else float(x) for x, y, s in zip(a, b, lt)]
    assert np.array_equal(val[3], np.array(want_select, dtype=np.float32), equal_nan=True)
    assert val[4].tolist() == [1.0 if s else 0.0 for s in lt] and desc[4][1] == "f32"
    assert val[5].tolist() == [float(x) != 0.0 for x in a] and desc[5][1] == "bool"
    assert val[6].tolist() == [0, 0, 1, 0, 3, 1] and val[7].tolist() == [0.0, 0.0, 1.0, 0.0, 3.0, 1.0]
    # Bool storage: bit i of word i / 32, least significant bit first (helium-ir/src/data_type.rs:159-167)
    bits = [True, False, True] + [False] * 30 + [True]
    assert nm.pack_bool(bits).tolist() == [0b101, 0b10]
    assert nm.unpack_bool(np.array([0b101, 0b10], dtype=np.uint32), 34).tolist() == bits


def test_helium_ir_scalar_functions_against_the_math_module():
    xs = np.array([-3.5, -1.0, -0.25, 0.0, 0.25, 1.0, 2.75, 9.0], dtype=np.float32)
    py = {"recip": lambda v: 1.0 / v if v != 0 else math.copysign(math.inf, v), "neg": lambda v: -v, "exp": math.exp,
          "sin": math.sin, "cos": math.cos, "tan": math.tan, "sigmoid": lambda v: 1.0 / (1.0 + math.exp(-v)),
          "tanh": math.tanh, "relu": lambda v: max(v, 0.0), "sqrt": lambda v: math.sqrt(v) if v >= 0 else math.nan,
          "log": lambda v: math.log(v) if v > 0 else (-math.inf if v == 0 else math.nan)}
    for fn, f in py.items():
        got = oracle_ir.unary(fn, xs)
        want = np.array([f(float(v)) for v in xs], dtype=np.float64).astype(np.float32)
        assert nm.ulps_close(got, want, max_ulps=1).all(), (fn, got, want)
    a = np.array([0.5, 2.0, 3.0, 1.5], dtype=np.float32)
    b = np.array([2.0, -1.0, 0.5, 1.5], dtype=np.float32)
    pyb = {"add": lambda x, y: x + y, "mul": lambda x, y: x * y, "pow": math.pow, "min": min, "max": max}
    for fn, f in pyb.items():
        want = np.array([f(float(x), float(y)) for x, y in zip(a, b)]).astype(np.float32)
        assert nm.ulps_close(oracle_ir.binary(fn, a, b), want, max_ulps=1).all(), fn
    t, f_ = np.array([True, True, False, False]), np.array([True, False, True, False])
    assert oracle_ir.binary("and", t, f_).tolist() == [True, False, False, False]
    assert oracle_ir.binary("or", t, f_).tolist() == [True, True, True, False]
    assert oracle_ir.binary("xor", t, f_).tolist() == [False, True, True, False]


def test_helium_ir_reduce_folds_the_trailing_dims():
    """op.rs:338-367 / jit.rs:402-458, against Python loops; the reference's own vectors are in pointwise_cases."""
    rng = np.random.default_rng(9)
    x = rng.standard_normal((3, 4, 5)).astype(np.float32)
    for depth in (1, 2, 3):
        keep = x.shape[: 3 - depth]
        for fn, f in (("sum", sum), ("max", max), ("min", min), ("mean", lambda v: sum(v) / len(v))):
            got = oracle_ir.reduce(fn, x, depth)
            assert list(got.shape) == list(keep) + [1]
            flat = x.reshape(keep + (-1,)).astype(np.float64)
            want = np.array([f([float(v) for v in flat[idx]]) for idx in np.ndindex(*keep)]).reshape(keep + (1,))
            assert np.allclose(got, want, rtol=1e-6, atol=1e-6), (fn, depth)


def test_bf16_rounding_is_round_to_nearest_even():
    """`half` crate semantics: ties go to the even mantissa; NaN stays NaN."""
    f = lambda bits: np.array([bits], dtype=np.uint32).view(np.float32)  # noqa: E731
    assert nm.f32_to_bf16_bits(f(0x3F808000))[0] == 0x3F80  # tie, even below
    assert nm.f32_to_bf16_bits(f(0x3F818000))[0] == 0x3F82  # tie, even above
    assert nm.f32_to_bf16_bits(f(0x3F808001))[0] == 0x3F81
    assert nm.f32_to_bf16_bits(f(0x7F7FFFFF))[0] == 0x7F80  # rounds up to infinity
    assert np.isnan(nm.bf16_bits_to_f32(nm.f32_to_bf16_bits(np.array([np.nan], dtype=np.float32))))[0]
    assert nm.bf16_bits_to_f32(np.array([0x3FC0], dtype=np.uint16))[0] == 1.5


# ---- fusion IR ----------------------------------------------------------------------------------------------------
def test_fusion_ir_scalar_functions_against_the_math_module():
    """helium-playground/src/opgraph.rs:317-338 with the meanings of torch_synthesizer.rs:30-84."""
    xs = np.array([-2.5, -1.0, -0.5, 0.0, 0.5, 1.0, 3.25], dtype=np.float32)
    c = 1.75
    py = {"neg": lambda v: -v, "relu": lambda v: max(v, 0.0),
          "gelu": lambda v: 0.5 * v * (1.0 + math.erf(v / math.sqrt(2.0))), "tanh": math.tanh, "exp": math.exp,
          "ln": lambda v: math.log(v) if v > 0 else (-math.inf if v == 0 else math.nan),
          "sqrt": lambda v: math.sqrt(v) if v >= 0 else math.nan, "add_constant": lambda v: v + c,
          "mul_constant": lambda v: v * c, "pow_constant": lambda v: math.pow(v, c) if v >= 0 else math.nan}
    for fn, f in py.items():
        got = oracle_fir.unary(fn, xs, c)
        want = np.array([f(float(v)) for v in xs], dtype=np.float64).astype(np.float32)
        assert nm.ulps_close(got, want, max_ulps=1).all(), (fn, got, want)
    assert np.array_equal(oracle_fir.unary("pow_constant", xs, 2.0), xs * xs)  # x*x (kernel_generator.rs:383-391)
    a = np.array([0.5, -2.0, 3.0, 1.5, -1.0], dtype=np.float32)
    b = np.array([2.0, -1.0, 0.0, 1.5, 4.0], dtype=np.float32)
    with np.errstate(all="ignore"):
        pyb = {"add": a + b, "sub": a - b, "mul": a * b, "div": a / b}
    for fn, want in pyb.items():
        assert np.array_equal(oracle_fir.binary(fn, a, b), want), fn
    assert nm.ulps_close(oracle_fir.binary("pow", np.abs(a), b), np.array([math.pow(abs(float(x)), float(y)) for x, y in zip(a, b)], dtype=np.float32), max_ulps=1).all()
    # Drelu(lhs, rhs) = rhs > 0 ? lhs : 0 (kernel_generator.rs:409-411, torch_synthesizer.rs:76-78)
    assert oracle_fir.binary("drelu", a, b).tolist() == [0.5, 0.0, 0.0, 1.5, -1.0]


def test_fusion_ir_reduction_depths_against_loops():
    """opgraph.rs:397-413: Rows -> [b,M,1], Columns -> [b,1,N], Item -> [b,1,1], Batch -> [1,1,1]."""
    rng = np.random.default_rng(4)
    x = rng.standard_normal((2, 3, 5)).astype(np.float32)
    rows = [[[sum(float(v) for v in x[b, m, :])] for m in range(3)] for b in range(2)]
    cols = [[[sum(float(x[b, m, n]) for m in range(3)) for n in range(5)]] for b in range(2)]
    item = [[[sum(float(v) for v in x[b].reshape(-1))]] for b in range(2)]
    batch = [[[sum(float(v) for v in x.reshape(-1))]]]
    for depth, want in (("rows", rows), ("columns", cols), ("item", item), ("batch", batch)):
        got = oracle_fir.reduction(depth, x)
        assert got.shape == np.array(want).shape, depth
        assert np.allclose(got, np.array(want), rtol=1e-6, atol=1e-6), depth
        node = {"op": "reduction", "x": 0, "depth": depth}
        assert oracle_fir.shape_of(node, {0: [2, 3, 5]}) == list(np.array(want).shape)
    assert oracle_fir.shape_of({"op": "broadcast", "x": 0, "axis": 1, "amount": 7}, {0: [2, 1, 5]}) == [2, 7, 5]
    assert oracle_fir.shape_of({"op": "transpose", "x": 0}, {0: [2, 3, 5]}) == [2, 5, 3]
    assert oracle_fir.shape_of({"op": "matmul", "a": 0, "b": 1}, {0: [2, 3, 5], 1: [2, 5, 4]}) == [2, 3, 4]


@pytest.mark.parametrize("mainloop", [False, True], ids=["epilogue", "mainloop_and_epilogue"])
def test_c4_graph_against_its_closed_forms(mainloop):
    """The README graph (README.md:33-79) evaluated by the oracle's graph walker equals the formulas it stands for,
    written directly in float64: z = relu(g12 + g13 + b6), c = tanh(g24 + g26 + b8), h = (1 - z) n9 + z c,
    L = sum (h - t)^2 / 4096, dh = 2 (h - t) / 4096, db8 = sum_rows z dh (1 - c^2), db6 = sum_rows [pre_z > 0] (dh c - dh n9)."""
    size = 48
    g, outs = configs.c4_graph(size, mainloop=mainloop, full_size_outputs=True)
    inputs = configs.c4_inputs(g, size)
    f = {k: nm.from_storage(v, "f32" if v.dtype == np.float32 else "bf16", v.shape).astype(np.float64) for k, v in inputs.items()}
    a = f[22] if mainloop else f[1]
    if mainloop:
        a = np.maximum(a, 0.0) * f[9]
        a = nm.bf16_bits_to_f32(nm.f32_to_bf16_bits(a.astype(np.float32))).astype(np.float64)  # sm80.rs:418-437
    g12 = a @ f[2]
    pre_z = g12 + f[13] + f[6]
    z = np.maximum(pre_z, 0.0)
    c = np.tanh(f[24] + f[26] + f[8])
    h = (1.0 - z) * f[9] + z * c
    d = h - f[11]
    inv = float(np.float32(0.00024414063))
    loss = (d * d * inv).sum()
    dh = d * 2.0 * inv
    dpre_c = z * dh * (1.0 - c * c)
    dpre_z = np.where(pre_z > 0, dh * c - dh * f[9], 0.0)
    got = oracle_fir.outputs(g.nodes, inputs, round_mainloop_to="bf16" if mainloop else None)
    val, _ = oracle_fir.evaluate(g.nodes, inputs, round_mainloop_to="bf16" if mainloop else None)
    assert np.allclose(val[39].reshape(()), loss, rtol=1e-5)
    assert np.allclose(val[58].reshape(-1), dpre_c.sum(axis=1).reshape(-1), rtol=1e-4, atol=1e-7)
    # an element whose pre-activation is within rounding of zero may fall on either side of Drelu's test
    near = np.abs(pre_z) < 1e-6
    assert np.allclose(np.where(near, 0, val[86]), np.where(near, 0, dpre_z), rtol=1e-4, atol=1e-8)
    assert np.allclose(val[57], dpre_c, rtol=1e-4, atol=1e-8)
    assert got[outs["loss"]].dtype == np.float32 and got[outs["dpre_c"]].dtype == np.uint16
    assert got[outs["db8"]].shape == (1, 1, size)


@pytest.mark.parametrize("mainloop", [False, True], ids=["epilogue", "mainloop_and_epilogue"])
@pytest.mark.parametrize("size", [40, 200])
def test_c_restatement_of_the_c4_fusion_against_closed_forms_and_the_numpy_oracle(size, mainloop):
    """oracle/c4_cpu.c (what bench.py times as the CPU baseline) against the same closed forms in float64 and against
    the graph walker; sizes that are no multiple of its row and column blocks."""
    from oracle import c4_cpu

    g, _ = configs.c4_graph(size, mainloop=mainloop)
    inputs = configs.c4_inputs(g, size)
    f = {k: nm.from_storage(v, "f32" if v.dtype == np.float32 else "bf16", v.shape).astype(np.float64) for k, v in inputs.items()}
    a = f[22] if mainloop else f[1]
    if mainloop:
        a = nm.bf16_bits_to_f32(nm.f32_to_bf16_bits((np.maximum(a, 0.0) * f[9]).astype(np.float32))).astype(np.float64)
    pre_z = a @ f[2] + f[13] + f[6]
    z, c = np.maximum(pre_z, 0.0), np.tanh(f[24] + f[26] + f[8])
    d = (1.0 - z) * f[9] + z * c - f[11]
    inv = float(np.float32(0.00024414063))
    dh = d * 2.0 * inv
    near = np.abs(pre_z) < 1e-5  # may fall on either side of Drelu's test
    want = {39: (d * d * inv).sum(), 58: (z * dh * (1.0 - c * c)).sum(axis=1).reshape(-1),
            87: np.where((pre_z > 0) & ~near, dh * c - dh * f[9], 0.0).sum(axis=1).reshape(-1)}
    got = c4_cpu.c4(inputs, size, mainloop=mainloop)
    slack = np.abs(np.where(near, dh * c - dh * f[9], 0.0)).sum(axis=1).reshape(-1)
    assert np.allclose(got[39][0], want[39], rtol=2e-5)
    assert np.allclose(got[58], want[58], rtol=1e-3, atol=1e-6 * np.abs(want[58]).max())
    assert np.all(np.abs(got[87] - want[87]) <= 1e-3 * np.abs(want[87]) + 1e-6 * np.abs(want[87]).max() + slack)
    walker = oracle_fir.outputs(g.nodes, inputs, round_mainloop_to="bf16" if mainloop else None)
    for k in (39, 58, 87):
        w = walker[k].reshape(-1).astype(np.float64)
        assert np.max(np.abs(got[k] - w)) <= 1e-5 * np.abs(w).max()
