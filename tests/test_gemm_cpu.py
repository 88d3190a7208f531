"""The generated fused-GEMM kernel run on the CPU (threads + barriers, MFMA and transposing-LDS-load stand-ins,
AddressSanitizer) against the oracle: index arithmetic, edge predication, mainloop and epilogue fusion."""
import os
import re

import numpy as np
import pytest

import helium_amd as ha
from oracle import fusion_ir as oracle
from oracle import numerics as nm

import gemm_cases
from cpu_emul import run_kernel


def launch_gemm(k, bufs):
    """Runs a fused-GEMM kernel object on the CPU as its host side launches it: `fused_matmul`, then, when the
    epilogue reduces, `fused_matmul_reduce` over the partial results the first launch parked in the workspace (which
    starts as NaN here, so a partial that no wave wrote shows). bufs: one (array, mode) per kernel argument.
    Returns the arrays of the output arguments, in argument order."""
    gx, gy = map(int, re.search(r"grid=(\d+)x(\d+)", k.description).groups())
    threads = int(re.search(r"threads=(\d+)", k.description).group(1))
    ws_floats, reduce_grid = map(int, re.search(r"reduce_ws=(\d+) reduce_grid=(\d+)", k.description).groups())
    counters = int(re.search(r"reduce_counters=(\d+)", k.description).group(1))
    if counters:
        # the reductions fold inside the kernel: the last workgroup to arrive at a counter adds the partials, and leaves
        # the counter at zero for the next launch
        assert not reduce_grid
        res = run_kernel(k.source, "fused_matmul", gx, threads,
                         bufs + [(np.full(ws_floats, np.nan, dtype=np.float32), 2), (np.zeros(counters, dtype=np.uint32), 2)], grid_y=gy)
        assert not res[-1].any(), "arrival counters are not back at zero"
        return res[:-2]
    if not reduce_grid:
        return run_kernel(k.source, "fused_matmul", gx, threads, bufs, grid_y=gy)
    res = run_kernel(k.source, "fused_matmul", gx, threads, bufs + [(np.full(ws_floats, np.nan, dtype=np.float32), 2)], grid_y=gy)
    ws, res = res[-1], res[:-1]
    out_args = [i for i, a in enumerate(k.args) if a["is_output"]]
    # the reduce launch takes the kernel arguments the description lists, in that order: the reduction outputs, or - when
    # it also evaluates a carried program - every argument of the epilogue, inputs included
    listed = [int(i) for i in re.search(r"reduce_args=\[([\d,]*)\]", k.description).group(1).split(",")]
    again = [(res[out_args.index(i)], 2) if k.args[i]["is_output"] else bufs[i] for i in listed]
    folded = iter(run_kernel(k.source, "fused_matmul_reduce", reduce_grid, 256, [(ws, 0)] + again))
    for i in listed:
        if k.args[i]["is_output"]:
            res[out_args.index(i)] = next(folded)
    return res


def run_emulated(g, inputs, tile, env=()):
    os.environ["HELIUM_HIP_GEMM_TILE"] = tile
    for name in env:
        os.environ[name] = "1"
    try:
        k = ha.TileKernel.fused(g)
    finally:
        del os.environ["HELIUM_HIP_GEMM_TILE"]
        for name in env:
            del os.environ[name]
    bufs = []
    for a in k.args:
        dt = nm.NP_STORAGE[a["dtype"]]
        bufs.append((np.zeros(a["numel"], dtype=dt), 2) if a["is_output"] else (inputs[a["node"]], 0))
    res = launch_gemm(k, bufs)
    outs = [a for a in k.args if a["is_output"]]
    return k, {a["node"]: (r, a["dtype"]) for a, r in zip(outs, res)}


def compare(got, want, rel=1e-2, eps=1e-3):
    for node, (g, dtype) in got.items():
        w = want[node].reshape(-1)
        if dtype == "bf16":
            g, w = nm.bf16_bits_to_f32(g), nm.bf16_bits_to_f32(w)
        g, w = g.astype(np.float64), w.astype(np.float64)
        # approx::relative_eq(epsilon 1e-3, max_relative 1e-2), helium-kernel-generator/tests/matmul.rs:140-147
        ok = (np.abs(g - w) <= eps) | (np.abs(g - w) <= rel * np.maximum(np.abs(g), np.abs(w)))
        assert ok.all(), (node, np.abs(g - w).max())


def readme_fusion(size, mainloop, full, bias_rows=False):
    from helium_amd import configs

    g, outs = configs.c4_graph(size, mainloop=mainloop, full_size_outputs=full, bias_rows=bias_rows)
    return g, configs.c4_inputs(g, size), sorted(outs.values())


CASES = [
    ("readme_epilogue_with_prefetched_aux_tensors", lambda: readme_fusion(128, False, False), "128,128,64,2,2"),
    ("readme_epilogue", lambda: readme_fusion(128, False, False), "128,128,64,2,2"),
    ("readme_epilogue_ragged_with_mainloop", lambda: readme_fusion(72, True, True), "128,128,64,2,2"),
    ("readme_epilogue_with_biases_along_the_rows", lambda: readme_fusion(136, False, False, bias_rows=True), "128,128,64,2,2"),
    ("plain_2x2_tiles", lambda: gemm_cases.plain(160, 136, 72), "128,128,64,2,2"),
    ("ragged_scalar_paths", lambda: gemm_cases.plain(97, 131, 67), "128,128,64,2,2"),
    ("mainloop_bias_relu_colsum", lambda: gemm_cases.bias_relu_colsum(130, 136, 80, mainloop=True), "128,128,64,2,2"),
    ("row_bias", lambda: gemm_cases.bias_relu_colsum(64, 72, 64, bias_axis=2), "128,128,64,2,2"),
    ("all_reductions_batched", lambda: gemm_cases.all_reductions(70, 72, 64), "128,128,64,2,2"),
    ("f16_operands", lambda: gemm_cases.plain(64, 64, 64, dtype="f16"), "128,128,64,2,2"),
    ("f32_operands", lambda: gemm_cases.plain(40, 48, 40, dtype="f32"), "128,128,32,2,2"),
    ("f32_mainloop_and_bf16_source_round_to_bf16", lambda: gemm_cases.bias_relu_colsum(64, 72, 40, mainloop=True, a_dtype="f32"), "128,128,64,2,2"),
    ("f32_linear_layer", lambda: gemm_cases.linear_layer(48, 40, 72), "128,128,32,2,2"),
    ("big_tile_256", lambda: gemm_cases.plain(256, 256, 64), "256,256,64,2,2"),
    ("eight_tiles_xcd_order", lambda: gemm_cases.plain(256, 512, 64), "128,128,64,2,2"),
    ("twelve_tiles_grouped_order", lambda: gemm_cases.plain(768, 260, 64), "128,128,64,2,2"),
    ("eight_waves_2x4", lambda: gemm_cases.bias_relu_colsum(140, 264, 72, mainloop=True), "128,256,64,2,4"),
    ("four_stage_ring_bk32", lambda: gemm_cases.plain(256, 256, 192), "256,256,32,2,4,4"),
    ("mainloop_in_registers_b_direct", lambda: gemm_cases.bias_relu_colsum(256, 256, 128, mainloop=True), "128,128,64,2,2"),
    ("tile_64x64_staged", lambda: gemm_cases.bias_relu_colsum(100, 72, 136), "64,64,64,2,2"),
    ("tile_64x64_direct", lambda: gemm_cases.plain(128, 192, 128), "64,64,64,2,2,3"),
    ("five_stage_ring_bk32", lambda: gemm_cases.plain(256, 256, 288), "256,256,32,2,4,5"),
    ("three_stage_ring_short_k", lambda: gemm_cases.plain(128, 256, 32), "128,128,32,2,2,3"),
    ("three_stage_ring_bk64", lambda: gemm_cases.bias_relu_colsum(128, 128, 320), "128,128,64,2,2,3"),
    ("eight_waves_4x2", lambda: gemm_cases.all_reductions(256, 130, 64, batch=1), "256,128,64,4,2"),
    ("nt_direct_both_operands", lambda: gemm_cases.transposed_b(128, 256, 192), "128,128,64,2,2"),
    ("nt_ragged_staged", lambda: gemm_cases.transposed_b(70, 100, 88, batch=2), "128,128,64,2,2"),
    ("nt_mainloop_scaled_rows_of_bt", lambda: gemm_cases.transposed_b(128, 128, 128, scaled=True), "128,128,64,2,2"),
    ("nt_f32_operands", lambda: gemm_cases.transposed_b(64, 96, 64, dtype="f32"), "64,64,32,2,2,3"),
    ("nt_eight_waves_256", lambda: gemm_cases.transposed_b(256, 256, 128), "256,256,64,2,4"),
    ("tn_direct_both_operands", lambda: gemm_cases.transposed_a(128, 256, 192), "128,128,64,2,2"),
    ("tn_ragged_staged", lambda: gemm_cases.transposed_a(70, 100, 88, batch=2), "128,128,64,2,2"),
    ("tt_both_transposed", lambda: gemm_cases.transposed_a(128, 128, 128, both=True), "128,128,64,2,2"),
    ("tn_f32_operands", lambda: gemm_cases.transposed_a(64, 96, 64, dtype="f32"), "64,64,32,2,2,3"),
    ("tn_eight_waves_256", lambda: gemm_cases.transposed_a(256, 256, 128), "256,256,64,2,4"),
    ("one_wave_32x32_f32_direct", lambda: gemm_cases.plain(64, 96, 128, dtype="f32"), "32,32,32,1,1,4"),
    ("two_waves_64x32_linear_layer", lambda: gemm_cases.linear_layer(48, 40, 72), "64,32,32,2,1,4"),
]


@pytest.mark.parametrize("name,build,tile", CASES, ids=[c[0] for c in CASES])
def test_fused_gemm_on_cpu(name, build, tile):
    g, inputs, outs = build()
    k, got = run_emulated(g, inputs, tile, env=("HELIUM_HIP_GEMM_EPIPIPE",) if "prefetched" in name else ())
    assert sorted(got) == sorted(outs), k.description
    f32_cases = ("f32_operands", "f32_linear_layer", "one_wave_32x32_f32_direct", "two_waves_64x32_linear_layer", "nt_f32_operands", "tn_f32_operands")
    rounding = "f16" if name == "f16_operands" else None if name in f32_cases else "bf16"
    want = oracle.outputs(g.nodes, inputs, round_mainloop_to=rounding)
    if rounding is None:
        compare(got, want, rel=1e-4, eps=1e-5)  # f32 multiplicands: 1e-4 relative
    else:
        compare(got, want)


def test_argument_order_is_producers_then_leaves():
    g, inputs, outs = gemm_cases.bias_relu_colsum(64, 64, 64, mainloop=True)
    k = ha.TileKernel.fused(g)
    ins = [a["node"] for a in k.args if not a["is_output"]]
    assert ins == sorted(inputs) and [a["node"] for a in k.args if a["is_output"]] == outs


# ---- helium-ir Matmul nodes (the GEMM instruction of the backend) -------------------------------------------
def ir_matmul_case(shape_a, shape_b, precision, dtype, seed=3):
    rng = np.random.default_rng(seed)
    g = ha.ir.OpGraph()
    a = g.new_input(shape_a, dtype); b = g.new_input(shape_b, dtype)
    mm = g.matmul(a, b, precision)
    g.new_output(mm)
    inputs = {a: nm.to_storage(rng.uniform(-1, 1, shape_a).astype(np.float32), dtype),
              b: nm.to_storage(rng.uniform(-1, 1, shape_b).astype(np.float32), dtype)}
    return g, mm, inputs


IR_CASES = [
    # name, A shape, B shape, precision, storage dtype, max |err|
    ("f32_exact_products", [70, 40], [40, 72], "f32_f32", "f32", 1e-4),
    ("tf32_runs_as_f32", [33, 64], [64, 31], "tf32_f32", "f32", 1e-4),
    ("bf16_multiplicands_of_f32_tensors", [64, 48], [48, 64], "bf16_f32", "f32", 1e-3),
    ("f16_accumulator_type", [64, 64], [64, 64], "f16_f16", "f16", 2e-2),
    ("batched_f32", [2, 40, 24], [2, 24, 36], "f32_f32", "f32", 1e-4),
    ("f32_direct_loads_four_stage_ring", [128, 160], [160, 256], "f32_f32", "f32", 1e-4),
]


@pytest.mark.parametrize("name,sa,sb,precision,dtype,tol", IR_CASES, ids=[c[0] for c in IR_CASES])
def test_ir_matmul_on_cpu(name, sa, sb, precision, dtype, tol):
    from oracle import helium_ir as oracle_ir

    g, mm, inputs = ir_matmul_case(sa, sb, precision, dtype)
    k = ha.backend.matmul_kernel(g, [mm])
    gx, gy = map(int, re.search(r"grid=(\d+)x(\d+)", k.description).groups())
    threads = int(re.search(r"threads=(\d+)", k.description).group(1))
    bufs = []
    for a in k.args:
        dt = nm.NP_STORAGE[a["dtype"]]
        bufs.append((np.zeros(a["numel"], dtype=dt), 2) if a["is_output"] else (inputs[a["node"]], 0))
    res = run_kernel(k.source, "fused_matmul", gx, threads, bufs, grid_y=gy)
    out = [a for a in k.args if a["is_output"]]
    assert [a["node"] for a in out] == [mm]
    want = oracle_ir.kernel_outputs(g.nodes, inputs, [mm])[mm]
    got = nm.from_storage(res[0], out[0]["dtype"], [res[0].size]).astype(np.float64)
    want = nm.from_storage(want.reshape(-1), out[0]["dtype"], [want.size]).astype(np.float64)
    assert np.abs(got - want).max() <= tol, (k.description, np.abs(got - want).max())


class _Part:
    """One kernel of a composite kernel object (the classes of a strided data gradient), with its own source and
    description and the composite's argument list."""

    def __init__(self, source, description, args):
        self.source, self.description, self.args = source, description, args


def _run_one_product(k, inputs, current=None):
    """One fused-GEMM kernel (anything with .source, .description and .args) on the CPU. inputs: {node: storage array};
    current: {node: array} the outputs start from (zeros otherwise). Returns {node: storage array} of the outputs."""
    gx, gy = map(int, re.search(r"grid=(\d+)x(\d+)", k.description).groups())
    threads = int(re.search(r"threads=(\d+)", k.description).group(1))
    split = int(re.search(r"split_k=(\d+)", k.description).group(1))
    m, n = (int(v) for v in re.search(r"gemm \[\d+,(\d+),\d+\]x\[(\d+)\]", k.description).groups())
    outs = [a for a in k.args if a["is_output"]]
    bufs = []
    for a in k.args:
        if a["is_output"]:
            bufs.append((current[a["node"]] if current else np.zeros(a["numel"], dtype=nm.NP_STORAGE[a["dtype"]]), 2))
        else:
            assert inputs[a["node"]].size == a["numel"], (a, inputs[a["node"]].size)
            bufs.append((inputs[a["node"]], 0))
    if split > 1:
        # a split-k product: partial tiles go to scratch, a second launch adds them up into the one output
        res = run_kernel(k.source, "fused_matmul", gx, threads, bufs + [(np.full(split * m * n, np.nan, dtype=np.float32), 2)], grid_y=gy)
        (out,) = outs
        res = run_kernel(k.source, "fused_matmul_finalize", (m * n + 31) // 32, 256, [(res[-1], 0), (np.zeros(out["numel"], dtype=nm.NP_STORAGE[out["dtype"]]), 1)])
    else:
        res = launch_gemm(k, bufs)
    return {a["node"]: r for a, r in zip(outs, res)}


def _run_repacked(k, inputs):
    """A convolution over a repacked few-channel image: the repacking launch, the product over the copies, and for a
    filter gradient the unpacking launch, each on the CPU with buffers of exactly the size the geometry gives."""
    head, inner_desc = k.description.split("\n", 1)
    f = {key: [int(v) for v in re.findall(r"-?\d+", val)] for key, val in re.findall(r"(\w+)=(\[[^\]]*\]|-?\d+)", head)}
    image_arg, filter_arg, grad = f["image_arg"][0], f["filter_arg"][0], f["filter_gradient"][0]
    n_, hp, wp, _ = f["packed"]
    o_, r_, s_, sp = f["filter"]
    pack_src, product_src = re.split(r"// ---- product\n", k.source.split("// ---- repack\n", 1)[1])
    image = inputs[k.args[image_arg]["node"]]
    image_p = np.zeros(n_ * hp * wp, dtype=np.uint64)
    if grad:
        (image_p,) = run_kernel(pack_src, "repack_conv_operands", f["pack_grid"][0], 256, [(image, 0), (image_p, 1)])
    else:
        filt = inputs[k.args[filter_arg]["node"]]
        image_p, filter_p = run_kernel(pack_src, "repack_conv_operands", f["pack_grid"][0], 256,
                                       [(image, 0), (filt, 0), (image_p, 1), (np.zeros(o_ * r_ * sp, dtype=np.uint64), 1)])
    args = [dict(a) for a in k.args]
    args[image_arg]["numel"] = image_p.size * 4
    args[filter_arg]["numel"] = o_ * r_ * sp * 4
    inner_inputs = dict(inputs)
    inner_inputs[args[image_arg]["node"]] = image_p.view(np.uint16)
    if not grad:
        inner_inputs[args[filter_arg]["node"]] = filter_p.view(np.uint16)
    res = _run_one_product(_Part(product_src, inner_desc, args), inner_inputs)
    if grad:
        a = k.args[filter_arg]
        packed = res[a["node"]]
        (res[a["node"]],) = run_kernel(pack_src, "unpack_filter_gradient", f["unpack_grid"][0], 256,
                                       [(packed, 0), (np.zeros(a["numel"], dtype=packed.dtype), 1)])
    return res


def run_ir_kernel_on_cpu(g, nodes, inputs):
    k = ha.backend.matmul_kernel(g, nodes)
    outs = [a for a in k.args if a["is_output"]]
    if k.description.startswith("composite"):
        head, *lines = k.description.split("\n")
        parts, zero_first = (int(v) for v in re.search(r"parts=(\d+) zero_first=(\d)", head).groups())
        sources = re.split(r"// ---- part \d+ of \d+\n", k.source)[1:]
        assert len(sources) == len(lines) == parts
        # what no part writes has to be zeroed first by the host; where every element is written the buffer starts as
        # NaN here, so an element that no part wrote shows
        current = {a["node"]: (np.zeros(a["numel"], dtype=nm.NP_STORAGE[a["dtype"]]) if zero_first
                               else nm.to_storage(np.full(a["numel"], np.nan, dtype=np.float32), a["dtype"])) for a in outs}
        for src, line in zip(sources, lines):
            current = _run_one_product(_Part(src, line, k.args), inputs, current)
        res = current
    elif k.description.startswith("repacked"):
        res = _run_repacked(k, inputs)
    else:
        res = _run_one_product(k, inputs)
    return k, {a["node"]: nm.from_storage(res[a["node"]], a["dtype"], [res[a["node"]].size]).astype(np.float64) for a in outs}


def test_ir_matmul_with_epilogue_on_cpu():
    """Matmul + bias broadcast + add + relu of a helium-ir graph as one fused GEMM (config 1 at a small size)."""
    from helium_amd import configs
    from oracle import helium_ir as oracle_ir

    g, names = configs.c1_ir_graph(40, 24, 72)
    host = configs.c1_inputs(names, 40, 24, 72, batched=False)
    k, got = run_ir_kernel_on_cpu(g, [3, 4, 5, 6], host)
    assert [a["node"] for a in k.args] == [0, 1, 2, 6], k.args
    val, _ = oracle_ir.evaluate(g.nodes, host)
    assert np.abs(got[6] - val[6].reshape(-1)).max() <= 1e-4


def test_ir_matmul_with_row_sums_on_cpu():
    from oracle import helium_ir as oracle_ir

    rng = np.random.default_rng(4)
    g = ha.ir.OpGraph()
    a = g.new_input([2, 40, 24], "bf16"); b = g.new_input([2, 24, 36], "bf16")
    y = g.unary(g.matmul(a, b, "bf16_f32"), "relu")
    oy = g.new_output(y); r = g.reduce(y, "sum", 1); g.new_output(r)
    host = {a: nm.to_storage(rng.uniform(-1, 1, (2, 40, 24)).astype(np.float32), "bf16"),
            b: nm.to_storage(rng.uniform(-1, 1, (2, 24, 36)).astype(np.float32), "bf16")}
    k, got = run_ir_kernel_on_cpu(g, [2, 3, r], host)
    val, desc = oracle_ir.evaluate(g.nodes, host)
    want_y = nm.from_storage(nm.to_storage(val[y], desc[y][1]), desc[y][1], val[y].shape).astype(np.float64).reshape(-1)
    assert np.abs(got[y] - want_y).max() <= 2e-2 * np.abs(want_y).max(), k.description
    assert np.abs(got[r] - val[r].reshape(-1)).max() <= 1e-3 * np.abs(val[r]).max()


# ---- Op::Conv as an implicit GEMM ---------------------------------------------------------------------------
def conv_case(image_shape, out_channels, kernel, dtype="bf16", stride=(1, 1), dilation=(1, 1), mode="same", seed=8):
    rng = np.random.default_rng(seed)
    g = ha.ir.OpGraph()
    filter_shape = [out_channels, kernel[0], kernel[1], image_shape[3]]
    x = g.new_input(list(image_shape), dtype); w = g.new_input(filter_shape, dtype)
    params = {"in_channels": image_shape[3], "out_channels": out_channels, "kernel_size": list(kernel),
              "stride": list(stride), "dilation": list(dilation), "padding_mode": mode}
    y = g.conv(x, w, params)
    g.new_output(y)
    inputs = {x: nm.to_storage(rng.uniform(-1, 1, image_shape).astype(np.float32), dtype),
              w: nm.to_storage((rng.uniform(-1, 1, filter_shape) * 0.25).astype(np.float32), dtype)}
    return g, y, inputs


def test_conv_reference_known_answer_on_cpu():
    """conv_simple (helium/tests/tensor_ops.rs:379-397): 1x1 kernel over two channels."""
    g = ha.ir.OpGraph()
    x = g.new_input([1, 1, 1, 2], "f32"); w = g.new_input([2, 1, 1, 2], "f32")
    y = g.conv(x, w, {"in_channels": 2, "out_channels": 2, "kernel_size": [1, 1]})
    g.new_output(y)
    assert g.descriptor(y) == ([1, 1, 1, 2], "f32")
    inputs = {x: np.array([1.0, 2.0], np.float32), w: np.array([10.0, 20.0, 30.0, 40.0], np.float32)}
    _, got = run_ir_kernel_on_cpu(g, [y], inputs)
    assert got[y].tolist() == [50.0, 110.0]


CONV_CASES = [
    # name, image NHWC, out channels, kernel, dtype, stride, dilation, padding mode, tile
    ("3x3_same_bf16", (2, 9, 10, 16), 24, (3, 3), "bf16", (1, 1), (1, 1), "same", "128,128,64,2,2"),
    ("3x3_stride2_bf16", (1, 12, 12, 8), 32, (3, 3), "bf16", (2, 2), (1, 1), "same", "64,64,64,2,2"),
    ("1x1_stride2_shortcut", (2, 8, 8, 32), 64, (1, 1), "bf16", (2, 2), (1, 1), "same", "128,128,64,2,2"),
    ("three_channel_image_7x7", (1, 10, 9, 3), 16, (7, 7), "bf16", (2, 2), (1, 1), "same", "128,128,64,2,2"),
    ("valid_and_dilated_f32", (1, 9, 9, 4), 8, (3, 3), "f32", (1, 1), (2, 1), "valid", "64,64,32,2,2"),
    ("full_padding_f16", (1, 6, 7, 8), 8, (3, 2), "f16", (1, 1), (1, 1), "full", "128,128,64,2,2"),
    # 64 channels = one k-tile per filter tap: the gather keeps the pixel terms of its rows across the k-loop
    ("hoisted_pixel_terms_ragged_rows", (2, 7, 9, 64), 32, (3, 3), "bf16", (1, 1), (1, 1), "same", "128,128,64,2,2"),
    ("hoisted_pixel_terms_stride2_eight_waves", (1, 12, 10, 128), 64, (3, 3), "bf16", (2, 2), (1, 1), "same", "256,64,64,4,2"),
    ("hoisted_pixel_terms_eight_waves_of_64x32", (2, 12, 11, 64), 128, (3, 3), "bf16", (1, 1), (1, 1), "same", "128,128,64,2,4"),
    ("hoisted_pixel_terms_f32_dilated", (1, 9, 8, 32), 16, (3, 3), "f32", (1, 1), (2, 2), "valid", "64,64,32,2,2"),
    # channel counts that are no multiple of a chunk: gathered element by element
    ("odd_channels_five_3x3", (2, 7, 6, 5), 16, (3, 3), "bf16", (1, 1), (1, 1), "same", "64,64,64,2,2"),
    ("odd_channels_three_f32_full", (1, 6, 5, 3), 8, (3, 3), "f32", (1, 1), (2, 1), "full", "64,64,32,2,2"),
    ("odd_channels_three_5x5_stride3", (1, 11, 13, 3), 8, (5, 5), "f16", (3, 3), (1, 1), "same", "64,64,64,2,2"),
    # the tiles of products with 32 columns: four waves of 64x32 (direct loads), 256x64 for the element-wise gather
    ("thirty_two_channels_out_narrow_tile", (2, 12, 12, 32), 32, (3, 3), "bf16", (2, 2), (1, 1), "same", "256,32,64,4,1"),
    ("three_channel_stem_wide_gather_tile", (2, 10, 10, 3), 32, (7, 7), "bf16", (1, 1), (1, 1), "same", "256,64,64,4,2"),
    # 3 or 4 channels, 16-bit, even stride along w: the product runs over a 4-channel copy of the image with the padding
    # written out, two pixels to a 16-byte chunk
    ("repacked_three_channel_stem", (2, 16, 16, 3), 32, (7, 7), "bf16", (2, 2), (1, 1), "same", "256,64,64,4,2"),
    ("repacked_four_channels_even_taps_valid", (1, 9, 14, 4), 16, (3, 4), "f16", (1, 2), (2, 1), "valid", "64,64,64,2,2"),
    ("repacked_three_channels_stride_2x4_full", (2, 8, 11, 3), 8, (5, 3), "bf16", (2, 4), (1, 1), "full", "128,128,64,2,2"),
]


def repacks(image, kernel, dtype, stride, dilation):
    return dtype != "f32" and image[3] in (3, 4) and stride[1] % 2 == 0 and dilation[1] == 1 and kernel[1] >= 2


@pytest.mark.parametrize("name,image,oc,kernel,dtype,stride,dilation,mode,tile", CONV_CASES, ids=[c[0] for c in CONV_CASES])
def test_conv_on_cpu(name, image, oc, kernel, dtype, stride, dilation, mode, tile):
    from oracle import helium_ir as oracle_ir

    g, y, inputs = conv_case(image, oc, kernel, dtype, stride, dilation, mode)
    os.environ["HELIUM_HIP_GEMM_TILE"] = tile
    try:
        k, got = run_ir_kernel_on_cpu(g, [y], inputs)
    finally:
        del os.environ["HELIUM_HIP_GEMM_TILE"]
    want = oracle_ir.kernel_outputs(g.nodes, inputs, [y])[y]
    want = nm.from_storage(want.reshape(-1), dtype, [want.size]).astype(np.float64)
    tol = 1e-4 if dtype == "f32" else 2e-2
    assert np.abs(got[y] - want).max() <= tol * max(1.0, np.abs(want).max()), (k.description, np.abs(got[y] - want).max())
    assert ("#define CONV_A_FAST 1" in k.source) == name.startswith("hoisted"), name
    assert k.description.startswith("repacked") == repacks(image, kernel, dtype, stride, dilation), k.description


BWD_DATA_CASES = [
    # name, image NHWC (the tensor whose gradient is computed), out channels, kernel, dtype, stride, dilation, mode, tile
    ("3x3_same_bf16", (2, 9, 10, 16), 24, (3, 3), "bf16", (1, 1), (1, 1), "same", "128,128,64,2,2"),
    ("3x3_stride2_bf16", (1, 12, 12, 8), 32, (3, 3), "bf16", (2, 2), (1, 1), "same", "64,64,64,2,2"),
    ("1x1_stride2_shortcut", (2, 8, 8, 32), 64, (1, 1), "bf16", (2, 2), (1, 1), "same", "128,128,64,2,2"),
    ("direct_loads_both_operands", (1, 16, 16, 128), 64, (3, 3), "bf16", (1, 1), (1, 1), "same", "128,128,64,2,2"),
    ("thirty_two_channels_in_narrow_tile_stride2", (2, 12, 12, 32), 64, (3, 3), "bf16", (2, 2), (1, 1), "same", "256,32,64,4,1"),
    ("thirty_two_channels_in_narrow_tile_1x1", (2, 12, 12, 32), 64, (1, 1), "bf16", (2, 2), (1, 1), "same", "256,32,64,4,1"),
    ("valid_and_dilated_f32", (1, 9, 9, 4), 8, (3, 3), "f32", (1, 1), (2, 1), "valid", "64,64,32,2,2"),
    ("hoisted_pixel_terms_stride2", (2, 10, 9, 16), 64, (3, 3), "bf16", (2, 2), (1, 1), "same", "128,128,64,2,2"),
    ("flow_gathered_element_by_element", (1, 9, 8, 16), 12, (3, 3), "bf16", (2, 1), (1, 1), "same", "64,64,64,2,2"),
    # one product per class of pixels (row and column modulo the stride): classes of 3x3, 3x2, 2x3 and 2x2 taps
    ("5x5_stride2_classes", (2, 11, 12, 8), 16, (5, 5), "bf16", (2, 2), (1, 1), "same", "64,64,64,2,2"),
    # ... of 1 to 4 taps per dim, one class that no tap reaches in valid mode; image extents that the stride does not divide
    ("3x3_stride3_valid_classes", (1, 10, 11, 8), 16, (3, 3), "bf16", (3, 3), (1, 1), "valid", "64,64,64,2,2"),
    ("7x7_stride2_full_f32", (1, 9, 10, 4), 8, (7, 7), "f32", (2, 2), (1, 1), "full", "64,64,32,2,2"),
]


@pytest.mark.parametrize("name,image,oc,kernel,dtype,stride,dilation,mode,tile", BWD_DATA_CASES, ids=[c[0] for c in BWD_DATA_CASES])
def test_conv_backward_data_on_cpu(name, image, oc, kernel, dtype, stride, dilation, mode, tile):
    """Op::ConvBackwardData as an implicit GEMM: the flow gathered as A (with the stride's divisibility test), the
    filter's rows picked as B. The oracle is the adjoint of the forward convolution."""
    from oracle import helium_ir as oracle_ir

    rng = np.random.default_rng(10)
    params = {"in_channels": image[3], "out_channels": oc, "kernel_size": list(kernel), "stride": list(stride),
              "dilation": list(dilation), "padding_mode": mode}
    out_hw = oracle_ir.conv_output_size(params, image[1:3], kernel)
    flow_shape = [image[0], out_hw[0], out_hw[1], oc]
    filter_shape = [oc, kernel[0], kernel[1], image[3]]
    g = ha.ir.OpGraph()
    dy = g.new_input(flow_shape, dtype); w = g.new_input(filter_shape, dtype)
    dx = g.conv_backward_data(dy, w, params, image[1:3])
    g.new_output(dx)
    assert g.descriptor(dx) == (list(image), dtype)
    inputs = {dy: nm.to_storage(rng.uniform(-1, 1, flow_shape).astype(np.float32), dtype),
              w: nm.to_storage((rng.uniform(-1, 1, filter_shape) * 0.25).astype(np.float32), dtype)}
    os.environ["HELIUM_HIP_GEMM_TILE"] = tile
    try:
        k, got = run_ir_kernel_on_cpu(g, [dx], inputs)
    finally:
        del os.environ["HELIUM_HIP_GEMM_TILE"]
    assert k.description.startswith("composite") == (tuple(stride) != (1, 1) and tuple(dilation) == (1, 1)), k.description
    want = oracle_ir.kernel_outputs(g.nodes, inputs, [dx])[dx]
    want = nm.from_storage(want.reshape(-1), dtype, [want.size]).astype(np.float64)
    tol = 1e-4 if dtype == "f32" else 2e-2
    assert np.abs(got[dx] - want).max() <= tol * max(1.0, np.abs(want).max()), (k.description, np.abs(got[dx] - want).max())


BWD_FILTER_CASES = [
    # name, image NHWC, out channels, kernel, dtype, stride, dilation, mode, tile
    ("3x3_same_bf16", (2, 9, 10, 16), 24, (3, 3), "bf16", (1, 1), (1, 1), "same", "128,128,64,2,2"),
    ("3x3_stride2_bf16", (2, 12, 12, 8), 32, (3, 3), "bf16", (2, 2), (1, 1), "same", "64,64,64,2,2"),
    ("1x1_stride2_shortcut", (2, 8, 8, 32), 64, (1, 1), "bf16", (2, 2), (1, 1), "same", "128,128,64,2,2"),
    ("direct_loads_both_operands", (4, 16, 16, 16), 128, (3, 3), "bf16", (1, 1), (1, 1), "same", "128,128,64,2,2"),
    ("valid_and_dilated_f32", (2, 9, 9, 4), 8, (3, 3), "f32", (1, 1), (2, 1), "valid", "64,64,32,2,2"),
    # channel counts that do not fill a 16-byte chunk: the image operand is gathered element by element
    ("three_channel_stem_7x7_stride2", (2, 16, 16, 3), 32, (7, 7), "bf16", (2, 2), (1, 1), "same", "64,128,64,2,2"),
    ("three_channel_stem_thirty_two_rows_tile", (2, 10, 10, 3), 32, (7, 7), "bf16", (1, 1), (1, 1), "same", "32,128,64,1,4"),
    ("three_channel_stem_two_wave_tile", (2, 10, 10, 3), 32, (7, 7), "bf16", (1, 1), (1, 1), "same", "32,64,64,1,2"),
    # over a repacked copy of the image; the gradient comes out in the packed filter layout and is unpacked
    ("repacked_four_channels_stride_1x2", (2, 9, 14, 4), 16, (3, 4), "f16", (1, 2), (2, 1), "valid", "64,64,64,2,2"),
    ("repacked_three_channels_5x3_full", (2, 8, 11, 3), 8, (5, 3), "bf16", (2, 4), (1, 1), "full", "128,128,64,2,2"),
    ("thirty_two_rows_tile_direct_loads", (2, 12, 12, 16), 32, (3, 3), "bf16", (1, 1), (1, 1), "same", "32,128,64,1,4"),
    ("five_channels_3x3_f16", (1, 7, 9, 5), 8, (3, 3), "f16", (1, 1), (1, 1), "same", "64,64,64,2,2"),
    ("three_channels_f32_full", (1, 6, 5, 3), 8, (3, 3), "f32", (1, 1), (1, 2), "full", "64,64,32,2,2"),
    # 128 output channels: tiles as tall as M and 256 wide (what the generator picks for this shape when the k range is split)
    ("tall_wide_tile_128_channels", (2, 16, 16, 64), 128, (3, 3), "bf16", (1, 1), (1, 1), "same", "128,256,64,2,4"),
]


@pytest.mark.parametrize("name,image,oc,kernel,dtype,stride,dilation,mode,tile", BWD_FILTER_CASES, ids=[c[0] for c in BWD_FILTER_CASES])
def test_conv_backward_filter_on_cpu(name, image, oc, kernel, dtype, stride, dilation, mode, tile):
    """Op::ConvBackwardFilter as a split-k implicit GEMM: the flow read as a [k][m] A operand, the image gathered
    as B, partial tiles added by the second launch."""
    from oracle import helium_ir as oracle_ir

    rng = np.random.default_rng(11)
    params = {"in_channels": image[3], "out_channels": oc, "kernel_size": list(kernel), "stride": list(stride),
              "dilation": list(dilation), "padding_mode": mode}
    out_hw = oracle_ir.conv_output_size(params, image[1:3], kernel)
    flow_shape = [image[0], out_hw[0], out_hw[1], oc]
    g = ha.ir.OpGraph()
    dy = g.new_input(flow_shape, dtype); x = g.new_input(list(image), dtype)
    dw = g.conv_backward_filter(dy, x, params)
    g.new_output(dw)
    assert g.descriptor(dw) == ([oc, kernel[0], kernel[1], image[3]], dtype)
    inputs = {dy: nm.to_storage((rng.uniform(-1, 1, flow_shape) * 0.5).astype(np.float32), dtype),
              x: nm.to_storage(rng.uniform(-1, 1, image).astype(np.float32), dtype)}
    os.environ["HELIUM_HIP_GEMM_TILE"] = tile
    try:
        k, got = run_ir_kernel_on_cpu(g, [dw], inputs)
    finally:
        del os.environ["HELIUM_HIP_GEMM_TILE"]
    want = oracle_ir.kernel_outputs(g.nodes, inputs, [dw])[dw]
    want = nm.from_storage(want.reshape(-1), dtype, [want.size]).astype(np.float64)
    tol = 1e-4 if dtype == "f32" else 2e-2
    assert np.abs(got[dw] - want).max() <= tol * max(1.0, np.abs(want).max()), (k.description, np.abs(got[dw] - want).max())
    assert k.description.startswith("repacked") == repacks(image, kernel, dtype, stride, dilation), k.description


def test_filter_gradient_of_128_channels_takes_tall_wide_tiles():
    """Without an override: a [128 x 576] gradient over 512 pixels gets 128x256 tiles and a split k range."""
    g = ha.ir.OpGraph()
    params = {"in_channels": 64, "out_channels": 128, "kernel_size": [3, 3], "stride": [1, 1], "dilation": [1, 1], "padding_mode": "same"}
    dy = g.new_input([2, 16, 16, 128], "bf16"); x = g.new_input([2, 16, 16, 64], "bf16")
    dw = g.conv_backward_filter(dy, x, params)
    g.new_output(dw)
    d = ha.backend.matmul_kernel(g, [dw]).description
    assert "tile=128x256x64" in d and "split_k=2" in d, d


def test_conv_backward_filter_with_many_partial_tiles_on_cpu(monkeypatch):
    """Sixteen shares of the k range: the launch that adds the partial tiles up takes them 16 bytes at a time."""
    monkeypatch.setenv("HELIUM_HIP_GEMM_SPLIT_K", "16")
    test_conv_backward_filter_on_cpu("sixteen_partial_tiles", (4, 16, 16, 16), 24, (3, 3), "bf16", (1, 1), (1, 1), "same", "64,64,64,2,2")


@pytest.mark.parametrize("dtype,precision,tol", [("f32", "f32_f32", 1e-4), ("bf16", "bf16_f32", 2e-2)])
def test_ir_matmul_with_transposed_operands_on_cpu(dtype, precision, tol):
    """x^T dy and dy w^T of a linear layer's backward pass: each SwapDims joins its Matmul and the kernel reads
    the untransposed tensor (A as [k][m], B as [n][k])."""
    import test_plan_cpu as plans
    from oracle import helium_ir as oracle_ir

    g, n = plans.linear_backward_graph(64, 96, 80, dtype, precision)
    rng = np.random.default_rng(14)
    host = {n["x"]: nm.to_storage(rng.uniform(-1, 1, (64, 96)).astype(np.float32), dtype),
            n["w"]: nm.to_storage(rng.uniform(-1, 1, (96, 80)).astype(np.float32), dtype),
            n["dy"]: nm.to_storage(rng.uniform(-1, 1, (64, 80)).astype(np.float32), dtype)}
    val, _ = oracle_ir.evaluate(g.nodes, host)
    for nodes, out in (([n["xt"], n["dw"]], n["dw"]), ([n["wt"], n["dx"]], n["dx"])):
        os.environ["HELIUM_HIP_GEMM_TILE"] = "64,64,32,2,2" if dtype == "f32" else "64,64,64,2,2"
        try:
            k, got = run_ir_kernel_on_cpu(g, nodes, host)
        finally:
            del os.environ["HELIUM_HIP_GEMM_TILE"]
        want = val[out].reshape(-1).astype(np.float64)
        assert np.abs(got[out] - want).max() <= tol * max(1.0, np.abs(want).max()), (k.description, np.abs(got[out] - want).max())


# ---- reductions over leading dims of the product (SwapDims + Reduce) in the epilogue ------------------------------
@pytest.mark.parametrize("m,n,k", [(40, 72, 24), (48, 48, 16)])
def test_ir_matmul_with_column_sums_on_cpu(m, n, k):
    """Config 1 whole: relu(X W + b) and its column sums, which helium-ir writes as SwapDims + Reduce, in one fused
    GEMM. The square case has a Reduce input of the product's own shape: only the path back to the Matmul tells which
    dim is folded."""
    from helium_amd import configs
    from oracle import helium_ir as oracle_ir

    g, names = configs.c1_ir_graph(m, k, n)
    host = configs.c1_inputs(names, m, k, n, batched=False)
    ops = [nd["id"] for nd in g.nodes if nd["node"] == "op"]
    kern, got = run_ir_kernel_on_cpu(g, ops, host)
    val, _ = oracle_ir.evaluate(g.nodes, host)
    outs = {nd["from"] for nd in g.nodes if nd["node"] == "output"}
    assert set(got) == outs and len(outs) == 2
    for node in outs:
        want = val[node].reshape(-1)
        assert got[node].shape == want.shape
        assert np.abs(got[node] - want).max() <= 1e-4 * max(1.0, np.abs(want).max()), (node, kern.description)


def test_ir_conv_with_batch_norm_statistics_on_cpu():
    """A convolution with the per-channel mean of its output and of its square (BatchNorm2d's statistics: SwapDims of
    batch and channel dims, Reduce over the three trailing dims) as one implicit GEMM; batch = channels, so the
    Reduce's input has the output's own shape."""
    from harness import frontend
    from oracle import helium_ir as oracle_ir

    rng = np.random.default_rng(21)
    g = ha.ir.OpGraph()
    rec = frontend.Recorder(g)
    x = g.new_input([8, 6, 5, 16], "bf16"); w = g.new_input([8, 3, 3, 16], "bf16")
    y = g.conv(x, w, {"in_channels": 16, "out_channels": 8, "kernel_size": [3, 3]})
    yt = g.swap_dims(y, 0, 3)
    mean = g.reduce(yt, "mean", 3)
    mean_sq = g.reduce(rec.pow_scalar(yt, 2.0), "mean", 3)
    for v in (y, mean, mean_sq):
        g.new_output(v)
    host = {x: nm.to_storage(rng.standard_normal((8, 6, 5, 16)).astype(np.float32), "bf16"),
            w: nm.to_storage((rng.standard_normal((8, 3, 3, 16)) * 0.2).astype(np.float32), "bf16"), **rec.scalars}
    ops = [nd["id"] for nd in g.nodes if nd["node"] == "op"]
    kern, got = run_ir_kernel_on_cpu(g, ops, host)
    val, desc = oracle_ir.evaluate(g.nodes, host)
    want_y = val[y].reshape(-1)
    assert np.abs(got[y] - want_y).max() <= 1e-2 * max(1.0, np.abs(want_y).max()), kern.description
    for node in (mean, mean_sq):
        want = val[node].reshape(-1)
        assert got[node].shape == want.shape
        assert np.abs(got[node] - want).max() <= 2e-3 * max(1.0, np.abs(want).max()), (node, got[node], want)


def test_epilogue_refuses_what_it_cannot_reduce():
    """Part of the rows (one image dim of a convolution), or a reduction that keeps its dims in another order, stays a
    kernel of its own."""
    g = ha.ir.OpGraph()
    x = g.new_input([4, 6, 5, 16], "bf16"); w = g.new_input([8, 3, 3, 16], "bf16")
    y = g.conv(x, w, {"in_channels": 16, "out_channels": 8, "kernel_size": [3, 3]})
    r = g.reduce(g.swap_dims(y, 2, 3), "sum", 1)   # folds q only
    g.new_output(y); g.new_output(r)
    with pytest.raises(ha.HeliumError):
        ha.backend.matmul_kernel(g, [nd["id"] for nd in g.nodes if nd["node"] == "op"])
