"""Shared test helpers: front-end lowerings (as helium/src/raw_tensor.rs writes them), runners that execute one
tile kernel either on the GPU through the C ABI or on the CPU under the emulation shim, and comparison helpers."""
import re

import numpy as np

from oracle import helium_ir as oracle_ir
from oracle import numerics as nm


# ---- front-end lowerings (helium/src/raw_tensor.rs) live in the package; the tests use the same ones
from harness.frontend import broadcast_to, div, scalar_tensor, sub  # noqa: E402,F401


# ---- runners -----------------------------------------------------------------------------------------------
def _launch_numbers(desc):
    return int(re.search(r"grid=(\d+)", desc).group(1)), int(re.search(r"threads=(\d+)", desc).group(1))


def run_tile_kernel_gpu(kernel, inputs_by_node):
    """Executes on the GPU; returns {leaf node: storage array}."""
    from helium_amd import DeviceBuffer

    bufs, outs = [], {}
    for a in kernel.args:
        nbytes = _storage_bytes(a)
        if a["is_output"]:
            b = DeviceBuffer(max(nbytes, 4))
            b.fill_u8(0xEE)
            outs[a["node"]] = (b, a)
        else:
            host = np.ascontiguousarray(inputs_by_node[a["node"]])
            assert host.nbytes == nbytes, (a, host.nbytes, nbytes)
            b = DeviceBuffer.from_numpy(host) if nbytes else DeviceBuffer(4)
        bufs.append(b)
    kernel.execute(bufs)
    return {node: b.to_numpy(nm.NP_STORAGE[a["dtype"]])[: _storage_elems(a)] for node, (b, a) in outs.items()}


def _storage_bytes(a):
    if a["dtype"] == "bool":
        return (a["numel"] + 31) // 32 * 4
    return a["numel"] * np.dtype(nm.NP_STORAGE[a["dtype"]]).itemsize


def _storage_elems(a):
    return (a["numel"] + 31) // 32 if a["dtype"] == "bool" else a["numel"]


def run_tile_kernel_cpu(kernel, inputs_by_node, entry, fills=None):
    """Executes the generated source on the CPU (tests/cpu_emul.py). The outputs the kernel's description lists
    under fills=[argument:pattern,...] start from that 32-bit pattern, as the launch pre-fills them; every other
    output starts as garbage. `fills`: {leaf node: pattern} the caller expects for the pre-filled ones."""
    from cpu_emul import run_kernel

    grid, threads = _launch_numbers(kernel.description)
    listed = re.search(r"fills=\[([^\]]*)\]", kernel.description)
    prefill = {int(a): int(v) for a, v in (item.split(":") for item in listed.group(1).split(",") if item)} if listed else {}
    buffers, order = [], []
    for i, a in enumerate(kernel.args):
        dt = nm.NP_STORAGE[a["dtype"]]
        if a["is_output"]:
            if i in prefill:  # pre-filled outputs are 32-bit typed (f32 reductions, u32 bitsets)
                if fills is not None:
                    assert fills[a["node"]] == prefill[i], (a, prefill)
                buffers.append((np.full(_storage_elems(a), prefill[i], dtype=np.uint32).view(dt), 2))
            else:
                buffers.append((np.empty(_storage_elems(a), dtype=dt), 1))
            order.append(a["node"])
        else:
            buffers.append((np.ascontiguousarray(inputs_by_node[a["node"]]), 0))
    # scratch of the cross-block reductions: partials, then arrival counters, which every launch must leave at zero
    ws = re.search(r"ws_floats=(\d+) ws_counters=(\d+) finalize_grid=(\d+)", kernel.description)
    n_floats, n_counters, finalize_grid = (int(v) for v in ws.groups()) if ws else (0, 0, 0)
    if n_floats:
        buffers.append((np.full(n_floats, np.nan, dtype=np.float32), 2))
        buffers.append((np.zeros(max(n_counters, 1), dtype=np.uint32), 2))
    outs = run_kernel(kernel.source, entry, grid, threads, buffers)
    if n_floats:
        assert not outs[-1].any(), "arrival counters not back at zero"
        partials, outs = outs[-2], outs[:-2]
        if finalize_grid:
            # the second launch: same arguments (outputs carried over), then the partials
            it = iter(outs)
            again = [(next(it), 2) if a["is_output"] else b for a, b in zip(kernel.args, buffers)]
            outs = run_kernel(kernel.source, entry + "_finalize", finalize_grid, threads, again + [(partials, 0)])
    return dict(zip(order, outs))


def reduction_fills(graph_nodes, leaf_ids):
    """32-bit fill pattern per reduction / bitset leaf, as PointwiseGraph::execute initialises them
    (helium/src/cuda/instr/pointwise.rs:62-74,113-119)."""
    by_id = {n["id"]: n for n in graph_nodes}
    fills = {}
    for leaf in leaf_ids:
        n = by_id[leaf]
        if n.get("op") == "reduce":
            ident = {"sum": 0.0, "mean": 0.0, "max": -np.inf, "min": np.inf}[n["fn"]]
            fills[leaf] = int(np.array([ident], dtype=np.float32).view(np.uint32)[0])
        elif n.get("dtype") == "bool":
            fills[leaf] = 0
    return fills


# ---- comparison --------------------------------------------------------------------------------------------
def assert_storage_close(got, want, dtype, what="", max_ulps=2, reduce_rel=None):
    """Float outputs: the reference tests' ulps criterion on the f32 value (bf16/f16 outputs: at most one step of
    the storage format apart). `reduce_rel`: relative tolerance for reductions (summation order is free)."""
    if dtype in ("u32", "bool"):
        assert np.array_equal(got, want), what
        return
    if dtype == "f32":
        g, w = np.asarray(got, np.float32), np.asarray(want, np.float32)
        if reduce_rel is not None:
            ok = np.isclose(g.astype(np.float64), w.astype(np.float64), rtol=reduce_rel, atol=1e-6) | (g == w)
        else:
            ok = nm.ulps_close(g, w, max_ulps=max_ulps)
    else:
        conv = nm.bf16_bits_to_f32 if dtype == "bf16" else nm.f16_bits_to_f32
        diff = np.abs(np.asarray(got, np.uint16).astype(np.int32) - np.asarray(want, np.uint16).astype(np.int32))
        ok = (diff <= 1) | (np.isnan(conv(got)) & np.isnan(conv(want)))
    if not ok.all():
        bad = np.flatnonzero(~ok.reshape(-1))[:5]
        raise AssertionError(f"{what}: {(~ok).sum()} of {ok.size} elements differ, e.g. at {bad}: got "
                             f"{np.asarray(got).reshape(-1)[bad]} want {np.asarray(want).reshape(-1)[bad]}")
