"""Measures a set of fusion plans on the GPU and fits the coefficients of the MI355X cost model to them.

The model (fused_graph.cpp: mi355x_cost) is linear in seven terms per plan (fusion_search.COST_TERMS); this script runs
every plan the four search objectives produce for a list of graphs, takes the terms through the C ABI
(he_fusion_plan_cost_terms) and the time per execution from HIP events, and solves the non-negative least squares
problem. It prints a table (what profiles/cost_model_fit.txt holds) and the initialiser for
Mi355xCoefficients::fitted(). Needs a GPU:  python -m harness.cost_fit [--steps K]
"""
import argparse
import time

import numpy as np

from helium_amd import configs, device, fusion, fusion_search as fs
from helium_amd.device import DeviceBuffer, Event, Stream

ITEMSIZE = {"bf16": 2, "f16": 2, "f32": 4}


def _gemm(m, n, k, aux=0, out="bf16", colsum=False, relu_a=False, mul_a=False, relu_b=False, bias_relu=False):
    g = fusion.OpGraph()
    a, b = g.producer([1, m, k], "bf16"), g.producer([1, k, n], "bf16")
    if relu_a:
        a = g.unary(a, "relu")
    if mul_a:
        a = g.binary(a, g.producer([1, m, k], "bf16"), "mul")
    if relu_b:
        b = g.unary(b, "relu")
    x = g.matmul(a, b)
    for _ in range(aux):
        x = g.binary(x, g.producer([1, m, n], "bf16"), "add")
    if bias_relu:
        x = g.unary(g.binary(x, g.broadcast(g.producer([1, 1, n], "f32"), 1, m), "add"), "relu")
    if colsum:
        g.consumer(g.reduction(x, "columns"), "f32")
    if out:
        g.consumer(x, out)
    return g


def _aux_relu_mul(m, n):
    g = fusion.OpGraph()
    g.consumer(g.binary(g.unary(g.producer([1, m, n], "bf16"), "relu"), g.producer([1, m, n], "bf16"), "mul"), "bf16")
    return g


def _aux_tanh_chain(m, n):
    g = fusion.OpGraph()
    x = g.binary(g.producer([1, m, n], "bf16"), g.producer([1, m, n], "bf16"), "add")
    x = g.unary(g.unary(x, "tanh"), "pow_constant", 2.0)
    g.consumer(g.unary(g.binary(x, g.producer([1, m, n], "bf16"), "mul"), "tanh"), "bf16")
    return g


def _with_consumers(g):
    """The search keeps what a Consumer reads (FusedGraph::clean): leaves that are bare reductions get one."""
    used = set()
    for n in g.nodes:
        for k in ("a", "b", "x", "lhs", "rhs"):
            if k in n:
                used.add(n[k])
    for n in list(g.nodes):
        if n["id"] not in used and n["op"] != "consumer":
            g.consumer(n["id"], "f32" if n["op"] == "reduction" else "bf16")
    return g


def graphs():
    s = 4096
    return {name: _with_consumers(g) for name, g in _graphs(s).items()}


def _graphs(s):
    return {
        "gemm 4096^3": _gemm(s, s, s),
        "gemm 2048^3": _gemm(2048, 2048, 2048),
        "gemm 8192x4096x4096": _gemm(8192, s, s),
        "gemm 4096x4096x8192": _gemm(s, s, 8192),
        "gemm + column sums only": _gemm(s, s, s, out=None, colsum=True),
        "gemm + 1 added tensor": _gemm(s, s, s, aux=1),
        "gemm + 3 added tensors": _gemm(s, s, s, aux=3),
        "gemm + 5 added tensors, column sums": _gemm(s, s, s, aux=5, out=None, colsum=True),
        "gemm + bias + relu": _gemm(s, s, s, bias_relu=True),
        "relu(A) gemm": _gemm(s, s, s, relu_a=True),
        "relu(A)*T gemm": _gemm(s, s, s, relu_a=True, mul_a=True),
        "relu(A)*T, relu(B) gemm": _gemm(s, s, s, relu_a=True, mul_a=True, relu_b=True),
        "C5a": configs.c5a_graph(s)[0],
        "C4": configs.c4_graph(s)[0],
        "C4m": configs.c4_graph(s, mainloop=True, full_size_outputs=True)[0],
        "C3": configs.c3_chain(make_inputs=False)[0],
        "relu(A0)*T": _aux_relu_mul(s, s),
        "tanh chain": _aux_tanh_chain(s, s),
    }


def _buffers(graph, rng, nsets):
    used = set()
    for n in graph.nodes:
        for k in ("a", "b", "x", "lhs", "rhs"):
            if k in n:
                used.add(n[k])
    sets = []
    for _ in range(nsets):
        prod, cons = {}, {}
        for n in graph.nodes:
            numel = int(np.prod(n["shape"]))
            if n["op"] == "producer":
                if n["dtype"] == "f32":
                    prod[n["id"]] = DeviceBuffer.from_numpy(rng.standard_normal(numel).astype(np.float32))
                else:
                    prod[n["id"]] = DeviceBuffer.from_numpy(configs.bf16_rne((rng.standard_normal(numel) * 0.05).astype(np.float32)))
            elif n["id"] not in used:  # a leaf: Consumer or reduction
                dt = n.get("dtype", "f32") if n["op"] == "consumer" else "f32"
                cons[n["id"]] = DeviceBuffer(max(256, numel * ITEMSIZE[dt]))
        sets.append((prod, cons))
    return sets


def measure(plan, sets, stream, steps, warmup):
    for i in range(warmup):
        plan.execute(*sets[i % len(sets)], stream=stream)
    stream.synchronize()
    start, stop = Event(), Event()
    start.record(stream)
    for i in range(steps):
        plan.execute(*sets[i % len(sets)], stream=stream)
    stop.record(stream)
    stop.synchronize()
    return start.elapsed_ms(stop) / steps * 1e-3


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=150)
    args = ap.parse_args()
    from scipy.optimize import nnls

    device.init(0)
    stream = Stream()
    rng = np.random.default_rng(5)
    rows = []
    for name, g in graphs().items():
        sets, seen = None, set()
        for objective in (fs.MAXIMAL, fs.MIN_NAIVE_COST, fs.MIN_ANALYTICAL_COST, fs.MIN_MI355X_COST):
            plan = fs.FusionPlan(g, objective)
            if plan.text in seen:
                continue
            seen.add(plan.text)
            if sets is None:
                per_set = sum(int(np.prod(n["shape"])) * ITEMSIZE.get(n.get("dtype", "f32"), 4) for n in g.nodes if n["op"] == "producer")
                sets = _buffers(g, rng, max(2, min(4, (600 << 20) // max(per_set, 1) + 1)))
            t0 = time.time()
            seconds = measure(plan, sets, stream, args.steps, args.warmup)
            terms = plan.cost_terms()
            kinds = "+".join(("core[m%d,e%d]" % (len(f["mainloop"]), len(f["epilogue"]))) if f["core"] else "aux[%d]" % len(f["aux"]) for f in plan.fusions)
            rows.append((name, kinds, seconds, [terms[k] for k in fs.COST_TERMS], plan.cost(fs.MIN_MI355X_COST)))
            print(f"measured {name} as {kinds}: {seconds * 1e6:.1f} us ({time.time() - t0:.1f} s)", flush=True)
        for prod, cons in sets or []:
            for b in list(prod.values()) + list(cons.values()):
                b.free()
    a = np.array([r[3] for r in rows], dtype=np.float64)
    t = np.array([r[2] for r in rows], dtype=np.float64)
    # relative errors matter: scale every row by its own time
    coef, _ = nnls(a / t[:, None], np.ones_like(t))
    print("\nterms: " + ", ".join(fs.COST_TERMS))
    print(f"{'plan':58s} {'measured us':>11s} {'fitted us':>10s} {'shipped us':>10s}")
    for (name, kinds, seconds, terms, shipped) in rows:
        print(f"{(name + ' as ' + kinds)[:58]:58s} {seconds * 1e6:11.1f} {float(np.dot(coef, terms)) * 1e6:10.1f} {shipped * 1e6:10.1f}")
    pred = a @ coef
    print(f"\nmean |relative error| of the fit: {float(np.mean(np.abs(pred - t) / t)):.3f}, worst {float(np.max(np.abs(pred - t) / t)):.3f}")
    print("Mi355xCoefficients::fitted(): {{" + ", ".join(f"{c:.4g}" for c in coef) + "}}")


if __name__ == "__main__":
    main()
