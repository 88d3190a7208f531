"""The largest pointwise / reduction kernels of the resnet-train training step, each run on its own.

Measurement harness, not product. The step is recorded and planned exactly as the bench workload C5b does
(harness/resnet.py, he_plan_generate); the pointwise instructions of the plan are ranked by the bytes their inputs and
outputs hold, and the first N are rebuilt from the planned graph through he_pointwise_create - the same lowering and
the same generated source as inside the step - and launched back to back on random operands, two operand sets taking
turns. One line per kernel: position in the plan, plan bytes, launch shape, time per launch, rate.

    python3 -m harness.step_kernels [--top 5] [--warm 50] [--reps 100] [--batch 128] [--image 224]

Under `rocprofv3 --pmc ...` the dispatches named pointwise_kernel appear in the order of the lines printed here,
warm + reps of each in a row (their fold launches are named pointwise_kernel_finalize, fills fill_many).
"""
import argparse
import sys

import numpy as np

import helium_amd as ha
from helium_amd.backend import Plan
from harness import resnet

ELEM = {"f32": 4, "u32": 4, "bf16": 2, "f16": 2, "bool": 0}


def _bytes(dtype, numel):
    return (numel + 31) // 32 * 4 if dtype == "bool" else numel * ELEM[dtype]


def _random(dtype, numel, rng):
    if dtype == "f32" and numel == 1:
        return np.full(1, 2.0, np.float32)  # scalars of the step: the exponent of x.pow_scalar(2.0) among them
    if dtype == "f32":
        return rng.uniform(0.5, 1.5, size=numel).astype(np.float32)
    if dtype == "u32":
        return rng.integers(0, 1000, size=numel, dtype=np.uint32)
    if dtype == "bool":
        return rng.integers(0, 2 ** 32, size=(numel + 31) // 32, dtype=np.uint32)
    f = rng.standard_normal(numel).astype(np.float32)
    if dtype == "f16":
        return f.astype(np.float16).view(np.uint16)
    return (f.view(np.uint32) >> 16).astype(np.uint16)  # bf16, truncated


def ranked_pointwise_instructions(plan):
    """[(plan bytes, position among all instructions, position among the pointwise ones, node ids)], largest first."""
    g = plan.graph()
    by_id = {n["id"]: n for n in g.nodes}
    consumers = {}
    for n in g.nodes:
        for i in (n.get("inputs") or ([n["from"]] if n["node"] == "output" else [])):
            consumers.setdefault(i, []).append(n["id"])
    rows, order, pw = [], 0, 0
    for instrs, _ in plan.planned_steps():
        for kind, nodes in instrs:
            if kind == "pointwise":
                inside = set(nodes)
                ins = {i for n in nodes for i in by_id[n].get("inputs", []) if i not in inside}
                outs = {n for n in nodes if any(c not in inside for c in consumers.get(n, []))}
                total = sum(_bytes(by_id[i]["dtype"], int(np.prod(by_id[i]["shape"]))) for i in ins | outs)
                rows.append((total, order, pw, nodes))
                pw += 1
            order += 1
    rows.sort(key=lambda r: -r[0])
    return g, rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--top", type=int, default=5)
    ap.add_argument("--warm", type=int, default=50)
    ap.add_argument("--reps", type=int, default=100)
    ap.add_argument("--batch", type=int, default=128)
    ap.add_argument("--image", type=int, default=224)
    args = ap.parse_args()

    ha.device.init(0)
    stream = ha.Stream()
    rec = resnet.record_training_step(args.batch, args.image)
    graph = rec["graph"].g
    graph.optimize()
    plan = Plan(graph)
    g, rows = ranked_pointwise_instructions(plan)
    print(f"training step at batch {args.batch}, {args.image}x{args.image}: {sum(len(s[0]) for s in plan.planned_steps())} instructions, "
          f"{len(rows)} of them pointwise / reduction kernels moving {sum(r[0] for r in rows) / 1e9:.2f} GB; the {args.top} largest:", flush=True)
    rng = np.random.default_rng(0)
    for total, order, pw, nodes in rows[: args.top]:
        k = ha.TileKernel.pointwise(g, nodes)
        arg_bytes = sum(_bytes(a["dtype"], a["numel"]) for a in k.args)
        sets = []
        for _ in range(2):
            bufs = []
            for a in k.args:
                if a["is_output"]:
                    bufs.append(ha.DeviceBuffer(max(4, _bytes(a["dtype"], a["numel"]))))
                else:
                    bufs.append(ha.DeviceBuffer.from_numpy(_random(a["dtype"], a["numel"], rng)))
            sets.append(bufs)
        for i in range(args.warm):
            k.execute(sets[i % 2], stream)
        stream.synchronize()
        s, e = ha.Event(), ha.Event()
        s.record(stream)
        for i in range(args.reps):
            k.execute(sets[i % 2], stream)
        e.record(stream)
        e.synchronize()
        us = s.elapsed_ms(e) * 1e3 / args.reps
        ins = [a for a in k.args if not a["is_output"]]
        outs = [a for a in k.args if a["is_output"]]
        big = lambda xs: ", ".join(f"{a['dtype']}[{a['numel']}]" for a in xs if _bytes(a["dtype"], a["numel"]) >= 1 << 20) or "-"
        print(f"#{order} (pointwise kernel {pw} of the step), {len(nodes)} nodes: {arg_bytes / 1e6:.1f} MB of operands "
              f"({total / 1e6:.1f} MB by the plan's count), {us:.1f} us per launch incl. fold launches, {arg_bytes / us / 1e6:.2f} TB/s\n"
              f"    {k.description}\n    large inputs: {big(ins)}; {len(ins)} inputs in all\n    large outputs: {big(outs)}; {len(outs)} outputs in all",
              flush=True)
        for bufs in sets:
            for b in bufs:
                b.free()
        del k
    return 0


if __name__ == "__main__":
    sys.exit(main())
