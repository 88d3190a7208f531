"""The measurement programs under harness/ that the profiles cite: what they do without a GPU (the probe kernels compile
for gfx950; the step-kernel ranking names the plan's instructions and rebuilds them with the library's own lowering)."""
import numpy as np

import helium_amd as ha
from helium_amd import device
from helium_amd.backend import Plan
from harness import gfx950_probes, resnet, step_kernels


def test_probe_kernels_compile_for_gfx950():
    cases = [(gfx950_probes.MFMA_LDS, dict(NA=1, NTR=1, BARRIER=1, ITERS=10)),
             (gfx950_probes.LOAD_COST, dict(NL=2, ITERS=10)),
             (gfx950_probes.STREAM, dict(DRAIN=0, BARRIER=1))]
    for src, defines in cases:
        head = "".join(f"#define {k} {v}\n" for k, v in defines.items())
        code = device.rtc_compile(head + src, "probe", ["-O3"])
        assert code[:4] == b"\x7fELF"


def test_step_kernels_ranks_and_rebuilds_the_pointwise_instructions_of_a_plan():
    rec = resnet.record_training_step(8, 64, width=8, num_classes=16)
    graph = rec["graph"].g
    graph.optimize()
    plan = Plan(graph)
    g, rows = step_kernels.ranked_pointwise_instructions(plan)
    instrs = [i for step, _ in plan.planned_steps() for i in step]
    assert len(rows) == sum(1 for kind, _ in instrs if kind == "pointwise")
    assert [r[0] for r in rows] == sorted((r[0] for r in rows), reverse=True)
    assert sorted(r[2] for r in rows) == list(range(len(rows)))
    for total, order, pw, nodes in rows[:3]:
        assert instrs[order] == ("pointwise", nodes)
        k = ha.TileKernel.pointwise(g, nodes)
        operands = sum(step_kernels._bytes(a["dtype"], a["numel"]) for a in k.args)
        assert operands == total, (k.description, operands, total)
        for a in k.args:
            if not a["is_output"]:
                v = step_kernels._random(a["dtype"], a["numel"], np.random.default_rng(0))
                assert v.nbytes == max(step_kernels._bytes(a["dtype"], a["numel"]), v.itemsize)
