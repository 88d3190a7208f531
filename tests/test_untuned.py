"""The production configuration: HELIUM_HIP_TUNING unset (the rest of the suite runs with it set, because tests steer
the generators through overrides). Overrides must then be ignored, cache keys carry no tuning prefix, and the kernels
must still match the oracle on the device."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(code, **extra_env):
    env = {k: v for k, v in os.environ.items() if not k.startswith("HELIUM_HIP_")}
    env.update(extra_env)
    env["PYTHONPATH"] = ROOT + os.pathsep + os.path.join(ROOT, "tests") + os.pathsep + env.get("PYTHONPATH", "")
    return subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=600)


def test_overrides_are_ignored_without_tuning_mode():
    code = """
import helium_amd as ha, gemm_cases
g, inputs, outs = gemm_cases.plain(512, 512, 256)
k = ha.TileKernel.fused(g)
print("DESC", k.description)
from helium_amd import ir
from helium_amd.backend import Plan
g2 = ir.OpGraph()
x = g2.new_input([64, 64], "f32"); g2.new_output(g2.unary(x, "relu"))
print("PLAN", sum(len(instrs) for instrs, _ in Plan(g2).steps))
"""
    r = _run(code, HELIUM_HIP_GEMM_TILE="128,128,64,2,2", HELIUM_HIP_GEMM_NO_DIRECT="1")
    assert r.returncode == 0, r.stderr[-2000:]
    desc = [l for l in r.stdout.splitlines() if l.startswith("DESC")][0]
    assert "tile=128x128x64" not in desc and "direct=11" in desc, desc
    assert "PLAN 1" in r.stdout
    # the same overrides are honoured in tuning mode
    r = _run(code, HELIUM_HIP_TUNING="1", HELIUM_HIP_GEMM_TILE="128,128,64,2,2", HELIUM_HIP_GEMM_NO_DIRECT="1")
    assert r.returncode == 0, r.stderr[-2000:]
    desc = [l for l in r.stdout.splitlines() if l.startswith("DESC")][0]
    assert "tile=128x128x64" in desc and "direct=00" in desc, desc


@pytest.mark.gpu
def test_the_hot_path_matches_the_oracle_without_tuning_mode(gpu):
    """One small pass of every part of the path (permute, fused GEMM, execute_graph, convolution) in a process of its
    own with tuning mode off, each checked against the oracle."""
    r = _run("import __graft_entry__ as e; e.smoke(); print('UNTUNED OK')")
    assert r.returncode == 0 and "UNTUNED OK" in r.stdout, (r.stdout[-1500:], r.stderr[-1500:])
