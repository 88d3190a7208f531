"""Generation-time overrides (HELIUM_HIP_GEMM_TILE and friends) are part of the kernel-cache and plan-cache keys while
tuning mode is on, and dead while it is off."""
import os
import subprocess
import sys

import helium_amd as ha
from helium_amd.backend import Plan

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _graph():
    g = ha.ir.OpGraph()
    a, b = g.new_input([1024, 1024], "bf16"), g.new_input([1024, 1024], "bf16")
    g.new_output(g.matmul(a, b, "bf16_f32"))
    return g


def _kernels_requested():
    """How many kernels have been asked of the compiler so far (compiled, or found in its memory / disk cache)."""
    return sum(ha.device.rtc_stats().values())


def _precompile(g):
    before = _kernels_requested()
    Plan(g).precompile()
    return _kernels_requested() - before


def test_a_changed_override_is_not_served_a_kernel_built_under_another(monkeypatch):
    # conftest switches tuning mode on for the test process
    monkeypatch.setenv("HELIUM_HIP_GEMM_TILE", "64,64,64,2,2")
    assert _precompile(_graph()) >= 1          # generated under this override
    assert _precompile(_graph()) == 0          # a structurally equal graph: plan cache and kernel cache both hit
    monkeypatch.setenv("HELIUM_HIP_GEMM_TILE", "128,128,64,2,2")
    assert _precompile(_graph()) >= 1          # same graph, other override: generated anew
    assert _precompile(_graph()) == 0
    monkeypatch.setenv("HELIUM_HIP_GEMM_TILE", "64,64,64,2,2")
    assert _precompile(_graph()) == 0          # and the first one is still there under its own key


def test_overrides_are_dead_without_tuning_mode():
    code = (
        "import sys; sys.path.insert(0, %r)\n"
        "import helium_amd as ha\n"
        "g = ha.ir.OpGraph(); a = g.new_input([1024, 1024], 'bf16'); b = g.new_input([1024, 1024], 'bf16')\n"
        "g.new_output(g.matmul(a, b, 'bf16_f32'))\n"
        "print(ha.backend.matmul_kernel(g, [2]).description)\n" % ROOT
    )
    env = {k: v for k, v in os.environ.items() if k != "HELIUM_HIP_TUNING"}
    env["HELIUM_HIP_GEMM_TILE"] = "128,128,64,2,2"
    env["HELIUM_HIP_GEMM_SKIP"] = "7"
    plain = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert plain.returncode == 0, plain.stderr
    assert "tile=128x128x64" not in plain.stdout
    tuned = subprocess.run([sys.executable, "-c", code], env=dict(env, HELIUM_HIP_TUNING="1"), capture_output=True, text=True, timeout=300)
    assert tuned.returncode == 0 and "tile=128x128x64" in tuned.stdout
