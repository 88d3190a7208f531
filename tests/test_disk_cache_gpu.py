"""The kernel disk cache on the device (the reference hints at one: helium-kernel-generator/Cargo.toml:42-44): a
code object that a process finds on disk loads and computes what the oracle does, and a file whose payload the device
rejects is compiled afresh."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# creates the config-3 auxiliary kernel (chain of ten pointwise ops and two sums) at a small size, runs it and compares
# with the oracle's float64 sums; prints the compile / disk-hit counters seen up to then
CHILD = r"""
import json, sys
import numpy as np
import helium_amd as ha
from helium_amd import configs, device
from oracle import fusion_ir as oracle
from helpers import run_tile_kernel_gpu
device.init(0)
g, inputs, outs = configs.c3_chain(256, 384, seed=11)
k = ha.TileKernel.auxiliary(g)
got = run_tile_kernel_gpu(k, inputs)
want = oracle.outputs(g.nodes, inputs)
assert set(got) == set(want)
worst = 0.0
for leaf, w in want.items():
    a = got[leaf].astype(np.float64)
    w = w.reshape(-1).astype(np.float64)
    worst = max(worst, float(np.abs(a - w).max() / max(np.abs(w).max(), 1e-30)))
print("STATS", json.dumps(dict(device.rtc_stats(), worst=worst)))
"""


def _child(cache_dir):
    env = dict(os.environ, HELIUM_HIP_CACHE_DIR=str(cache_dir))
    env["PYTHONPATH"] = ROOT + os.pathsep + os.path.join(ROOT, "tests") + os.pathsep + env.get("PYTHONPATH", "")
    out = subprocess.run([sys.executable, "-c", CHILD], env=env, capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr[-3000:]
    return json.loads([l for l in out.stdout.splitlines() if l.startswith("STATS")][0][6:])


def test_a_kernel_served_from_disk_loads_and_matches_the_oracle(gpu, tmp_path):
    first = _child(tmp_path)
    assert first["compiles"] >= 1 and first["disk_hits"] == 0 and first["worst"] <= 1e-3, first
    files = sorted(f for f in os.listdir(tmp_path) if f.endswith(".hekc"))
    assert files
    second = _child(tmp_path)   # a fresh process: every code object comes from the files of the first
    assert second["compiles"] == 0 and second["disk_hits"] == first["compiles"] and second["worst"] <= 1e-3, second


def test_the_shipped_cache_serves_the_benchmark_kernel(gpu):
    """The in-tree cache that build() fills is what a GPU box starts from: the config-3 kernel at the benchmark's size
    must come out of it without a compile."""
    code = CHILD.replace("configs.c3_chain(256, 384, seed=11)", "configs.c3_chain(4096, 4096, seed=11)")
    env = {k: v for k, v in os.environ.items() if k not in ("HELIUM_HIP_CACHE_DIR", "HELIUM_HIP_TUNING")}
    env["PYTHONPATH"] = ROOT + os.pathsep + os.path.join(ROOT, "tests") + os.pathsep + env.get("PYTHONPATH", "")
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=900)
    assert out.returncode == 0, out.stderr[-3000:]
    stats = json.loads([l for l in out.stdout.splitlines() if l.startswith("STATS")][0][6:])
    assert stats["compiles"] == 0 and stats["disk_hits"] >= 1 and stats["worst"] <= 1e-3, stats


def test_a_payload_the_device_rejects_is_compiled_afresh(gpu, tmp_path):
    """A file with a sound header and checksum whose payload is no code object for this device (a cache directory
    carried over from another machine): loading falls back to a fresh compile past the caches."""
    import struct

    first = _child(tmp_path)
    assert first["worst"] <= 1e-3
    for name in os.listdir(tmp_path):
        if not name.endswith(".hekc"):
            continue
        path = os.path.join(tmp_path, name)
        blob = open(path, "rb").read()
        header, payload = blob[:32], bytearray(blob[32:])
        # an ELF that names another machine: e_machine (offset 18) and e_flags (offset 48) zeroed
        payload[18:20] = b"\x00\x00"
        payload[48:52] = b"\x00\x00\x00\x00"
        # FNV-1a 64 over the payload, as the cache's header stores it
        h = 0xcbf29ce484222325
        for byte in payload:
            h = ((h ^ byte) * 0x100000001b3) & 0xFFFFFFFFFFFFFFFF
        magic, fmt, reserved, length, _ = struct.unpack("<8sIIQQ", header)
        assert magic == b"HEKCACHE" and length == len(payload)
        open(path, "wb").write(struct.pack("<8sIIQQ", magic, fmt, reserved, length, h) + bytes(payload))
    again = _child(tmp_path)
    assert again["worst"] <= 1e-3, again
