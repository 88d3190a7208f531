"""The kernel disk cache (the reference only hints at one: helium-kernel-generator/Cargo.toml:42-44, feature
`disk-cache`): a second process finds the first one's code object, and a file that is damaged is compiled again."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r"""
import sys
sys.path.insert(0, %r)
from helium_amd import device
src = 'extern "C" __global__ void cached_probe(float* x) { x[threadIdx.x] = x[threadIdx.x] * 3.0f + 1.0f; }'
code = device.rtc_compile(src, "cached_probe")
assert code[:4] == b"\x7fELF", code[:8]
s = device.rtc_stats()
print(s["compiles"], s["disk_hits"], len(code))
""" % ROOT


def _child(cache_dir):
    env = dict(os.environ, HELIUM_HIP_CACHE_DIR=str(cache_dir))
    out = subprocess.run([sys.executable, "-c", CHILD], env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    compiles, disk_hits, size = (int(v) for v in out.stdout.split())
    return compiles, disk_hits, size


def test_second_process_hits_the_disk_and_damaged_files_are_recompiled(tmp_path):
    compiles, disk_hits, size = _child(tmp_path)
    assert (compiles, disk_hits) == (1, 0)
    files = [f for f in os.listdir(tmp_path) if f.endswith(".hekc")]
    assert len(files) == 1 and not [f for f in os.listdir(tmp_path) if ".tmp" in f]
    path = os.path.join(tmp_path, files[0])
    good = open(path, "rb").read()
    assert len(good) > size and good[:8] == b"HEKCACHE"

    assert _child(tmp_path) == (0, 1, size)          # found on disk, nothing compiled

    open(path, "wb").write(good[: len(good) // 2])   # truncated (an interrupted copy)
    assert _child(tmp_path) == (1, 0, size)
    assert open(path, "rb").read() == good           # and written afresh

    flipped = bytearray(good)
    flipped[-100] ^= 0x40                            # one bit of the code object
    open(path, "wb").write(bytes(flipped))
    assert _child(tmp_path) == (1, 0, size)

    open(path, "wb").write(good[32:])                # a bare code object, as an older format stored it
    assert _child(tmp_path) == (1, 0, size)
    assert _child(tmp_path) == (0, 1, size)


def test_cache_can_be_switched_off(tmp_path):
    env = dict(os.environ, HELIUM_HIP_CACHE_DIR="off")
    out = subprocess.run([sys.executable, "-c", CHILD], env=env, capture_output=True, text=True, timeout=300, cwd=tmp_path)
    assert out.returncode == 0, out.stderr
    assert out.stdout.split()[:2] == ["1", "0"] and not os.listdir(tmp_path)
