"""The device pool on the GPU, in the spirit of the reference's allocator/device.rs:208-234 (random allocations never
overlap): every live allocation is stamped with a value of its own when it is made and must still hold it when it is
released, across scopes and from two host threads at once."""
import ctypes as C
import threading

import numpy as np
import pytest

from helium_amd import allocator
from helium_amd._ffi import check, lib
from helium_amd.backend import stats

pytestmark = pytest.mark.gpu


def _stamp(ptr, nbytes, value):
    check(lib.he_memset_d32_async(C.c_void_p(ptr), value, nbytes // 4, None))


def _read_ends(ptr, nbytes):
    out = np.zeros(2, dtype=np.uint32)
    check(lib.he_memcpy_d2h_async(out.ctypes.data_as(C.c_void_p), C.c_void_p(ptr), 4, None))
    check(lib.he_memcpy_d2h_async(out[1:].ctypes.data_as(C.c_void_p), C.c_void_p(ptr + nbytes - 4), 4, None))
    check(lib.he_device_synchronize())
    return out


def _churn(seed, thread_token, errors, steps=400):
    try:
        rng = np.random.default_rng(seed)
        live = []  # (ptr, block, nbytes, stamp, scope)
        scope = allocator.pool_begin_scope(thread_token)
        for step in range(steps):
            if step % 50 == 49:  # a new scope; the old one's device work is over (everything here is synchronous)
                for ptr, block, nbytes, stamp, s in [x for x in live if x[4] == scope]:
                    assert (_read_ends(ptr, nbytes) == stamp).all()
                    allocator.pool_release(ptr, block, s)
                live = [x for x in live if x[4] != scope]
                allocator.pool_end_scope(scope)
                scope = allocator.pool_begin_scope(thread_token)
            if not live or rng.random() < 0.55:
                nbytes = int(rng.integers(1, 8 << 20)) * 4
                ptr, block = allocator.pool_allocate(nbytes, scope)
                assert ptr % 256 == 0 and block.size >= nbytes
                stamp = (seed << 20) + step
                _stamp(ptr, nbytes, stamp)
                for optr, _, onb, _, _ in live:
                    assert ptr + nbytes <= optr or optr + onb <= ptr, "live allocations overlap"
                live.append((ptr, block, nbytes, stamp, scope))
            else:
                ptr, block, nbytes, stamp, s = live.pop(int(rng.integers(len(live))))
                assert (_read_ends(ptr, nbytes) == stamp).all(), "an allocation was written by someone else"
                allocator.pool_release(ptr, block, s)
        for ptr, block, nbytes, stamp, s in live:
            assert (_read_ends(ptr, nbytes) == stamp).all()
            allocator.pool_release(ptr, block, s)
        allocator.pool_end_scope(scope)
    except BaseException as e:  # noqa: BLE001 - reported by the test's own thread
        errors.append(e)


def test_random_allocations_across_scopes_and_two_threads_never_overlap(gpu):
    before = stats()
    errors = []
    threads = [threading.Thread(target=_churn, args=(seed, 1000 + seed, errors)) for seed in (1, 2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise errors[0]
    after = stats()
    # memory comes in pages of at least 1 GiB and is handed out again rather than fetched anew
    assert after["pool_driver_allocs"] - before["pool_driver_allocs"] <= 4
    assert after["pool_reuses"] - before["pool_reuses"] >= 300
    assert (after["pool_bytes"] - before["pool_bytes"]) % (1 << 30) == 0


def test_a_failing_execution_still_ends_its_scope(gpu):
    """A graph whose input storage is missing fails before any device work; one whose instruction fails half way
    leaves queued work behind: in both cases the pool must not keep a scope open."""
    import helium_amd as ha
    from helium_amd.backend import Tensor, execute_graph

    g = ha.ir.OpGraph()
    x = g.new_input([64, 64], "f32")
    y = g.new_input([64, 64], "f32")
    g.new_output(g.binary(g.unary(x, "exp"), y, "add"))
    xs = Tensor.from_numpy(np.ones((64, 64), dtype=np.float32), "f32")
    with pytest.raises(ha.HeliumError):
        execute_graph(g, {x: xs})
    out = execute_graph(g, {x: xs, y: xs})
    (t,) = out.values()
    assert np.allclose(t.to_numpy(), np.e + 1.0)
