"""he_tile_kernel_execute_noalloc: the launches of he_tile_kernel_execute with the kernels' scratch in the library's
static device array. Its outputs must equal the allocating entry point's bit for bit (the partial results are folded in
a fixed order), call after call on the one shared array, whatever the previous call left there."""
import re

import numpy as np
import pytest

import helium_amd as ha
from helium_amd import configs

pytestmark = pytest.mark.gpu


def _aux_case(rows, cols, seed):
    g, inputs, _ = configs.c3_chain(rows, cols, seed=seed)
    return ha.TileKernel.auxiliary(g), inputs


def _gemm_case(size, seed):
    g, _ = configs.c4_graph(size)
    return ha.TileKernel.fused(g), configs.c4_inputs(g, size, seed=seed)


def _run(kernel, inputs, noalloc):
    bufs, outs = [], []
    for a in kernel.args:
        if a["is_output"]:
            nbytes = a["numel"] * (4 if a["dtype"] in ("f32", "u32") else 2)
            b = ha.DeviceBuffer(nbytes)
            b.fill_u8(0xA5)  # an output the kernel fails to write shows
            outs.append((b, a))
            bufs.append(b)
        else:
            bufs.append(ha.DeviceBuffer.from_numpy(inputs[a["node"]]))
    (kernel.execute_noalloc if noalloc else kernel.execute)(bufs)
    return [b.to_numpy(np.float32 if a["dtype"] == "f32" else np.uint16) for b, a in outs]


def test_outputs_equal_the_allocating_entry_point_call_after_call(gpu):
    # reductions whose partials meet in scratch: an auxiliary kernel with arrival counters (1024 x 1024: folds inside
    # the kernel), a fused GEMM with a fold launch, then the same two kinds again, smaller, on whatever those left
    cases = [_aux_case(1024, 1024, 5), _gemm_case(512, 6), _aux_case(256, 384, 7), _gemm_case(256, 8)]
    assert "ws_counters=0" not in cases[0][0].description or "ws_counters=0" not in cases[2][0].description
    want = [_run(k, inp, noalloc=False) for k, inp in cases]
    for round_ in range(2):
        for (k, inp), w in zip(cases, want):
            got = _run(k, inp, noalloc=True)
            assert len(got) == len(w) and len(w) >= 2
            for a, b in zip(got, w):
                assert np.array_equal(a, b), (k.description, round_)


def test_first_call_on_a_gemm_with_arrival_counters_loads_nothing(gpu):
    """A small fused GEMM folds its column sums inside the kernel (arrival counters, cleared by the library's fill kernel
    at the head of every allocation-free call). Created after he_init, its first call must find every code object
    loaded - the fill kernel's included - so the call neither compiles nor looks anything up."""
    import gemm_cases
    from helium_amd import device

    g, inputs, _ = gemm_cases.bias_relu_colsum(192, 320, 128)
    k = ha.TileKernel.fused(g)
    assert int(re.search(r"reduce_counters=(\d+)", k.description).group(1)) > 0, k.description
    before = device.rtc_stats()
    got = _run(k, inputs, noalloc=True)   # the allocation-free entry point first: nothing was launched before
    assert device.rtc_stats() == before
    want = _run(k, inputs, noalloc=False)
    assert len(got) == len(want) >= 2
    for a, b in zip(got, want):
        assert np.array_equal(a, b), k.description


def test_a_kernel_that_needs_more_scratch_is_refused(gpu):
    g, _, _ = configs.c3_chain(16384, 16384, make_inputs=False)
    k = ha.TileKernel.auxiliary(g)
    floats = int(re.search(r"ws_floats=(\d+)", k.description).group(1))
    assert floats * 4 > (8 << 20)
    dummy = [ha.DeviceBuffer(256) for _ in k.args]
    with pytest.raises(ha.HeliumError, match="allocation-free entry point holds"):
        k.execute_noalloc(dummy)
