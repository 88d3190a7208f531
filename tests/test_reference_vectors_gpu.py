"""The reference's own test vectors (helium/tests/autodiff.rs, loss.rs, tensor_ops.rs:172-318,379-397) through plan
generation and execute_graph on the GPU: the graphs are recorded as the reference's front end records them
(tests/reference_cases.py), the expected values are the ones the reference asserts (tests/golden/*.json)."""
import math

import numpy as np
import pytest

from oracle import numerics as nm

import reference_cases as rc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", rc.AUTODIFF, ids=lambda c: c["name"])
def test_autodiff_and_loss_vectors(gpu, case):
    G, raws = rc.record_autodiff(case)
    got = rc.evaluate_on_device(G, raws)
    for k, want in case["expected"].items():
        want = np.array(want, dtype=np.float32)
        if case.get("exact"):
            assert np.array_equal(got[k], want), (case["name"], k, got[k])
        else:
            assert nm.ulps_close(got[k], want, max_ulps=4).all(), (case["name"], k, got[k], want)


def test_gradient_descent_converges_on_the_square_root(gpu):
    """basic_gradient_descent (autodiff.rs:121-145): a fresh graph per iteration, so every iteration goes through
    plan generation (cached after the first: the graphs are structurally equal) and the executor."""
    guess = 1.0
    for _ in range(2000):
        G, error, new_guess = rc.gradient_descent_step(guess)
        got = rc.evaluate_on_device(G, {"error": error, "guess": new_guess})
        if math.sqrt(float(got["error"][0])) < 1e-3:
            break
        guess = float(got["guess"][0])
    else:
        pytest.fail("did not converge")
    assert abs(guess - math.sqrt(1001.0)) < 1e-4


@pytest.mark.parametrize("case", rc.TENSOR_OPS["matmul"], ids=lambda c: c["name"])
def test_matmul_vectors(gpu, case):
    G, raw, expected = rc.record_matmul(case)
    got = rc.evaluate_on_device(G, {"y": raw})["y"]
    assert nm.ulps_close(got, expected, max_ulps=4, epsilon=case["epsilon"]).all(), (got, expected)


def test_conv_simple(gpu):
    case = rc.TENSOR_OPS["conv"][0]
    G, raw = rc.record_conv(case)
    got = rc.evaluate_on_device(G, {"y": raw})["y"]
    assert np.array_equal(got, np.array(case["expected"], dtype=np.float32))
