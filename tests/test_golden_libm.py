"""Known-answer vectors recorded from glibc 2.35 (tests/golden/make_libm_kat.py).

CPU part: the oracle on THIS host must reproduce them, i.e. the host libm is the
one the vectors came from; if it is not, the GPU-vs-oracle comparisons elsewhere
are comparisons against a different libm and this test says so.
GPU part: the device restatements reproduce every recorded value bit for bit."""
import os

import numpy as np
import pytest

import oracle
from tests.helpers import assert_bit_exact

KAT = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "libm_glibc235.npz"))

UNARY = {"log": 3, "exp": 4, "sin": 5, "cos": 6, "tan": 7, "asin": 8, "acos": 9, "atan": 10}
ACT = {"sigmoid": 3, "softplus": 4, "tanh": 5, "gelu": 8}


@pytest.mark.parametrize("name", sorted(UNARY))
def test_host_libm_matches_recorded_unary(name):
    assert_bit_exact(oracle.unary(UNARY[name], KAT["x"]), KAT["unary_" + name], name)


@pytest.mark.parametrize("name", sorted(ACT))
def test_host_libm_matches_recorded_activation(name):
    assert_bit_exact(oracle.activate(KAT["x"], ACT[name]), KAT["act_" + name], name)


def test_host_libm_matches_recorded_pow():
    assert_bit_exact(oracle.binary(4, KAT["pow_a"], KAT["pow_b"]), KAT["pow"], "pow")


@pytest.mark.gpu
def test_gpu_reproduces_recorded_values(gpu):
    from tests import gpuops
    for name, op in UNARY.items():
        assert_bit_exact(gpuops.unary(op, KAT["x"]), KAT["unary_" + name], name)
    for name, act in ACT.items():
        assert_bit_exact(gpuops.activate(KAT["x"], act), KAT["act_" + name], name)
    assert_bit_exact(gpuops.binary(4, KAT["pow_a"], KAT["pow_b"]), KAT["pow"], "pow")
