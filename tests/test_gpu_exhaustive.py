"""Every libm-backed op on the GPU against the host libm (through the oracle).

By default: ALL 2^32 float bit patterns for the functions whose device code
differs from what the host sweep (tests/test_libm_exact_cpu.py) compiles -- tanh
(its two divisions are a reciprocal plus one correction on the device), sigmoid
(a wave-wide choice between that short division and the full one) -- and for
exp, softplus and gelu, which the benchmark workloads and those two build on,
and for powf(x, -0.75), LRN's default power
(about 12 s each: the oracle side runs on a thread pool).  The other ten run
every 61st bit pattern plus 8k-wide windows around the branch points of the
algorithms, the same set the host sweep uses; SHADOW_GPU_FULL_SWEEP=1 (or a
comma-separated list of names) sweeps all 2^32 for them too.

    SHADOW_GPU_FULL_SWEEP=1 python -m pytest tests/test_gpu_exhaustive.py -m gpu -s

tanh and sigmoid choose between a short and a long form per wave and vector (all
64 lanes, four consecutive elements each, inside |x| < 9.75 resp. |x| < 87:
short).  The sweep above hands every such choice 256 consecutive bit patterns
starting at a multiple of 256 (a tanh wave makes two, one per vector of its lanes),
and both limits are multiples of 256 as bit patterns, so there every
in-range input is computed by the short form and every other input by the long
one.  test_in_range_inputs_through_the_long_form covers what is left: all
in-range inputs again, 255 to a wave with a NaN as the 256th, which sends the
wave the long way.
"""
import concurrent.futures
import os

import numpy as np
import pytest

import oracle
from tests import gpuops
from tests.test_libm_exact_cpu import EDGES

pytestmark = pytest.mark.gpu

WANT = os.environ.get("SHADOW_GPU_FULL_SWEEP", "")
CASES = {"log": ("unary", 3), "exp": ("unary", 4), "sin": ("unary", 5), "cos": ("unary", 6),
         "tan": ("unary", 7), "asin": ("unary", 8), "acos": ("unary", 9), "atan": ("unary", 10),
         "sqrt": ("unary", 2), "reciprocal": ("unary", 14), "sigmoid": ("act", 3), "softplus": ("act", 4),
         "tanh": ("act", 5), "hardswish": ("act", 7), "gelu": ("act", 8),
         # powf(x, -0.75) through Binary's scalar form: the power LRN takes by default
         "pow_minus_three_quarters": ("pow", -0.75)}
ALWAYS_FULL = ("tanh", "sigmoid", "exp", "softplus", "gelu", "pow_minus_three_quarters")
POW = 4  # shadow/operators/kernels/binary.hpp: kAdd, kSub, kMul, kDiv, kPow, kMax, kMin
CHUNK = 1 << 26
SLICE = 1 << 21


def _oracle_slice(kind, code, x):
    if kind == "pow":
        return oracle.binary_scalar(POW, x, code)
    return oracle.unary(code, x) if kind == "unary" else oracle.activate(x, code)


def _compare(name, bits, pool):
    """Mismatches between the GPU and the oracle on the float32 values with these bit patterns."""
    kind, code = CASES[name]
    x = bits.view(np.float32)
    if kind == "pow":
        got = gpuops.binary_scalar(POW, x, code)
    else:
        got = gpuops.unary(code, x) if kind == "unary" else gpuops.activate(x, code)
    parts = [x[i:i + SLICE] for i in range(0, x.size, SLICE)]
    want = np.concatenate(list(pool.map(lambda p: _oracle_slice(kind, code, p), parts)))
    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    idx = np.flatnonzero(~same)
    return idx.size, [hex(int(v)) for v in bits[idx[:8]]]


def _full(name):
    return name in ALWAYS_FULL or WANT == "1" or name in WANT.split(",")


@pytest.mark.parametrize("name", sorted(CASES))
def test_all_float_inputs(gpu, name):
    oracle.lib()
    workers = min(16, os.cpu_count() or 1)
    bad_total, first = 0, []
    with concurrent.futures.ThreadPoolExecutor(workers) as pool:
        if _full(name):
            for start in range(0, 1 << 32, CHUNK):
                bits = np.arange(start, start + CHUNK, dtype=np.uint64).astype(np.uint32)
                bad, where = _compare(name, bits, pool)
                bad_total += bad
                first = (first + where)[:8]
                print("%s: %2d/64 chunks, %d mismatches so far" % (name, start // CHUNK + 1, bad_total), flush=True)
            covered = "2^32"
        else:
            windows = [np.arange(0, 1 << 32, 61, dtype=np.uint64)]
            for edge in EDGES:
                for sign in (0, 0x80000000):
                    lo = max(0, (edge | sign) - 4096)
                    windows.append(np.arange(lo, min(lo + 8192, 1 << 32), dtype=np.uint64))
            bits = np.concatenate(windows).astype(np.uint32)
            bad_total, first = _compare(name, bits, pool)
            covered = "%d sampled" % bits.size
    assert bad_total == 0, "%s: %d of %s inputs differ, e.g. %s" % (name, bad_total, covered, first)


WAVE_ELEMENTS = 256  # 64 lanes, one 128-bit vector each: what one wave of the elementwise kernels covers
SHORT_FORM_LIMIT = {"tanh": 0x411C0000, "sigmoid": 0x42AE0000}  # bit patterns of 9.75f and 87.0f


@pytest.mark.parametrize("name", sorted(SHORT_FORM_LIMIT))
def test_in_range_inputs_through_the_long_form(gpu, name):
    limit = SHORT_FORM_LIMIT[name]
    assert limit % WAVE_ELEMENTS == 0 and CHUNK % WAVE_ELEMENTS == 0
    oracle.lib()
    per_chunk = (CHUNK // WAVE_ELEMENTS) * (WAVE_ELEMENTS - 1)
    bad_total, first, done = 0, [], 0
    with concurrent.futures.ThreadPoolExecutor(min(16, os.cpu_count() or 1)) as pool:
        for sign in (0, 0x80000000):
            for start in range(0, limit, per_chunk):
                count = min(per_chunk, limit - start)
                groups = -(-count // (WAVE_ELEMENTS - 1))
                bits = np.full(groups * WAVE_ELEMENTS, 0x7FC00000, np.uint32)  # NaN wherever nothing else is put
                tmp = np.full(groups * (WAVE_ELEMENTS - 1), 0x7FC00000, np.uint32)
                tmp[:count] = (np.arange(start, start + count, dtype=np.uint64) | sign).astype(np.uint32)
                bits.reshape(groups, WAVE_ELEMENTS)[:, :WAVE_ELEMENTS - 1] = tmp.reshape(groups, WAVE_ELEMENTS - 1)
                bad, where = _compare(name, bits, pool)
                bad_total += bad
                first = (first + where)[:8]
                done += count
        print("%s: %d in-range inputs through the long form, %d mismatches" % (name, done, bad_total), flush=True)
    assert done == 2 * limit
    assert bad_total == 0, "%s: %d inputs differ, e.g. %s" % (name, bad_total, first)
