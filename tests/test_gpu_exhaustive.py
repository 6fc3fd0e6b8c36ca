"""Opt-in: every libm-backed op on the GPU against the host libm (through the
oracle) on ALL 2^32 float bit patterns.  Needs SHADOW_GPU_FULL_SWEEP=1, a GPU
and a few minutes of host time per function (the oracle side runs on a thread
pool); SHADOW_GPU_FULL_SWEEP=<names> restricts it, e.g. "tanh,exp".

    SHADOW_GPU_FULL_SWEEP=1 python -m pytest tests/test_gpu_exhaustive.py -m gpu -s
"""
import concurrent.futures
import os

import numpy as np
import pytest

import oracle
from tests import gpuops

pytestmark = pytest.mark.gpu

WANT = os.environ.get("SHADOW_GPU_FULL_SWEEP", "")
CASES = {"log": ("unary", 3), "exp": ("unary", 4), "sin": ("unary", 5), "cos": ("unary", 6),
         "tan": ("unary", 7), "asin": ("unary", 8), "acos": ("unary", 9), "atan": ("unary", 10),
         "sqrt": ("unary", 2), "reciprocal": ("unary", 14), "sigmoid": ("act", 3), "softplus": ("act", 4),
         "tanh": ("act", 5), "hardswish": ("act", 7), "gelu": ("act", 8)}
CHUNK = 1 << 26
SLICE = 1 << 21


def _oracle_slice(kind, code, x):
    return oracle.unary(code, x) if kind == "unary" else oracle.activate(x, code)


@pytest.mark.parametrize("name", sorted(CASES))
def test_all_float_inputs(gpu, name):
    if not WANT or (WANT != "1" and name not in WANT.split(",")):
        pytest.skip("set SHADOW_GPU_FULL_SWEEP=1 (or a list of names) to run the 2^32 sweep")
    kind, code = CASES[name]
    oracle.lib()
    workers = min(16, os.cpu_count() or 1)
    bad_total, first = 0, []
    with concurrent.futures.ThreadPoolExecutor(workers) as pool:
        for start in range(0, 1 << 32, CHUNK):
            x = np.arange(start, start + CHUNK, dtype=np.uint64).astype(np.uint32).view(np.float32)
            got = gpuops.unary(code, x) if kind == "unary" else gpuops.activate(x, code)
            parts = [x[i:i + SLICE] for i in range(0, CHUNK, SLICE)]
            want = np.concatenate(list(pool.map(lambda p: _oracle_slice(kind, code, p), parts)))
            same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
            if not same.all():
                idx = np.flatnonzero(~same)
                bad_total += idx.size
                if len(first) < 8:
                    first += [hex(int(v)) for v in x.view(np.uint32)[idx[:8]]]
            print("%s: %2d/64 chunks, %d mismatches so far" % (name, start // CHUNK + 1, bad_total), flush=True)
    assert bad_total == 0, "%s: %d of 2^32 inputs differ, e.g. %s" % (name, bad_total, first)
