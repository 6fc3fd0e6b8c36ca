"""The device math restatements (shadow_amd/csrc/libm_exact.h), compiled for the
host, against this machine's libm -- the arithmetic the oracle and the reference
use.  The default run covers every 61st bit pattern plus dense windows around
the algorithms' branch points (~10 s); SHADOW_LIBM_FULL=1 sweeps all 2^32
patterns of each function (~2 min on 8 cores)."""
import ctypes
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
FUNCS = {"exp": 0, "tanh": 1, "sigmoid": 2, "expm1": 3}
# float bit patterns where the restated algorithms switch paths
EDGES = [0x00000000, 0x00800000, 0x24000000, 0x33000000, 0x3eb17218, 0x3f000000, 0x3f800000,
         0x3F851592, 0x4195b844, 0x41b00000, 0x42b00000, 0x42b17218, 0x42cff1b5, 0x42ce8ed0,
         0x7f800000]


@pytest.fixture(scope="module")
def sweep():
    lib = ctypes.CDLL(os.path.join(HERE, "native", "libm_sweep.so"))
    lib.libm_sweep.restype = ctypes.c_longlong
    lib.libm_sweep.argtypes = [ctypes.c_int, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_uint32,
                               ctypes.c_int, ctypes.POINTER(ctypes.c_uint32), ctypes.c_int]
    return lib


@pytest.mark.parametrize("name", sorted(FUNCS))
def test_restatement_matches_host_libm(sweep, name):
    rep = (ctypes.c_uint32 * 8)()
    threads = min(8, os.cpu_count() or 1)

    def run(start, count, stride):
        bad = sweep.libm_sweep(FUNCS[name], start, count, stride, threads, rep, 8)
        assert bad == 0, "%s: %d mismatches, e.g. input bits %s" % (
            name, bad, [hex(v) for v in rep[:min(bad, 8)]])

    if os.environ.get("SHADOW_LIBM_FULL"):
        run(0, 1 << 32, 1)
        return
    run(0, (1 << 32) // 61 + 1, 61)
    for edge in EDGES:
        for sign in (0, 0x80000000):
            lo = max(0, (edge | sign) - 4096)
            run(lo, 8192, 1)
