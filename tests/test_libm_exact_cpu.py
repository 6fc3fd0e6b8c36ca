"""The device math restatements (shadow_amd/csrc/libm_exact.h), compiled for the
host, against this machine's libm -- the arithmetic the oracle and the reference
use.  The default run covers every 61st bit pattern plus dense windows around
the algorithms' branch points (~20 s); SHADOW_LIBM_FULL=1 sweeps all 2^32
patterns of each one-argument function and 10 x 2^32 (x, y) pairs of powf
(~10 min on 8 cores).  All of them have been swept in full with 0 mismatches
against glibc 2.35."""
import ctypes
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
FUNCS = {"exp": 0, "tanh": 1, "sigmoid": 2, "expm1": 3, "log": 4, "sin": 5, "cos": 6, "atan": 7,
         "asin": 8, "acos": 9, "log1p": 10, "erf": 11, "softplus": 12, "gelu": 13, "tan": 14}
# float bit patterns where the restated algorithms switch paths
EDGES = [0x00000000, 0x00800000, 0x04000000, 0x24000000, 0x24800000, 0x31000000, 0x31800000,
         0x32000000, 0x32800000, 0x33000000, 0x39000000, 0x39800000, 0x3eb17218, 0x3ed413d7,
         0x3e95f61f, 0x3ee00000, 0x3f000000, 0x3f2ca140, 0x3f300000, 0x3f330000, 0x3f490fda,
         0x3f580000, 0x3f79999a, 0x3f800000, 0x3F851592, 0x3f980000, 0x3fa00000, 0x3fc90fda,
         0x401c0000, 0x4036db6e, 0x40490fda, 0x40c00000, 0x411c0000, 0x41200000, 0x4195b844, 0x41b00000, 0x42b00000,
         0x42b17218, 0x42cff1b5, 0x42ce8ed0, 0x42f00000, 0x4c000000, 0x5a000000, 0x7f800000]


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


def test_tanh_step_table_holds_its_definitions(sweep):
    """kTanhStepTab[k + 3] = {k ln2_hi (exact), fl(k ln2_lo), T, off, 2^k, k >= 1} for k = -3 ... 28, with
    T = 0 (k = 0, -1), 1 (k <= -2), fl(1 - 2^-k) otherwise and off = -0.5 (k = -1), -1 (k <= -2), 0 otherwise --
    recomputed here in numpy fp32."""
    sweep.libm_tanh_step.restype = ctypes.c_int
    sweep.libm_tanh_step.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_float)]
    f = np.float32
    ln2_hi, ln2_lo = f(6.9313812256e-01), f(9.0580006145e-06)
    entry = (ctypes.c_float * 8)()
    n = sweep.libm_tanh_step(-1, entry)
    assert n == 32
    for i in range(n):
        k = i - 3
        assert sweep.libm_tanh_step(i, entry) == 32  # bytes per entry
        assert float(f(k) * ln2_hi) == k * float(ln2_hi)  # the product is exact
        T = f(0) if k in (0, -1) else (f(1) if k <= -2 else f(1) - f(2.0 ** -k))
        off = f(-0.5) if k == -1 else (f(-1) if k <= -2 else f(0))
        want = [f(k) * ln2_hi, f(k) * ln2_lo, T, off, f(2.0 ** k), f(1 if k >= 1 else 0), f(0), f(0)]
        got = np.array(list(entry), np.float32)
        assert np.array_equal(got.view(np.uint32), np.array(want, np.float32).view(np.uint32)), (k, got, want)


def test_powf_restatement_matches_host_libm(sweep):
    """y fixed at a few values and y random (all bit patterns / scaled into
    [-40, 40]) while x walks an arithmetic progression of bit patterns."""
    sweep.libm_sweep_pow.restype = ctypes.c_longlong
    sweep.libm_sweep_pow.argtypes = [ctypes.c_uint32, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint32,
                                     ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_uint32),
                                     ctypes.c_int]
    rep = (ctypes.c_uint32 * 16)()
    threads = min(8, os.cpu_count() or 1)
    full = bool(os.environ.get("SHADOW_LIBM_FULL"))
    count, stride = ((1 << 32, 1) if full else ((1 << 32) // 127 + 1, 127))
    cases = [(1, 1), (2, 2), (2, 77), (0, 0x40000000), (0, 0x3f000000), (0, 0xc0400000), (0, 0),
             (0, 0x7fa00000), (0, 0x41200000), (0, 0xbf400000)]  # the last: -0.75, the power LRN takes by default
    for mode, ybits in cases:
        bad = sweep.libm_sweep_pow(0, count, stride, ybits, mode, threads, rep, 16)
        assert bad == 0, "powf mode %d y=%#x: %d mismatches, e.g. (x, y) bits %s" % (
            mode, ybits, bad, [hex(v) for v in rep[:min(2 * bad, 8)]])
