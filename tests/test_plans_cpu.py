"""Which family of kernels a shape is routed to, pinned for the shapes the
benchmark tables and profiles quote (shdw_hip_softmax_plan / _normalize_plan /
_pooling2d_plan run the launching code's own decision, host only).  A threshold
that moves one of these shapes to another family fails here and has to come with
a new measurement.  (Reduce's plans: test_abi_and_host_cpu.py.)

Each entry: shape -> (path, variant, workgroups).  Paths are the SHDW_PATH_*
values of include/shadow_hip.h."""
import ctypes
import re
import os

import pytest

import shadow_amd
from shadow_amd import ints

ROWS, ROWS_STREAM, SHORT_ROWS, QUADS, PACKED, LONG_SLAB, SLAB, COLUMNS_REG, TILE, TALL, COLUMNS = range(1, 12)
PLANE_REDUCE, PLANE, PLANE_STREAM, SMALL_PLANES, BAND, WINDOW, HALVE, SAME = range(20, 28)

SOFTMAX = {  # (outer, dim, inner)
    (16, 49, 16384): (COLUMNS_REG, 64, 1024),      # softmax_channels_dense
    (64, 49, 16384): (COLUMNS_REG, 64, 4096),
    (64, 1000, 1): (SLAB, 0, 64),                   # classifier head
    (64, 150, 5329): (TILE, 6, 5376),               # 150 classes on 73 x 73
    (64, 150, 5184): (TILE, 6, 5184),
    (65536, 196, 1): (ROWS, 8, 2048),
    (64, 21, 262144): (COLUMNS_REG, 32, 65536),
    (4096, 1000, 1): (ROWS, 2, 512),
    (8192, 4096, 1): (SLAB, 0, 8192),
    (1568, 4096, 2): (SLAB, 0, 1568),
    (127, 513, 196): (TILE, 4, 1651),
    (65, 1000, 196): (TILE, 4, 845),
    (256, 256, 196): (TILE, 5, 1792),
    (513, 1000, 25): (LONG_SLAB, 0, 513),
    (3211264, 2, 2): (SHORT_ROWS, 4, 3136),
    (1605632, 8, 1): (SHORT_ROWS, 8, 1568),
    (512, 8, 3136): (COLUMNS_REG, 16, 6272),
    (802816, 16, 1): (SHORT_ROWS, 16, 784),
    (262144, 49, 1): (ROWS, 32, 2048),
    (64, 2, 200704): (QUADS, 0, 12544),
    (64, 4, 50176): (QUADS, 0, 3136),
    (100, 1000, 49): (TILE, 4, 400),
}

NORMALIZE = {  # (outer, dim, inner, p)
    (16, 49, 16384, 2.0): (COLUMNS_REG, 64, 1024),  # normalize_l2_channels_dense
    (64, 49, 16384, 2.0): (COLUMNS_REG, 64, 4096),
    (64, 512, 1, 2.0): (SLAB, 0, 64),               # embedding
    (64, 256, 3136, 2.0): (TILE, 5, 6272),
    (64, 512, 1444, 2.0): (TILE, 5, 2944),          # the SSD conv4_3 map
    (4096, 512, 1, 2.0): (ROWS_STREAM, 4, 256),
    (4096, 512, 1, 1.0): (ROWS_STREAM, 4, 256),
    (4096, 300, 1, 2.0): (ROWS, 4, 256),
    (1568, 4096, 2, 2.0): (SLAB, 0, 1568),
    (127, 513, 196, 2.0): (TILE, 4, 1651),
    (513, 1000, 25, 2.0): (LONG_SLAB, 0, 513),
    (782, 513, 32, 2.0): (LONG_SLAB, 0, 782),
    (64, 2, 200704, 2.0): (QUADS, 0, 12544),
    (64, 2, 200704, 1.0): (QUADS, 0, 12544),
    (64, 49, 16384, 3.0): (COLUMNS, 0, 16384),      # any other p: two passes with powf
    (64, 512, 1444, 3.0): (TALL, 6, 1472),
    (3211264, 2, 2, 2.0): (PACKED, 128, 25088),
    (802816, 16, 1, 2.0): (PACKED, 256, 3136),
}

POOLING = {  # ((n, c, h, w), pool type, kernel, stride, pad)
    ((16, 64, 112, 112), 0, 3, 2, 0): (BAND, 203, 7168),       # the ResNet stem
    ((64, 64, 112, 112), 0, 3, 2, 0): (BAND, 203, 4096),
    ((16, 64, 112, 112), 0, 3, 2, 1): (HALVE, 3, 6272),         # half as wide: no staging
    ((16, 64, 112, 112), 1, 2, 2, 0): (HALVE, 2, 6272),
    ((128, 2048, 7, 7), 1, 7, 1, 0): (PLANE, 0, 0),            # global average
    ((128, 2048, 7, 7), 0, 7, 1, 0): (PLANE_REDUCE, 0, 0),
    ((64, 1024, 14, 14), 1, 14, 1, 0): (PLANE, 0, 0),
    ((64, 1024, 14, 14), 0, 14, 1, 0): (PLANE_REDUCE, 0, 0),
    ((32, 512, 28, 28), 1, 28, 1, 0): (PLANE_STREAM, 0, 0),
    ((16, 256, 56, 56), 1, 56, 1, 0): (PLANE_STREAM, 0, 0),
    ((64, 1024, 14, 14), 0, 13, 1, 6): (SMALL_PLANES, 113, 16384),
    ((64, 1024, 14, 14), 1, 13, 1, 6): (SMALL_PLANES, 113, 16384),
    ((64, 1024, 14, 14), 0, 3, 1, 1): (SMALL_PLANES, 3, 16384),
    ((64, 1024, 14, 14), 0, 2, 2, 0): (SMALL_PLANES, 2, 3277),
    ((512, 512, 7, 7), 0, 7, 1, 3): (SMALL_PLANES, 107, 13108),
    ((64, 512, 19, 19), 0, 9, 1, 4): (SMALL_PLANES, 109, 10923),
    ((19, 1000, 26, 26), 0, 5, 1, 2): (SMALL_PLANES, 105, 9500),
    ((16, 64, 112, 112), 0, 5, 1, 2): (BAND, 305, 7168),
    ((16, 64, 112, 112), 0, 3, 1, 1): (SAME, 3, 12544),        # as large as its input: no staging
    ((16, 64, 112, 112), 1, 3, 1, 1): (SAME, 3, 12544),
    ((4, 3, 720, 1280), 1, 5, 3, 1): (BAND, 800, 2880),
    ((2, 3, 2000, 3000), 0, 4, 4, 0): (WINDOW, 0, 8790),
}


def ask(fn, *args):
    path, variant, grid = ctypes.c_int(), ctypes.c_int(), ctypes.c_uint()
    rc = fn(*args, ctypes.byref(path), ctypes.byref(variant), ctypes.byref(grid))
    return rc, (path.value, variant.value, grid.value)


@pytest.mark.parametrize("shape", sorted(SOFTMAX))
def test_softmax_plan(shape):
    assert ask(shadow_amd.hip().shdw_hip_softmax_plan, *shape) == (0, SOFTMAX[shape])


@pytest.mark.parametrize("shape", sorted(NORMALIZE))
def test_normalize_plan(shape):
    assert ask(shadow_amd.hip().shdw_hip_normalize_plan, *shape) == (0, NORMALIZE[shape])


@pytest.mark.parametrize("case", sorted(POOLING))
def test_pooling_plan(case):
    (n, c, h, w), pool_type, k, s, p = case
    out = [n, c, (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1]
    got = ask(shadow_amd.hip().shdw_hip_pooling2d_plan, ints([n, c, h, w]), pool_type, k, k, s, s, p, p, ints(out))
    assert got == (0, POOLING[case])


def test_pooling_plan_of_the_stem_with_the_output_size_rounded_up():
    """3x3 at stride 2 without padding on 112 x 112 with Shadow's default rounding gives 56 x 56: the last window
    of a row hangs over by one column, and the row is still half as wide as its input."""
    lib = shadow_amd.hip()
    for n, grid in ((16, 6272), (64, 25088)):
        got = ask(lib.shdw_hip_pooling2d_plan, ints([n, 64, 112, 112]), 0, 3, 3, 2, 2, 0, 0, ints([n, 64, 56, 56]))
        assert got == (0, (HALVE, 3, grid))


def test_plans_of_empty_and_invalid_shapes():
    lib = shadow_amd.hip()
    assert ask(lib.shdw_hip_softmax_plan, 0, 5, 7) == (0, (0, 0, 0))
    assert ask(lib.shdw_hip_normalize_plan, 4, 0, 7, 2.0) == (0, (0, 0, 0))
    assert ask(lib.shdw_hip_softmax_plan, -1, 5, 7)[0] == -1
    assert ask(lib.shdw_hip_softmax_plan, 1 << 20, 1 << 10, 1 << 10)[0] == -1  # more than 2^31 - 1 elements
    assert lib.shdw_hip_softmax_plan(4, 5, 7, None, None, None) == 0
    assert ask(lib.shdw_hip_pooling2d_plan, ints([1, 1, 4, 4]), 2, 2, 2, 2, 2, 0, 0, ints([1, 1, 2, 2]))[0] == -1
    assert ask(lib.shdw_hip_pooling2d_plan, ints([1, 1, 4, 4]), 0, 0, 2, 2, 2, 0, 0, ints([1, 1, 2, 2]))[0] == -1


def test_path_values_match_the_header():
    text = open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "shadow_hip.h")).read()
    found = {m.group(1): int(m.group(2)) for m in re.finditer(r"SHDW_PATH_(\w+) = (\d+)", text)}
    mine = {"ROWS": ROWS, "ROWS_STREAM": ROWS_STREAM, "SHORT_ROWS": SHORT_ROWS, "QUADS": QUADS, "PACKED": PACKED,
            "LONG_SLAB": LONG_SLAB, "SLAB": SLAB, "COLUMNS_REG": COLUMNS_REG, "TILE": TILE, "TALL": TALL,
            "COLUMNS": COLUMNS, "POOL_PLANE_REDUCE": PLANE_REDUCE, "POOL_PLANE": PLANE,
            "POOL_PLANE_STREAM": PLANE_STREAM, "POOL_SMALL_PLANES": SMALL_PLANES, "POOL_BAND": BAND,
            "POOL_WINDOW": WINDOW, "POOL_HALVE": HALVE, "POOL_SAME": SAME, "NONE": 0}
    assert found == mine
