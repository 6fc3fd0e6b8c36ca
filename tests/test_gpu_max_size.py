"""The largest tensors the int32 element counts of the interface admit: 2^31 - 1 floats
(8.6 GB) through the elementwise, per-channel, reduction, softmax, pooling, broadcast,
norm and data-moving kernels.
The expected values come from numpy or the oracle on the same data, compared in pieces
so that the host never holds more than the input and one output; the data is a 2^20-float random block
repeated, which keeps every index of the tensor in play (the last vector ends
three floats short) without minutes of random-number generation."""
import numpy as np
import pytest

import oracle
import shadow_amd
from shadow_amd import Buffer, check, ints
from tests import gpuops
from tests.helpers import bits, normal

pytestmark = pytest.mark.gpu
F = np.float32
N = 2 ** 31 - 1
PIECE = 1 << 26


@pytest.fixture(scope="module")
def big():
    block = normal(901, 1 << 20, 2.0)
    block[::97] = 0.0
    block[5::1013] = -0.0
    x = np.tile(block, N // block.size + 1)[:N]
    dx = Buffer.from_numpy(x)
    dy = Buffer(4 * N)
    yield x, dx, dy
    dx.free()
    dy.free()


def same_in_pieces(dy, want_of, what):
    """dy against want_of(lo, hi) piece by piece, bit for bit."""
    got = dy.download(count=N)
    for lo in range(0, N, PIECE):
        hi = min(N, lo + PIECE)
        w = want_of(lo, hi)
        if not np.array_equal(bits(got[lo:hi]), bits(np.asarray(w, F))):
            bad = lo + int(np.flatnonzero(bits(got[lo:hi]) != bits(np.asarray(w, F)))[0])
            raise AssertionError("%s: first difference at element %d of %d" % (what, bad, N))


def test_elementwise_at_the_largest_count(gpu, big):
    x, dx, dy = big
    lib = shadow_amd.hip()
    check(lib.shdw_hip_activate(1, 0.0, N, dx.ptr, dy.ptr, None))  # relu: x > 0 ? x : 0
    gpuops._sync()
    same_in_pieces(dy, lambda lo, hi: np.where(x[lo:hi] > 0, x[lo:hi], F(0)), "relu")
    check(lib.shdw_hip_unary(0, N, dx.ptr, dy.ptr, None))  # abs
    gpuops._sync()
    same_in_pieces(dy, lambda lo, hi: np.abs(x[lo:hi]), "abs")
    check(lib.shdw_hip_binary(0, N, dx.ptr, dx.ptr, dy.ptr, None))  # x + x
    gpuops._sync()
    same_in_pieces(dy, lambda lo, hi: x[lo:hi] + x[lo:hi], "add")


def test_scale_at_the_largest_count(gpu, big):
    x, dx, dy = big
    lib = shadow_amd.hip()
    num, inner = 7, 1 << 20  # rows of a mebi-float, the last one cut short by the end of the tensor
    scale = np.linspace(0.5, 2.0, num).astype(F)
    bias = np.linspace(-1.0, 1.0, num).astype(F)
    ds, db = Buffer.from_numpy(scale), Buffer.from_numpy(bias)
    check(lib.shdw_hip_scale_bias(N, num, inner, dx.ptr, ds.ptr, db.ptr, 0, dy.ptr, None))
    gpuops._sync()

    def want(lo, hi):
        c = (np.arange(lo, hi, dtype=np.int64) // inner) % num
        t = x[lo:hi] * scale[c]  # a rounded multiply, then a rounded add
        return t + bias[c]
    same_in_pieces(dy, want, "scale + bias")
    ds.free()
    db.free()


def test_reduce_at_the_largest_count(gpu, big):
    x, dx, dy = big
    lib = shadow_amd.hip()
    shape, axes = [N], [0]
    need = lib.shdw_hip_reduce_workspace_bytes(1, ints(shape), 1, ints(axes))
    ws = Buffer(max(16, need))
    for op, want in ((2, x.max()), (3, x.min())):
        check(lib.shdw_hip_reduce(op, 1, ints(shape), 1, ints(axes), dx.ptr, dy.ptr, ws.ptr, need, None))
        gpuops._sync()
        got = dy.download(count=1)[0]
        assert bits(np.array([got], F))[0] == bits(np.array([want], F))[0], (op, got, want)
    total = float(np.sum(x, dtype=np.float64))
    l1 = float(np.sum(np.abs(x), dtype=np.float64))
    for op, want in ((1, total), (5, l1), (4, total / N)):
        check(lib.shdw_hip_reduce(op, 1, ints(shape), 1, ints(axes), dx.ptr, dy.ptr, ws.ptr, need, None))
        gpuops._sync()
        got = float(dy.download(count=1)[0])
        assert abs(got - want) <= 1e-5 * abs(want) + 1e-3, (op, got, want)
    # two reduced axes around a kept one: [k][3][m] over axes 0 and 2
    m = 1 << 10
    k = (N // (3 * m))
    shape, axes = [k, 3, m], [0, 2]
    need = lib.shdw_hip_reduce_workspace_bytes(3, ints(shape), 2, ints(axes))
    ws2 = Buffer(max(16, need))
    check(lib.shdw_hip_reduce(1, 3, ints(shape), 2, ints(axes), dx.ptr, dy.ptr, ws2.ptr, need, None))
    gpuops._sync()
    got = dy.download(count=3).astype(np.float64)
    want = x[:k * 3 * m].reshape(k, 3, m).sum(axis=(0, 2), dtype=np.float64)
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-2), (got, want)
    ws.free()
    ws2.free()


# Softmax over the last axis of as many rows as fit: the first, a middle and the last million rows against
# the oracle bit for bit, and every row through a property that does not depend on the size: the row sums
# (Reduce over axis 1, then max and min of those on the device) lie within rounding of 1.
@pytest.mark.parametrize("dim", [2, 21, 1000])
def test_softmax_over_the_last_axis_at_the_largest_count(gpu, big, dim):
    x, dx, dy = big
    lib = shadow_amd.hip()
    outer = N // dim
    check(lib.shdw_hip_softmax(outer, dim, 1, dx.ptr, dy.ptr, None))
    gpuops._sync()
    rows = min(outer, (1 << 20) // dim * 4)
    for r0 in (0, (outer - rows) // 2, outer - rows):
        got = dy.download(count=rows * dim, offset_bytes=4 * r0 * dim)
        want = oracle.softmax(x[r0 * dim:(r0 + rows) * dim], rows, dim, 1)
        assert np.array_equal(bits(got), bits(np.asarray(want, F).ravel())), "softmax rows from %d" % r0
    sums = Buffer(4 * outer)
    shape, axes = [outer, dim], [1]
    need = lib.shdw_hip_reduce_workspace_bytes(2, ints(shape), 1, ints(axes))
    ws = Buffer(max(16, need))
    check(lib.shdw_hip_reduce(1, 2, ints(shape), 1, ints(axes), dy.ptr, sums.ptr, ws.ptr, need, None))
    out = Buffer(16)
    need2 = lib.shdw_hip_reduce_workspace_bytes(1, ints([outer]), 1, ints([0]))
    ws2 = Buffer(max(16, need2))
    ends = []
    for op in (2, 3):
        check(lib.shdw_hip_reduce(op, 1, ints([outer]), 1, ints([0]), sums.ptr, out.ptr, ws2.ptr, need2, None))
        gpuops._sync()
        ends.append(float(out.download(count=1)[0]))
    assert 1 - 1e-5 <= ends[1] <= ends[0] <= 1 + 1e-5, ends
    for b in (sums, ws, ws2, out):
        b.free()


# The stem's 3x3 stride-2 max pooling and a whole-plane average on a tensor of 2^31 - 2^20 floats: the first
# and the last planes against the oracle.
def test_pooling_at_the_largest_count(gpu, big):
    x, dx, dy = big
    lib = shadow_amd.hip()
    shape = [8, 64, 2048, 2047]
    out = [8, 64, 1024, 1024]
    check(lib.shdw_hip_pooling2d(ints(shape), 0, 3, 3, 2, 2, 1, 1, ints(out), dx.ptr, dy.ptr, None))
    gpuops._sync()
    plane_in, plane_out = shape[2] * shape[3], out[2] * out[3]
    for p0 in (0, 8 * 64 - 2):
        got = dy.download(count=2 * plane_out, offset_bytes=4 * p0 * plane_out)
        xin = x[p0 * plane_in:(p0 + 2) * plane_in]
        want = oracle.pooling(xin, [1, 2] + shape[2:], 0, [3, 3], [2, 2], [1, 1], [1, 2] + out[2:])
        assert np.array_equal(bits(got), bits(np.asarray(want, F).ravel())), "max pooling planes from %d" % p0
    planes = 8 * 64 * 64  # planes of 256 x 255
    shape, out = [planes // 64, 64, 256, 255], [planes // 64, 64, 1, 1]
    check(lib.shdw_hip_pooling2d(ints(shape), 1, 256, 255, 1, 1, 0, 0, ints(out), dx.ptr, dy.ptr, None))
    gpuops._sync()
    got = dy.download(count=planes)
    want = oracle.pooling(x[:planes * 256 * 255], shape, 1, [256, 255], [1, 1], [0, 0], out)
    assert np.array_equal(bits(got), bits(np.asarray(want, F).ravel())), "whole-plane average"


def test_broadcast_and_batch_norm_at_the_largest_count(gpu, big):
    x, dx, dy = big
    lib = shadow_amd.hip()
    shape, n = [8, 64, 2048, 2047], 8 * 64 * 2048 * 2047
    plane = 2048 * 2047
    b = np.linspace(-3.0, 3.0, 64).astype(F)
    db = Buffer.from_numpy(b)
    check(lib.shdw_hip_broadcast_binary(0, 4, ints(shape), ints([1, 64, 1, 1]), ints(shape), dx.ptr, db.ptr, dy.ptr, None))
    gpuops._sync()
    got = dy.download(count=n)
    for lo in range(0, n, PIECE):
        hi = min(n, lo + PIECE)
        c = (np.arange(lo, hi, dtype=np.int64) // plane) % 64
        assert np.array_equal(bits(got[lo:hi]), bits(x[lo:hi] + b[c])), "channel add from %d" % lo
    # BatchNorm over rows of 2047 floats: a vector ends in the next row
    mean, var = np.linspace(-1.0, 1.0, 64).astype(F), np.linspace(0.25, 9.0, 64).astype(F)
    dm, dv = Buffer.from_numpy(mean), Buffer.from_numpy(var)
    rows = n // 2047
    check(lib.shdw_hip_batch_norm(rows * 2047, 64, 2047, dx.ptr, dm.ptr, dv.ptr, 1.0, 1e-5, dy.ptr, None))
    gpuops._sync()
    got = dy.download(count=rows * 2047)
    d = np.sqrt(np.abs(var * F(1.0)) + F(1e-5)).astype(F)
    for lo in range(0, rows * 2047, PIECE):
        hi = min(rows * 2047, lo + PIECE)
        c = (np.arange(lo, hi, dtype=np.int64) // 2047) % 64
        assert np.array_equal(bits(got[lo:hi]), bits((x[lo:hi] - mean[c] * F(1.0)) / d[c])), "batch norm from %d" % lo
    for buf in (db, dm, dv):
        buf.free()


def test_movers_at_the_largest_count(gpu, big):
    x, dx, dy = big
    lib = shadow_amd.hip()
    # interleaved -> planar: the thin transposition
    rows = N // 3
    check(lib.shdw_hip_permute(2, ints([rows, 3]), ints([1, 0]), dx.ptr, dy.ptr, None))
    gpuops._sync()
    got = dy.download(count=3 * rows)
    src = x[:3 * rows].reshape(rows, 3)
    for k in range(3):
        assert np.array_equal(bits(got[k * rows:(k + 1) * rows]), bits(src[:, k])), "planar channel %d" % k
    # a square-ish transposition through the LDS tiles
    r, c = 32768, 65535
    check(lib.shdw_hip_permute(2, ints([r, c]), ints([1, 0]), dx.ptr, dy.ptr, None))
    gpuops._sync()
    got = dy.download(count=r * c).reshape(c, r)
    src = x[:r * c].reshape(r, c)
    for lo in range(0, c, 4096):
        assert np.array_equal(bits(got[lo:lo + 4096]), bits(np.ascontiguousarray(src[:, lo:lo + 4096].T))), \
            "transposed rows from %d" % lo
    # Concat of two inputs along the middle axis: chunks of 1023 rows of 1025 floats into rows of twice that
    chunk = 1023 * 1025
    outer = N // (2 * chunk)
    for k in range(2):
        check(lib.shdw_hip_copy_chunks(outer, chunk, dx.ptr + 4 * k * outer * chunk, chunk, 0, dy.ptr, 2 * chunk,
                                       k * chunk, None))
    gpuops._sync()
    got = dy.download(count=2 * outer * chunk).reshape(outer, 2, chunk)
    for k in range(2):
        src = x[k * outer * chunk:(k + 1) * outer * chunk].reshape(outer, chunk)
        assert np.array_equal(bits(got[:, k, :]), bits(src)), "concat input %d" % k


def test_normalize_and_row_norm_at_the_largest_count(gpu, big):
    x, dx, dy = big
    lib = shadow_amd.hip()
    for dim, inner in ((512, 1), (64, 49)):
        outer = N // (dim * inner)
        check(lib.shdw_hip_normalize(outer, dim, inner, 2.0, 1e-12, dx.ptr, dy.ptr, None))
        gpuops._sync()
        slab = dim * inner
        slabs = max(1, (1 << 22) // slab)
        for s0 in (0, (outer - slabs) // 2, outer - slabs):
            got = dy.download(count=slabs * slab, offset_bytes=4 * s0 * slab)
            want = oracle.normalize(x[s0 * slab:(s0 + slabs) * slab], slabs, dim, inner, 2.0, 1e-12)
            assert np.array_equal(bits(got), bits(np.asarray(want, F).ravel())), "normalize [%d,%d] from %d" % (dim, inner, s0)
    rows, length = N // 784, 784
    check(lib.shdw_hip_group_norm(rows, length, 1e-5, dx.ptr, None, None, 1, 1, dy.ptr, None))
    gpuops._sync()
    count = (1 << 22) // length
    for r0 in (0, rows - count):
        got = dy.download(count=count * length, offset_bytes=4 * r0 * length)
        want = oracle.normalize_rows(x[r0 * length:(r0 + count) * length], count, length, 1e-5)
        assert np.max(np.abs(got - np.asarray(want, F).ravel())) <= 2e-5, "row norm from %d" % r0
