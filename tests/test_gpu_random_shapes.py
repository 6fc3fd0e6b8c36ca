"""Randomly drawn shapes (fixed seeds) through the kernels whose launch shape
depends on row length, alignment or extent, against the oracle: the hand-picked
cases of the other files name the paths, these look for what falls between."""
import numpy as np
import pytest

import oracle
import shadow_amd
from shadow_amd import Buffer, check, ints
from tests import gpuops
from tests.helpers import assert_bit_exact, assert_rel_close

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_reduce_random_shapes(gpu, seed):
    rng = np.random.default_rng(seed)
    for _ in range(40):
        kind = rng.integers(0, 3)
        if kind == 0:    # strided, few to many columns
            shape = [int(rng.integers(1, 40)), int(rng.integers(1, 600)), int(rng.integers(2, 140))]
        elif kind == 1:  # rows, short and long
            shape = [int(rng.integers(200, 3000)), int(rng.integers(1, 140))]
        else:            # channels over small maps
            shape = [int(rng.integers(1, 6)), int(rng.integers(1, 300)), int(rng.integers(1, 12)),
                     int(rng.integers(1, 12))]
        op = int(rng.integers(0, 7))
        x = rng.normal(0, 1, shape).astype(F) if op else rng.uniform(0.9, 1.1, shape).astype(F)
        if rng.random() < 0.3:
            x[rng.random(shape) < 0.3] = 0.0
        if rng.random() < 0.3:
            x[rng.random(shape) < 0.2] = -0.0
        want, _ = oracle.reduce(op, x, shape, [1])
        got, _ = gpuops.reduce(op, x, shape, [1])
        if op in (2, 3):
            assert_bit_exact(got, want, "reduce %d over axis 1 of %s" % (op, shape))
        else:
            assert_rel_close(got, want, 1e-5, "reduce %d over axis 1 of %s" % (op, shape))


# Any ascending axis set of a 2- to 5-d tensor: single-stage views, a reduced dim in front of them
# (either order of the two stages), sliced windows, and what is left to the wave-per-output kernel.
@pytest.mark.parametrize("seed", [22, 23, 24, 25])
def test_reduce_random_axis_sets(gpu, seed):
    rng = np.random.default_rng(seed)
    for _ in range(50):
        nd = int(rng.integers(2, 6))
        shape = [int(rng.choice([1, 2, 3, 5, 7, 8, 16, 33, 40, 64, 100])) for _ in range(nd)]
        if rng.random() < 0.4:  # one long dim: leading-dim-first plans, sliced rows
            shape[int(rng.integers(0, nd))] = int(rng.choice([300, 1000, 5000]))
        while np.prod(shape) > 3_000_000:
            shape[int(np.argmax(shape))] //= 2
        axes = [a for a in range(nd) if rng.random() < 0.5] or [int(rng.integers(0, nd))]
        op = int(rng.integers(0, 7))
        x = rng.normal(0, 1, shape).astype(F) if op else rng.uniform(0.97, 1.03, shape).astype(F)
        if rng.random() < 0.4:
            x[rng.random(shape) < 0.4] = 0.0
            x[rng.random(shape) < 0.3] = -0.0
        want, _ = oracle.reduce(op, x, shape, axes)
        got, _ = gpuops.reduce(op, x, shape, axes)
        what = "reduce %d of %s over %s" % (op, shape, axes)
        if op in (2, 3):
            assert_bit_exact(got, want, what)
        else:
            assert_rel_close(got, want, 1e-5, what)


@pytest.mark.parametrize("seed", [4, 5])
def test_norm_rows_random_shapes(gpu, seed):
    rng = np.random.default_rng(seed)
    for _ in range(40):
        outer, inner = int(rng.integers(1, 600)), int(rng.integers(1, 2300))
        if rng.random() < 0.3:  # many short rows
            outer, inner = int(rng.integers(1024, 5000)), int(rng.integers(1, 140))
        x = (rng.normal(0, 3, outer * inner) + 0.75).astype(F)
        want = oracle.normalize_rows(x, outer, inner, 1e-5)
        got = gpuops.group_norm(x, outer, inner, 1e-5, offset=int(rng.integers(0, 4)))
        assert_rel_close(got, want, 1e-5, "norm rows %d x %d" % (outer, inner))


@pytest.mark.parametrize("seed", [6, 7, 16, 17])
def test_column_ops_random_shapes(gpu, seed):
    rng = np.random.default_rng(seed)
    for _ in range(40):
        outer, dim, inner = int(rng.integers(1, 5)), int(rng.integers(1, 600)), int(rng.integers(1, 200))
        if rng.random() < 0.3:
            inner = 1
        if rng.random() < 0.3:  # long columns: large slabs (inner < 64) and chunked walks (inner >= 16)
            dim, inner = int(rng.integers(513, 5000)), int(rng.integers(1, 80))
        x = rng.normal(0, 4, outer * dim * inner).astype(F)
        what = "[%d, %d, %d]" % (outer, dim, inner)
        assert_bit_exact(gpuops.softmax(x, outer, dim, inner), oracle.softmax(x, outer, dim, inner), "softmax " + what)
        p = float(rng.choice([1.0, 2.0]))
        assert_bit_exact(gpuops.normalize(x, outer, dim, inner, p, 1e-12),
                         oracle.normalize(x, outer, dim, inner, p, 1e-12), "normalize " + what)
        assert_bit_exact(gpuops.ssd_normalize(x, outer, dim, inner, False, True, 1e-10),
                         oracle.ssd_normalize(x, outer, dim, inner, False, True, 1e-10), "ssd normalize " + what)


# The last axis of a thousand rows and more: whole rows per wave in LDS (2 to 64 of them), Normalize over
# rows from 401 on in chunks along 4 to 64 rows per wave; zeros, infinities and NaNs in some rows.
@pytest.mark.parametrize("seed", [26, 27, 28])
def test_last_axis_random_shapes(gpu, seed):
    rng = np.random.default_rng(seed)
    for t in range(14):
        dim = int(np.exp(rng.uniform(np.log(17), np.log(2500))))
        outer = int(rng.integers(1024, max(1025, min(150000, 3_000_000 // dim))))
        x = rng.normal(0, 4, outer * dim).astype(F)
        if t % 3 == 0:
            x[rng.random(x.size) < 0.2] = 0.0
            x[rng.random(x.size) < 0.001] = rng.choice([np.inf, -np.inf, np.nan])
        what = "[%d, %d, 1]" % (outer, dim)
        assert_bit_exact(gpuops.softmax(x, outer, dim, 1), oracle.softmax(x, outer, dim, 1), "softmax " + what)
        p = float(rng.choice([1.0, 2.0, 3.0]))
        assert_bit_exact(gpuops.normalize(x, outer, dim, 1, p, 1e-12), oracle.normalize(x, outer, dim, 1, p, 1e-12),
                         "normalize p=%g %s" % (p, what))
        scale = rng.uniform(0.5, 2.0, dim).astype(F)
        assert_bit_exact(gpuops.ssd_normalize(x, outer, dim, 1, False, False, 1e-10, scale),
                         oracle.ssd_normalize(x, outer, dim, 1, False, False, 1e-10, scale), "ssd normalize " + what)


@pytest.mark.parametrize("seed", [8, 9, 20, 21])
def test_broadcast_random_shapes(gpu, seed):
    rng = np.random.default_rng(seed)
    for _ in range(60):
        nd = int(rng.integers(1, 5)) if rng.random() < 0.6 else int(rng.integers(5, 9))  # up to 8 axes
        out = [int(rng.integers(1, 20 if nd < 5 else 7)) for _ in range(nd)]
        a = [d if rng.random() < 0.7 else 1 for d in out]
        b = [d if rng.random() < 0.5 else 1 for d in out]
        out = [max(p, q) for p, q in zip(a, b)]
        op = int(rng.choice([0, 1, 2, 3, 5, 6]))
        xa, xb = rng.normal(0, 1, a).astype(F), rng.uniform(0.5, 2, b).astype(F)
        assert_bit_exact(gpuops.broadcast_binary(op, xa, a, xb, b, out), oracle.broadcast_binary(op, xa, a, xb, b, out),
                         "broadcast %d %s x %s" % (op, a, b))


@pytest.mark.parametrize("seed", [10, 11])
def test_mover_random_shapes(gpu, seed):
    rng = np.random.default_rng(seed)
    lib = shadow_amd.hip()
    for _ in range(50):
        n, c = int(rng.integers(1, 4)), int(rng.integers(1, 70))
        ih, iw, oh, ow = [int(v) for v in rng.integers(1, 60, 4)]
        typ = int(rng.integers(0, 2))
        align = int(rng.integers(0, 2)) if typ == 1 else 0
        if align and (oh < 2 or ow < 2):
            continue
        x = rng.normal(0, 2, (n, c, ih, iw)).astype(F)
        want = oracle.resize_op(x, [oh, ow], [1.0], typ, bool(align))
        dx, dy = Buffer.from_numpy(x.ravel()), Buffer(4 * want.size)
        check(lib.shdw_hip_resize(ints([n, c, ih, iw]), ints([n, c, oh, ow]), typ, align, dx.ptr, dy.ptr, None))
        gpuops._sync()
        assert_bit_exact(dy.download(count=want.size), want.ravel(),
                         "resize type %d align %d %s -> %s" % (typ, align, x.shape, [oh, ow]))
        dy.free()
        pads = [int(v) for v in rng.integers(0, 4, 4)]
        want = oracle.pad_op(x, pads, 0.5)
        dy = Buffer(4 * want.size)
        check(lib.shdw_hip_pad(ints([n, c, ih, iw]), ints(pads), 0.5, dx.ptr, dy.ptr, None))
        gpuops._sync()
        assert_bit_exact(dy.download(count=want.size), want.ravel(), "pad %s of %s" % (pads, x.shape))
        dy.free()
        group = int(rng.choice([d for d in range(1, c + 1) if c % d == 0]))
        dy = Buffer(4 * x.size)
        check(lib.shdw_hip_shuffle_channel(n, c, ih * iw, group, dx.ptr, dy.ptr, None))
        gpuops._sync()
        assert_bit_exact(dy.download(count=x.size), oracle.shuffle_channel_op(x, group).ravel(),
                         "shuffle %d groups of %s" % (group, x.shape))
        dx.free()
        dy.free()


# Concat / Slice / Stack all go through one strided chunk copy: chunks, pitches and offsets that are and are
# not whole vectors, chunks of one to three floats, pointers off the vector boundary.
@pytest.mark.parametrize("seed", [29, 30])
def test_copy_chunks_random(gpu, seed):
    rng = np.random.default_rng(seed)
    lib = shadow_amd.hip()
    for _ in range(80):
        outer = int(rng.integers(1, 60))
        chunk = int(np.exp(rng.uniform(0, np.log(3000))))
        if rng.random() < 0.3:
            chunk = 4 * max(1, chunk // 4)
        src_off, dst_off = int(rng.integers(0, 9)), int(rng.integers(0, 9))
        src_pitch = src_off + chunk + int(rng.integers(0, 9))
        dst_pitch = dst_off + chunk + int(rng.integers(0, 9))
        if rng.random() < 0.3:
            src_off, dst_off, src_pitch, dst_pitch = [4 * (v // 4 + (k >= 2)) + (chunk if k >= 2 else 0)
                                                      for k, v in enumerate((src_off, dst_off, src_pitch - chunk,
                                                                             dst_pitch - chunk))]
            src_pitch, dst_pitch = max(src_pitch, src_off + chunk), max(dst_pitch, dst_off + chunk)
        shift = int(rng.integers(0, 4)) if rng.random() < 0.3 else 0
        src = rng.normal(0, 1, outer * src_pitch + shift).astype(F)
        dst = rng.normal(0, 1, outer * dst_pitch + shift).astype(F)
        want = dst.copy()
        for n in range(outer):
            want[shift + n * dst_pitch + dst_off: shift + n * dst_pitch + dst_off + chunk] = \
                src[shift + n * src_pitch + src_off: shift + n * src_pitch + src_off + chunk]
        ds, dd = Buffer.from_numpy(src), Buffer.from_numpy(dst)
        check(lib.shdw_hip_copy_chunks(outer, chunk, ds.ptr + 4 * shift, src_pitch, src_off, dd.ptr + 4 * shift,
                                       dst_pitch, dst_off, None))
        gpuops._sync()
        assert_bit_exact(dd.download(count=dst.size), want, "chunks of %d, pitches %d -> %d, offsets %d -> %d, shift %d"
                         % (chunk, src_pitch, dst_pitch, src_off, dst_off, shift))
        ds.free()
        dd.free()


@pytest.fixture()
def ws(gpu):
    w = shadow_amd.Workspace("Native", 0)
    yield w
    w.close()


def _run(ws, op_type, x, args, top):
    ws.set_blob("x", x)
    op = ws.create_op(op_type, ["x"], [top], args)
    op.run()
    return ws.get_blob(top)


@pytest.mark.parametrize("seed", [12, 13, 18, 19])
def test_pooling_random_shapes(ws, seed):
    rng = np.random.default_rng(seed)
    for t in range(60):
        n, c = int(rng.integers(1, 4)), int(rng.integers(1, 40))
        h, w = int(rng.integers(1, 70)), int(rng.integers(1, 70))
        kmax = 13 if t % 3 == 0 else 7
        kh, kw = int(rng.integers(1, min(h, kmax) + 1)), int(rng.integers(1, min(w, kmax) + 1))
        sh, sw = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        ph, pw = int(rng.integers(0, kh)), int(rng.integers(0, kw))
        pool, full = int(rng.integers(0, 2)), bool(rng.integers(0, 2))
        x = rng.normal(0, 2, (n, c, h, w)).astype(F)
        if t % 4 == 0:  # ties between +0 and -0, cells the maximum never takes
            x[rng.random(x.shape) < 0.5] = 0.0
            x[rng.random(x.shape) < 0.3] = -0.0
            x[rng.random(x.shape) < 0.05] = -np.inf
        args = {"pool": pool, "kernel_size": [kh, kw], "stride": [sh, sw], "pad": [ph, pw], "full_pooling": full}
        try:
            want = oracle.pooling_op(x, pool, [kh, kw], [sh, sw], [ph, pw], full_pooling=full)
        except oracle.OracleCheckError:
            continue
        got = _run(ws, "Pooling", x, args, "pool%d" % t)
        assert got.shape == want.shape
        assert_bit_exact(got, want, "pooling %s %s" % (x.shape, args))


@pytest.mark.parametrize("seed", [14, 15])
def test_permute_reorg_gather_random_shapes(ws, seed):
    rng = np.random.default_rng(seed)
    for t in range(50):
        nd = int(rng.integers(2, 6))
        shape = [int(rng.integers(1, 12)) for _ in range(nd)]
        order = [int(v) for v in rng.permutation(nd)]
        x = rng.normal(0, 1, shape).astype(F)
        assert_bit_exact(_run(ws, "Permute", x, {"order": order}, "perm%d" % t), oracle.permute_op(x, order),
                         "permute %s by %s" % (shape, order))
        s = int(rng.integers(1, 4))
        shape = (int(rng.integers(1, 3)), s * s * int(rng.integers(1, 6)), s * int(rng.integers(1, 12)),
                 s * int(rng.integers(1, 12)))
        typ = int(rng.integers(0, 2))
        x = rng.normal(0, 1, shape).astype(F)
        assert_bit_exact(_run(ws, "Reorg", x, {"type": typ, "stride": s}, "reorg%d" % t), oracle.reorg_op(x, typ, s),
                         "reorg type %d stride %d of %s" % (typ, s, shape))
        axis = int(rng.integers(0, 4))
        idx = [int(v) for v in rng.integers(0, shape[axis], int(rng.integers(1, 6)))]
        assert_bit_exact(_run(ws, "Gather", x, {"axis": axis, "indexes": idx}, "gather%d" % t),
                         oracle.gather_op(x, axis, idx), "gather %s on axis %d of %s" % (idx, axis, shape))
