"""GPU parity for Axpy, BatchNorm, Softmax, Normalize and Pooling: the C ABI entry
points and the operators through Operator::Run(), bit for bit against the oracle
(these kernels fold every column / window in the reference's order, so there is
no tolerance anywhere in this file)."""
import ctypes

import numpy as np
import pytest

import oracle
import shadow_amd
from shadow_amd import ShadowError
from tests import gpuops
from tests.helpers import assert_bit_exact, assert_rel_close, normal, uniform, with_specials

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture()
def ws(gpu):
    w = shadow_amd.Workspace("Native", 0)
    yield w
    w.close()


def run(ws, op_type, inputs, args, top="out"):
    names = []
    for name, arr in inputs:
        ws.set_blob(name, arr)
        names.append(name)
    op = ws.create_op(op_type, names, [top], args)
    op.run()
    return ws.get_blob(top)


# ------------------------------------------------------------------- axpy ---
@pytest.mark.parametrize("outer,inner", [(1, 1), (6, 49), (48, 64), (10, 3136), (7, 5), (300, 3), (33, 1001)])
def test_axpy_rows(gpu, outer, inner):
    alpha = with_specials(normal(1, outer), 1)
    x, y = normal(2, outer * inner, 3.0), normal(3, outer * inner)
    want = oracle.axpy_rows(alpha, x, y, inner)
    assert_bit_exact(gpuops.axpy_rows(alpha, x, y, inner), want, "axpy_rows")
    assert_bit_exact(gpuops.axpy_rows(alpha, x, y, inner, inplace=True), want, "axpy_rows in place")


def test_axpy_op(ws):
    alpha, x, y = normal(4, (4, 16)), normal(5, (4, 16, 7, 7)), normal(6, (4, 16, 7, 7))
    got = run(ws, "Axpy", [("alpha", alpha), ("x", x), ("y", y)], {})
    assert got.shape == x.shape
    assert_bit_exact(got, oracle.axpy_op(alpha, x, y), "axpy op")
    got = run(ws, "Axpy", [("alpha", alpha.reshape(4, 16, 1, 1)), ("x", x), ("y", y)], {})
    assert_bit_exact(got, oracle.axpy_op(alpha, x, y), "axpy op, 4-d alpha")
    ws.set_blob("bad", np.zeros((4, 15), F))
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("Axpy", ["bad", "x", "y"], ["o2"], {}).run()
    with pytest.raises(ShadowError, match="three inputs"):
        ws.create_op("Axpy", ["x", "y"], ["o3"], {}).run()


# ------------------------------------------------------------- batch norm ---
# Rows (inner extents) of 1, 2 and 3: up to four rows per 128-bit vector; of 5, 6, 7, 49, 99: a vector ends
# in the next row; a last vector that ends with the tensor.
@pytest.mark.parametrize("shape", [(2, 3, 4, 4), (4, 64, 7, 7), (3, 5, 9, 11), (2, 7, 1, 1), (1, 130, 28, 28),
                                   (5, 9, 1, 2), (3, 7, 1, 3), (4, 6, 5, 1), (3, 11, 2, 3), (2, 5, 1, 7), (7, 3, 1, 1),
                                   (9, 1, 1, 1), (2, 2, 9, 11), (3, 1001, 1, 1), (2, 1000, 1, 3)])
@pytest.mark.parametrize("sf", [1.0, 0.0010000181])
def test_batch_norm(gpu, shape, sf):
    x = with_specials(normal(7, shape, 3.0), 7)
    c, inner = shape[1], int(np.prod(shape[2:]))
    mean, var = normal(8, c), uniform(9, c, -0.5, 900.0)
    want = oracle.batch_norm(x, mean, var, c, inner, sf, 1e-5)
    assert_bit_exact(gpuops.batch_norm(x, mean, var, c, inner, sf, 1e-5), want, "batch_norm")
    assert_bit_exact(gpuops.batch_norm(x, mean, var, c, inner, sf, 1e-5, inplace=True), want, "in place")


@pytest.mark.parametrize("shape", [(2, 3, 4, 4), (4, 64, 7, 7), (3, 5, 9, 11), (2, 7, 1, 1), (1, 130, 28, 28),
                                   (5, 9, 1, 2), (3, 7, 1, 3), (2, 5, 1, 7), (3, 1001, 1, 1)])
@pytest.mark.parametrize("form", ["scale", "bias", "both"])
@pytest.mark.parametrize("relu", [False, True])
def test_batch_norm_scale_in_one_launch(gpu, shape, form, relu):
    """BatchNorm -> Scale [-> ReLU] fused equals the oracle's operators one after the other, bit for bit."""
    x = with_specials(normal(13, shape, 3.0), 13)
    c, inner = shape[1], int(np.prod(shape[2:]))
    mean, var = normal(14, c), uniform(15, c, -0.5, 900.0)
    scale = uniform(16, c, 0.5, 1.5) if form != "bias" else None
    bias = uniform(17, c, -0.3, 0.3) if form != "scale" else None
    for sf in (1.0, 0.0010000181):
        want = oracle.batch_norm(x, mean, var, c, inner, sf, 1e-5)
        want = oracle.scale_bias(want, scale, bias, c, inner)
        if relu:
            want = oracle.activate(want, 1)
        got = gpuops.batch_norm_scale(x, mean, var, c, inner, sf, 1e-5, scale, bias, relu)
        assert_bit_exact(got, want, "batch_norm + scale")
        got = gpuops.batch_norm_scale(x, mean, var, c, inner, sf, 1e-5, scale, bias, relu, inplace=True)
        assert_bit_exact(got, want, "in place")


def test_batch_norm_op(ws):
    x = normal(10, (3, 12, 6, 5), 2.0)
    mean, var = normal(11, 12), uniform(12, 12, 0.1, 5.0)
    got = run(ws, "BatchNorm", [("x", x), ("mean", mean), ("var", var)], {})
    assert_bit_exact(got, oracle.batch_norm_op(x, mean, var), "bn op")
    for scale in (999.982, 0.0):
        got = run(ws, "BatchNorm", [("x", x), ("mean", mean), ("var", var), ("s", F([scale]))], {"eps": 1e-3})
        assert_bit_exact(got, oracle.batch_norm_op(x, mean, var, F([scale]), eps=1e-3), "bn op scaled")
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("BatchNorm", ["x", "mean", "var"], ["o2"], {"use_global_stats": False})
    ws.set_blob("short", np.zeros(11, F))
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("BatchNorm", ["x", "short", "var"], ["o3"], {}).run()
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("BatchNorm", ["x", "mean"], ["o4"], {}).run()


# -------------------------------------------------------------------- lrn ---
@pytest.mark.parametrize("shape,size", [((2, 96, 55, 55), 5), ((1, 256, 27, 27), 5), ((2, 7, 3, 5), 5), ((1, 2, 4, 4), 5),
                                        ((3, 16, 1, 1), 3), ((2, 6, 2, 3), 1), ((2, 5, 2, 2), 9), ((1, 40, 3, 3), 11),
                                        ((3, 1, 17, 19), 3), ((1, 70, 5, 52), 63), ((300, 4, 1, 1), 3)])
@pytest.mark.parametrize("alpha,beta,k", [(1e-4, 0.75, 1.0), (0.5, 2.0, 2.0)])
def test_lrn(gpu, shape, size, alpha, beta, k):
    """The running sum over the channels, its scale and the power, against the oracle's two passes."""
    x = with_specials(normal(31, shape, 3.0), 31)
    want, _ = oracle.lrn(x, shape, size, alpha, beta, k)
    assert_bit_exact(gpuops.lrn(x, shape, size, alpha, beta, k), want, "lrn")
    assert_bit_exact(gpuops.lrn(x, shape, size, alpha, beta, k, inplace=True), want, "in place")


def test_lrn_scales_below_one_and_negative(gpu):
    """k = 0 and a negative alpha: powf meets zeros, tiny and negative bases."""
    shape = (2, 12, 5, 7)
    x = normal(32, shape, 1e-3)
    x[0, :, 0, 0] = 0
    for alpha, k in ((1.0, 0.0), (-2.0, 1e-6), (1e30, 1.0)):
        want, _ = oracle.lrn(x, shape, 5, alpha, 0.75, k)
        assert_bit_exact(gpuops.lrn(x, shape, 5, alpha, 0.75, k), want, "lrn alpha %g k %g" % (alpha, k))


def test_lrn_argument_errors(gpu):
    lib = gpu
    buf = shadow_amd.Buffer(4 * 2 * 3 * 4 * 4)
    ints = shadow_amd.ints
    sh = ints([2, 3, 4, 4])
    assert lib.shdw_hip_lrn(sh, 4, 1.0, 0.75, 1.0, buf.ptr, buf.ptr, None) == -1   # even window
    assert lib.shdw_hip_lrn(sh, 0, 1.0, 0.75, 1.0, buf.ptr, buf.ptr, None) == -1
    assert lib.shdw_hip_lrn(sh, 9, 1.0, 0.75, 1.0, buf.ptr, buf.ptr, None) == -1   # four channels behind the centre, three there
    assert lib.shdw_hip_lrn(sh, 5, 1.0, 0.75, 1.0, None, buf.ptr, None) == -1
    assert lib.shdw_hip_lrn(ints([2, 80, 1, 1]), 65, 1.0, 0.75, 1.0, buf.ptr, buf.ptr, None) == -2  # window over 63
    assert lib.shdw_hip_lrn(ints([2, 0, 4, 4]), 1, 1.0, 0.75, 1.0, None, None, None) == 0    # empty


def test_lrn_op(ws):
    x = normal(33, (2, 10, 6, 5), 2.0)
    got = run(ws, "LRN", [("x", x)], {"local_size": 3, "alpha": 0.001, "beta": 0.75, "k": 2.0})
    assert_bit_exact(got, oracle.lrn_op(x, 3, 0.001, 0.75, 0, 2.0), "lrn op")
    got = run(ws, "LRN", [("x", x)], {})
    assert_bit_exact(got, oracle.lrn_op(x), "lrn op, default arguments")
    with pytest.raises(ShadowError, match="odd values"):
        ws.create_op("LRN", ["x"], ["o2"], {"local_size": 4})
    with pytest.raises(ShadowError, match="Across Channels"):
        ws.create_op("LRN", ["x"], ["o3"], {"norm_region": 1})
    ws.set_blob("flat", np.zeros((4, 6), F))
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("LRN", ["flat"], ["o4"], {}).run()
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("LRN", ["x"], ["o5"], {"local_size": 23}).run()


# ------------------------------------------------------------ grid sample ---
@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("padding_mode", [0, 1])
@pytest.mark.parametrize("shape,out_hw", [((2, 3, 5, 7), (4, 6)), ((1, 13, 1, 9), (3, 3)), ((3, 1, 8, 1), (2, 5)),
                                          ((2, 20, 6, 6), (11, 13)), ((2, 64, 56, 56), (56, 56)), ((1, 8, 31, 17), (64, 70)),
                                          ((300, 2, 3, 3), (1, 1))])
def test_grid_sample(gpu, mode, padding_mode, shape, out_hw):
    x = with_specials(normal(41, shape, 2.0), 41)
    grid = uniform(42, (shape[0],) + out_hw + (2,), -1.3, 1.3)  # a fifth of the coordinates outside the input
    out_shape = list(shape[:2]) + list(out_hw)
    want = oracle.grid_sample(x, shape, grid, mode, padding_mode, out_shape)
    assert_bit_exact(gpuops.grid_sample(x, shape, grid, mode, padding_mode, out_shape), want, "grid sample")


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("padding_mode", [0, 1])
def test_grid_sample_on_cell_centres_ties_and_coordinates_that_fit_no_int(gpu, mode, padding_mode):
    shape, out_hw = (2, 5, 9, 5), (9, 8)
    x = normal(43, shape)
    gy, gx = np.meshgrid(np.linspace(-1, 1, 9), np.linspace(-1, 1, 8), indexing="ij")  # rows: exact centres; columns: ties and thirds
    grid = np.broadcast_to(np.stack([gx, gy], -1).astype(F), (2,) + out_hw + (2,)).copy()
    grid[1, 0, :, 0] = [1e30, -1e30, np.inf, -np.inf, 3e9, -3e9, 2.0 ** 31, -1.0000001]
    grid[1, 1, :, 1] = [1e30, -1e30, np.inf, -np.inf, 3e9, -3e9, 2.0 ** 31, 1.0000001]
    if mode == 0:  # a NaN coordinate has a defined answer in the nearest mode only (the conversion's)
        grid[1, 2, :4, 0] = np.nan
        grid[1, 3, 4:, 1] = np.nan
    out_shape = list(shape[:2]) + list(out_hw)
    want = oracle.grid_sample(x, shape, grid, mode, padding_mode, out_shape)
    assert_bit_exact(gpuops.grid_sample(x, shape, grid, mode, padding_mode, out_shape), want, "grid sample")


def test_grid_sample_bilinear_gives_nan_for_a_nan_coordinate(gpu):
    shape, out_hw = (1, 3, 4, 4), (2, 2)
    x = normal(44, shape)
    grid = np.zeros((1, 2, 2, 2), F)
    grid[0, 0, 0, 0] = np.nan
    grid[0, 1, 1, 1] = np.nan
    for padding_mode in (0, 1):
        got = gpuops.grid_sample(x, shape, grid, 1, padding_mode, [1, 3, 2, 2]).reshape(1, 3, 2, 2)
        assert np.isnan(got[:, :, 0, 0]).all() and np.isnan(got[:, :, 1, 1]).all()
        assert_bit_exact(got, oracle.grid_sample(x, shape, grid, 1, padding_mode, [1, 3, 2, 2]), "the oracle's rule")


def test_grid_sample_argument_errors(gpu):
    lib, ints = gpu, shadow_amd.ints
    buf = shadow_amd.Buffer(4 * 64)
    a, o = ints([1, 2, 2, 2]), ints([1, 2, 2, 2])
    assert lib.shdw_hip_grid_sample(a, o, 2, 0, buf.ptr, buf.ptr, buf.ptr, None) == -1
    assert lib.shdw_hip_grid_sample(a, o, 1, 2, buf.ptr, buf.ptr, buf.ptr, None) == -1
    assert lib.shdw_hip_grid_sample(a, ints([1, 3, 2, 2]), 1, 0, buf.ptr, buf.ptr, buf.ptr, None) == -1   # channels differ
    assert lib.shdw_hip_grid_sample(a, ints([2, 2, 2, 2]), 1, 0, buf.ptr, buf.ptr, buf.ptr, None) == -1   # batches differ
    assert lib.shdw_hip_grid_sample(a, o, 1, 0, buf.ptr, buf.ptr, buf.ptr, None) == -1                    # output is the input
    assert lib.shdw_hip_grid_sample(a, o, 1, 0, None, buf.ptr, buf.ptr, None) == -1
    assert lib.shdw_hip_grid_sample(ints([1, 2, 0, 2]), o, 1, 0, buf.ptr, buf.ptr, buf.ptr, None) == -1   # nothing to sample
    assert lib.shdw_hip_grid_sample(a, ints([1, 2, 0, 2]), 1, 0, None, None, None, None) == 0             # nothing to fill


def test_grid_sample_op(ws):
    x, grid = normal(45, (2, 6, 7, 5), 2.0), uniform(46, (2, 4, 9, 2), -1.2, 1.2)
    for mode in (0, 1):
        for padding_mode in (0, 1):
            got = run(ws, "GridSample", [("x", x), ("grid", grid)], {"mode": mode, "padding_mode": padding_mode})
            assert got.shape == (2, 6, 4, 9)
            assert_bit_exact(got, oracle.grid_sample_op(x, grid, mode, padding_mode), "grid sample op")
    got = run(ws, "GridSample", [("x", x), ("grid", grid)], {})
    assert_bit_exact(got, oracle.grid_sample_op(x, grid), "bilinear with zeros outside by default")
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("GridSample", ["x", "grid"], ["o2"], {"mode": 2})
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("GridSample", ["x", "grid"], ["o3"], {"padding_mode": 2})
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("GridSample", ["x"], ["o4"], {}).run()
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("GridSample", ["x", "grid"], ["x"], {}).run()
    ws.set_blob("three", np.zeros((2, 4, 9, 3), F))
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("GridSample", ["x", "three"], ["o5"], {}).run()
    ws.set_blob("other", np.zeros((3, 4, 9, 2), F))
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("GridSample", ["x", "other"], ["o6"], {}).run()


# ---------------------------------------------------------------- softmax ---
SOFTMAX_SHAPES = [  # outer, dim, inner: both layouts, LDS limits, odd sizes
    (1, 1, 1), (64, 1000, 1), (3, 10, 1), (5, 7, 3), (2, 21, 63), (2, 21, 64), (2, 21, 65),
    (4, 8, 1024), (1, 15000, 1), (1, 16000, 1), (2, 300, 50), (2, 310, 50), (300, 4, 2),
    (1, 2, 5000), (3, 1, 17),
    # columns too long for registers over a wide inner extent: the three-walk kernel
    (2, 150, 300), (1, 65, 4097), (3, 100, 64), (1, 1000, 70),
    # around the longest column whose tile fits LDS beside the exp table
    (1, 509, 40), (1, 510, 40), (1, 511, 20), (1, 512, 33),
    # slabs of more than 60 KB
    (3, 4096, 7), (2, 20000, 1), (2, 1300, 15), (1, 39000, 1), (1, 39936, 1), (1, 40000, 1),
    # tall columns: chunks of rows through LDS, tiles of 16 / 32 / 64 positions, vectors or not,
    # a cut last tile, a last chunk of one row, many workgroups
    (2, 1300, 30), (2, 600, 64), (1, 1000, 100), (3, 513, 17), (1, 2048, 196), (2, 700, 68), (1, 4097, 16),
    (1, 1025, 3136), (40, 520, 128), (1100, 513, 16), (2, 769, 49), (1, 20000, 20),
    # a thousand and more rows over the last axis: every wave on its own rows (1 to 32 rows per wave, both
    # tile sizes, a ragged last wave and workgroup)
    (1100, 17, 1), (2000, 49, 1), (1025, 1000, 1), (1024, 1023, 1), (1030, 1024, 1), (1100, 2049, 1), (1024, 4096, 1),
    (1500, 64, 1), (3001, 21, 1), (1027, 333, 1), (5000, 150, 1),
    # long slabs over fewer than 16 positions, in chunks of whole rows: ragged last chunks, one to fifteen positions
    (2, 5000, 3), (1, 16000, 1), (1, 1100, 14), (3, 2731, 6), (2, 8193, 2), (1, 3000, 15), (5, 1537, 10),
]


@pytest.mark.parametrize("outer,dim,inner", SOFTMAX_SHAPES)
def test_softmax(gpu, outer, dim, inner):
    x = normal(13, outer * dim * inner, 5.0)
    want = oracle.softmax(x, outer, dim, inner)
    assert_bit_exact(gpuops.softmax(x, outer, dim, inner), want, "softmax")
    assert_bit_exact(gpuops.softmax(x, outer, dim, inner, inplace=True), want, "softmax in place")


# Slabs of more than 60 KB over 16 to 256 positions with a few hundred slabs to hand out, a workgroup per slab
# in chunks of whole rows where the columns are too short or too long for the tile kernels (under 65 or over
# 512 rows): positions that are and are not multiples of 16 (Softmax takes only the latter), one row per
# chunk, the slab counts either side of where the form starts; the same shapes inside the tile kernels' range.
@pytest.mark.parametrize("outer,dim,inner", [(192, 700, 25), (200, 350, 49), (193, 160, 100), (192, 65, 255),
                                             (384, 61, 256), (400, 130, 128), (191, 700, 25), (383, 130, 128),
                                             (200, 1000, 17), (385, 500, 32), (192, 61, 257), (192, 600, 100),
                                             (384, 520, 64), (193, 513, 255),
                                             # columns of 513 to 1024 rows in tiles of 16 positions: rows on 64-byte
                                             # boundaries, on multiples of four, ending inside a lane's four; the
                                             # position counts either side of where Softmax and Normalize take them
                                             (2, 1024, 64), (3, 513, 196), (2, 1000, 67), (1, 700, 130), (5, 1023, 33),
                                             (2, 600, 49), (3, 1024, 31), (2, 800, 63)])
def test_column_ops_over_long_slabs_of_many_positions(gpu, outer, dim, inner):
    x = normal(45, outer * dim * inner, 4.0)
    assert_bit_exact(gpuops.softmax(x, outer, dim, inner), oracle.softmax(x, outer, dim, inner), "softmax")
    for p in (1.0, 2.0, 2.5):
        assert_bit_exact(gpuops.normalize(x, outer, dim, inner, p, 1e-12), oracle.normalize(x, outer, dim, inner, p, 1e-12),
                         "normalize p=%g" % p)
    assert_bit_exact(gpuops.normalize(x, outer, dim, inner, 2.0, 1e-12, inplace=True, offset=1),
                     oracle.normalize(x, outer, dim, inner, 2.0, 1e-12), "normalize in place, off the vector boundary")
    scale = uniform(46, dim, 0.5, 2.0)
    assert_bit_exact(gpuops.ssd_normalize(x, outer, dim, inner, False, False, 1e-5, scale),
                     oracle.ssd_normalize(x, outer, dim, inner, False, False, 1e-5, scale), "ssd normalize")
    z = with_specials(x.copy(), 47)
    assert_bit_exact(gpuops.softmax(z, outer, dim, inner), oracle.softmax(z, outer, dim, inner), "softmax specials")


# Long rows over the last axis: Normalize moves along 4, 8, 16, 32 or 64 rows per wave by the number and the
# length of the rows (whole and cut chunks, a cut last vector, a last wave with rows missing); Softmax has
# the rows in LDS up to 1023 elements and a workgroup per row beyond.
@pytest.mark.parametrize("outer,dim", [(1500, 401), (1024, 4097), (1100, 8191), (40003, 402), (70001, 401),
                                       (131077, 403), (2049, 513), (1030, 20000), (9001, 500), (17001, 405),
                                       (1201, 1023), (1201, 1024), (8563, 1500)])
def test_softmax_and_normalize_over_long_rows(gpu, outer, dim):
    x = normal(33, outer * dim, 4.0)
    assert_bit_exact(gpuops.softmax(x, outer, dim, 1), oracle.softmax(x, outer, dim, 1), "softmax")
    assert_bit_exact(gpuops.normalize(x, outer, dim, 1, 2.0, 1e-12), oracle.normalize(x, outer, dim, 1, 2.0, 1e-12),
                     "normalize")
    if outer < 3000:
        assert_bit_exact(gpuops.softmax(x, outer, dim, 1, inplace=True, offset=1), oracle.softmax(x, outer, dim, 1),
                         "softmax in place, off the vector boundary")
        scale = uniform(34, dim, 0.5, 2.0)
        assert_bit_exact(gpuops.ssd_normalize(x, outer, dim, 1, False, False, 1e-5, scale),
                         oracle.ssd_normalize(x, outer, dim, 1, False, False, 1e-5, scale), "ssd normalize")


# Rows of 2 to 16 elements over the last axis, four rows per lane: row counts that end inside a lane's four
# rows, inside a vector and inside a wave's span; off the vector boundary in place; infinities and NaNs.
@pytest.mark.parametrize("dim", list(range(2, 17)))
def test_softmax_over_short_rows(gpu, dim):
    for outer in (1024, 1027, 4099, 70001):
        x = normal(40 + dim, outer * dim, 4.0)
        want = oracle.softmax(x, outer, dim, 1)
        assert_bit_exact(gpuops.softmax(x, outer, dim, 1), want, "softmax [%d,%d,1]" % (outer, dim))
        assert_bit_exact(gpuops.softmax(x, outer, dim, 1, inplace=True, offset=1 + outer % 3), want,
                         "softmax [%d,%d,1] in place, off the vector boundary" % (outer, dim))
    x = with_specials(normal(41, 5003 * dim, 30.0), 41)
    assert_bit_exact(gpuops.softmax(x, 5003, dim, 1), oracle.softmax(x, 5003, dim, 1), "softmax specials")


# Two to four rows over 16 and more positions: four positions per lane with their columns in registers; rows that
# are and are not whole vectors long (the last quad of a slab cut), Normalize / SSDNormalize over two rows.
@pytest.mark.parametrize("outer,dim,inner", [(5, 2, 16), (3, 3, 17), (2, 4, 64), (7, 2, 49), (1, 3, 1001), (300, 2, 20),
                                             (2, 4, 18), (9, 1, 33), (4, 2, 3136)])
def test_column_ops_over_two_to_four_rows(gpu, outer, dim, inner):
    x = with_specials(normal(48, outer * dim * inner, 6.0), 48)
    want = oracle.softmax(x, outer, dim, inner)
    assert_bit_exact(gpuops.softmax(x, outer, dim, inner), want, "softmax")
    assert_bit_exact(gpuops.softmax(x, outer, dim, inner, inplace=True, offset=1), want, "softmax in place, off the vector boundary")
    x = normal(49, outer * dim * inner, 3.0)
    for p in (1.0, 2.0):
        want = oracle.normalize(x, outer, dim, inner, p, 1e-12)
        assert_bit_exact(gpuops.normalize(x, outer, dim, inner, p, 1e-12), want, "normalize p=%g" % p)
        assert_bit_exact(gpuops.normalize(x, outer, dim, inner, p, 1e-12, inplace=True, offset=3), want, "normalize in place")
    for shared in (True, False):
        scale = uniform(50, 1 if shared else dim, 0.5, 2.0)
        assert_bit_exact(gpuops.ssd_normalize(x, outer, dim, inner, False, shared, 1e-6, scale),
                         oracle.ssd_normalize(x, outer, dim, inner, False, shared, 1e-6, scale), "ssd normalize")


# Slabs of dim * inner <= 9 floats with inner > 1 go the same way, four slabs per lane; the next larger ones.
@pytest.mark.parametrize("outer,dim,inner", [(5003, 2, 2), (4099, 2, 4), (1027, 3, 3), (70001, 4, 2), (1500, 3, 2),
                                             (1029, 2, 3), (2001, 5, 2), (1025, 3, 4), (1024, 2, 7), (33333, 7, 2)])
def test_softmax_over_short_slabs(gpu, outer, dim, inner):
    x = normal(43, outer * dim * inner, 4.0)
    want = oracle.softmax(x, outer, dim, inner)
    assert_bit_exact(gpuops.softmax(x, outer, dim, inner), want, "softmax")
    assert_bit_exact(gpuops.softmax(x, outer, dim, inner, inplace=True, offset=3), want, "softmax in place, off the vector boundary")
    x = with_specials(normal(44, outer * dim * inner, 30.0), 44)
    assert_bit_exact(gpuops.softmax(x, outer, dim, inner), oracle.softmax(x, outer, dim, inner), "softmax specials")


@pytest.mark.parametrize("outer,dim,inner", [(40, 50, 1), (2, 12, 200), (2, 80, 100), (2, 6000, 3), (1, 700, 64),
                                             (1200, 100, 1), (1030, 1500, 1)])
def test_softmax_special_values(gpu, outer, dim, inner):
    x = with_specials(normal(14, outer * dim * inner, 30.0), 14)
    assert_bit_exact(gpuops.softmax(x, outer, dim, inner), oracle.softmax(x, outer, dim, inner), "softmax specials")


# A NaN takes the running maximum over and the next element takes it back, so with
# NaNs in a column the order of the walk shows in the result (first, middle and last
# row, several in one column); the tile kernel takes the maxima in parallel only where
# the tile holds none.  Both tile widths, ragged rows, tiles with and without NaNs.
@pytest.mark.parametrize("outer,dim,inner", [(2, 80, 100), (1, 150, 333), (2, 300, 70), (1, 512, 41), (3, 66, 16),
                                             (2, 600, 41), (1, 1030, 64)])
def test_softmax_with_nans_in_the_columns(gpu, outer, dim, inner):
    x = normal(23, (outer, dim, inner), 4.0)
    x[0, 0, 1] = np.nan
    x[0, dim - 1, 5] = np.nan
    x[0, dim // 2, 9] = np.nan
    x[0, 3, 13] = x[0, dim - 2, 13] = x[0, 40, 13] = np.nan
    x[outer - 1, 17, inner - 1] = np.nan
    x[0, :, 15] = np.nan
    x = x.reshape(-1)
    assert_bit_exact(gpuops.softmax(x, outer, dim, inner), oracle.softmax(x, outer, dim, inner), "softmax with NaNs")


# Spreads wide enough for exp to reach tiny, denormal and zero results, next to
# ordinary columns, in each kernel layout.
@pytest.mark.parametrize("outer,dim,inner", [(3, 40, 1), (2, 12, 200), (2, 48, 130), (2, 150, 300), (1, 100, 70),
                                             (1, 1000, 70), (2, 300, 50), (2, 21, 63)])
def test_softmax_with_underflowing_exponentials(gpu, outer, dim, inner):
    x = normal(19, (outer, dim, inner), 3.0)
    x[:, :, ::3] *= F(12.0)      # gaps up to ~100: exp down to 1e-44 and 0
    x[:, 1::2, 1::5] -= F(95.0)  # every other class far below the rest
    x = x.reshape(-1)
    assert_bit_exact(gpuops.softmax(x, outer, dim, inner), oracle.softmax(x, outer, dim, inner), "softmax tails")


@pytest.mark.parametrize("shape,axis", [((8, 1000), 1), ((2, 21, 33, 35), 1), ((3, 4, 5), -1), ((6, 2, 3), 0)])
def test_softmax_op(ws, shape, axis):
    x = normal(15, shape, 3.0)
    got = run(ws, "Softmax", [("x", x)], {"axis": axis})
    assert got.shape == x.shape
    assert_bit_exact(got, oracle.softmax_op(x, axis), "softmax op")


def test_softmax_op_defaults_and_errors(ws):
    x = normal(16, (2, 5, 3))
    assert_bit_exact(run(ws, "Softmax", [("x", x)], {}), oracle.softmax_op(x, 1), "default axis")
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("Softmax", ["x"], ["o2"], {"axis": 3}).run()


# -------------------------------------------------------------- normalize ---
@pytest.mark.parametrize("p", [1.0, 2.0, 3.0, 0.5])
@pytest.mark.parametrize("outer,dim,inner", [(64, 512, 1), (5, 7, 3), (2, 16, 100), (3, 9, 64), (1, 20000, 1),
                                             (2, 1, 9), (1, 33, 4097),
                                             # 65..1024 deep over a wide inner extent: tiles of 64 and 32 positions
                                             (2, 100, 100), (1, 512, 72), (3, 300, 37), (2, 1024, 20), (1, 65, 4097),
                                             (2, 256, 64), (1, 1025, 40),
                                             # tall columns in chunks through LDS; slabs of more than 60 KB
                                             (2, 1300, 30), (1, 2048, 196), (2, 1100, 68), (1, 4097, 16),
                                             (30, 1026, 128), (3, 4096, 7), (1, 39000, 1),
                                             (2, 5000, 3), (1, 1100, 14), (3, 2731, 6), (2, 8193, 2),
                                             (1100, 17, 1), (1025, 1000, 1), (1030, 1024, 1), (1024, 4096, 1), (3001, 21, 1)])
def test_normalize(gpu, p, outer, dim, inner):
    x = normal(17, outer * dim * inner, 2.0)
    want = oracle.normalize(x, outer, dim, inner, p, 1e-12)
    assert_bit_exact(gpuops.normalize(x, outer, dim, inner, p, 1e-12), want, "normalize")
    assert_bit_exact(gpuops.normalize(x, outer, dim, inner, p, 1e-12, inplace=True), want, "in place")


@pytest.mark.parametrize("p", [1.0, 2.0, 2.5])
def test_normalize_special_values(gpu, p):
    x = with_specials(normal(18, 30 * 64, 2.0), 18)
    for eps in (1e-12, 0.0, 10.0):
        assert_bit_exact(gpuops.normalize(x, 30, 64, 1, p, eps), oracle.normalize(x, 30, 64, 1, p, eps),
                         "normalize specials eps=%g" % eps)
    z = np.zeros(4 * 6 * 5, F)
    assert_bit_exact(gpuops.normalize(z, 4, 6, 5, p, 1e-12), oracle.normalize(z, 4, 6, 5, p, 1e-12), "zeros")


@pytest.mark.parametrize("args", [{}, {"p": 1.0}, {"p": 3.0, "axis": -1, "eps": 1e-6}, {"axis": 0}])
def test_normalize_op(ws, args):
    x = normal(19, (4, 32, 5, 3), 2.0)
    got = run(ws, "Normalize", [("x", x)], args)
    want = oracle.normalize_op(x, args.get("p", 2.0), args.get("axis", 1), args.get("eps", 1e-12))
    assert got.shape == x.shape
    assert_bit_exact(got, want, "normalize op")


# ----------------------------------------------------------- SSDNormalize ---
SSD_SHAPES = [(2, 5, 12), (3, 512, 1), (2, 16, 100), (3, 9, 64), (1, 600, 3), (2, 1, 9), (1, 33, 4097),
              (2, 64, 1444), (5, 3, 7), (1, 128, 4096), (3, 20, 1025), (2, 512, 361), (1, 1000, 50), (2, 70, 33),
              (1, 512, 1444), (2, 1030, 24), (2, 1100, 68), (1, 2049, 31), (3, 4096, 7), (2, 5000, 3), (1, 1100, 14),
              (1100, 17, 1), (1025, 1000, 1), (1030, 2049, 1)]


@pytest.mark.parametrize("scale_kind", ["none", "shared", "channel"])
@pytest.mark.parametrize("batch,channel,spatial", SSD_SHAPES)
def test_ssd_normalize_per_position(gpu, batch, channel, spatial, scale_kind):
    """Channel sums fold in index order on one lane: no tolerance."""
    x = normal(60, batch * channel * spatial, 2.0)
    scale = {"none": None, "shared": F([20.0]), "channel": normal(61, channel) + F(20)}[scale_kind]
    shared = scale_kind != "channel"
    want = oracle.ssd_normalize(x, batch, channel, spatial, False, shared, 1e-5, scale)
    assert_bit_exact(gpuops.ssd_normalize(x, batch, channel, spatial, False, shared, 1e-5, scale), want, "ssd")
    assert_bit_exact(gpuops.ssd_normalize(x, batch, channel, spatial, False, shared, 1e-5, scale, inplace=True), want,
                     "ssd in place")


@pytest.mark.parametrize("scale_kind", ["none", "shared", "channel"])
@pytest.mark.parametrize("batch,channel,spatial", SSD_SHAPES + [(2, 512, 1444), (70, 8, 2048), (3, 7, 11111),
                                                                  (70000, 2, 3), (66000, 1, 8)])
def test_ssd_normalize_per_item(gpu, batch, channel, spatial, scale_kind):
    """The item's fp64 sum is split over workgroups and lanes: 1e-5 relative, and
    the count of differing outputs (none in these cases) is checked as well."""
    x = normal(62, batch * channel * spatial, 2.0) + F(0.25)
    scale = {"none": None, "shared": F([20.0]), "channel": normal(63, channel) + F(20)}[scale_kind]
    shared = scale_kind != "channel"
    want = oracle.ssd_normalize(x, batch, channel, spatial, True, shared, 1e-5, scale)
    got = gpuops.ssd_normalize(x, batch, channel, spatial, True, shared, 1e-5, scale)
    assert assert_rel_close(got, want, 1e-5, "ssd per item") == 0
    got = gpuops.ssd_normalize(x, batch, channel, spatial, True, shared, 1e-5, scale, inplace=True)
    assert assert_rel_close(got, want, 1e-5, "ssd per item in place") == 0


def test_ssd_normalize_special_values(gpu):
    x = with_specials(normal(64, 6 * 32 * 10, 2.0), 64)
    for across in (False, True):
        for eps in (1e-5, 0.0):
            want = oracle.ssd_normalize(x, 6, 32, 10, across, True, eps)
            assert_bit_exact(gpuops.ssd_normalize(x, 6, 32, 10, across, True, eps), want,
                             "ssd specials across=%s eps=%g" % (across, eps))
    z = np.zeros(4 * 6 * 5, F)
    for across in (False, True):
        for eps in (1e-5, 0.0):
            assert_bit_exact(gpuops.ssd_normalize(z, 4, 6, 5, across, True, eps),
                             oracle.ssd_normalize(z, 4, 6, 5, across, True, eps), "ssd zeros")


@pytest.mark.parametrize("args", [{}, {"across_spatial": False}, {"across_spatial": False, "channel_shared": False},
                                  {"channel_shared": False, "eps": 1e-3}])
def test_ssd_normalize_op(ws, args):
    x = normal(65, (3, 24, 9, 7), 2.0)
    across, shared, eps = args.get("across_spatial", True), args.get("channel_shared", True), args.get("eps", 1e-5)
    scale = F([20.0]) if shared else uniform(66, 24, 10.0, 30.0)
    got = run(ws, "SSDNormalize", [("x", x)], args)
    assert got.shape == x.shape
    assert assert_rel_close(got, oracle.ssd_normalize_op(x, None, across, shared, eps), 1e-5, "ssd op") == 0
    got = run(ws, "SSDNormalize", [("x", x), ("s", scale)], args)
    assert assert_rel_close(got, oracle.ssd_normalize_op(x, scale, across, shared, eps), 1e-5, "ssd op scale") == 0
    if shared:
        with pytest.raises(ShadowError, match="Check Failed"):
            run(ws, "SSDNormalize", [("x", x), ("s2", F([1.0, 2.0]))], args)


# ---------------------------------------------------------------- pooling ---
POOL_2D = [
    ((2, 3, 12, 12), [3], [2], [0], True), ((2, 3, 12, 12), [3], [2], [1], True),
    ((2, 3, 12, 12), [3], [2], [1], False), ((1, 2, 7, 9), [2, 3], [2, 1], [1, 0], True),
    ((2, 4, 7, 7), [7], [1], [0], True), ((1, 1, 5, 5), [5], [3], [2], True),
    ((3, 2, 8, 8), [2], [2], [0], False), ((1, 2, 6, 6), [3], [3], [2], True),
    ((2, 16, 56, 56), [3], [2], [0], True), ((1, 5, 33, 17), [5, 3], [1, 2], [2, 1], False),
    # several row bands per plane, padded and unpadded; kernels with and without an unrolled form
    ((1, 3, 112, 112), [3], [2], [0], True), ((1, 3, 112, 112), [3], [2], [1], True),
    ((2, 2, 90, 70), [2], [2], [0], True), ((1, 2, 64, 64), [3], [1], [1], False),
    ((1, 2, 75, 61), [4, 3], [3, 2], [1, 1], True), ((1, 1, 150, 50), [2], [1], [0], False),
    # rows too wide for more than two output rows per band, then too wide for any band
    ((1, 1, 9, 2000), [3], [1], [1], True), ((1, 1, 7, 3000), [3], [2], [0], True),
    ((1, 2, 40, 40), [13], [5], [6], True),
    # windows of 16 cells and more on small planes: the two-step maximum (pyramid pooling: 5, 9, 13 at stride 1)
    ((2, 8, 13, 13), [5], [1], [2], False), ((2, 8, 13, 13), [9], [1], [4], False), ((2, 8, 13, 13), [13], [1], [6], False),
    ((1, 5, 19, 19), [13], [1], [6], True), ((3, 3, 14, 14), [7], [1], [3], True), ((1, 7, 20, 20), [4, 5], [2, 1], [1, 2], True),
    ((2, 2, 16, 11), [6, 4], [3, 2], [0, 1], False),
    # planes of 513 to 1024 outputs: whole planes for the two-step maximum, bands for the rest
    ((2, 5, 26, 26), [13], [1], [6], False), ((1, 3, 32, 32), [5], [1], [2], False), ((2, 3, 30, 23), [9, 4], [1, 1], [4, 2], True),
    ((1, 2, 33, 32), [5], [1], [2], False),
    # row bands at a column stride of 1, four outputs per lane: pads of 0 .. 3 (the first quad starts 0 .. 3
    # outputs left of the row), rows that end inside a quad, the unrolled 3x3 and 5x5 and other windows,
    # a row stride of 2, windows that overhang below and to the right
    ((1, 3, 40, 45), [3], [1], [1], False), ((1, 2, 40, 47), [5], [1], [2], False), ((1, 2, 41, 46), [5], [1], [0], False),
    ((2, 2, 36, 50), [5, 3], [1, 1], [2, 1], True), ((1, 2, 50, 37), [3, 7], [2, 1], [1, 3], True),
    ((1, 3, 33, 65), [4, 6], [1, 1], [3, 3], False), ((1, 2, 70, 70), [7], [1], [3], False),
    ((1, 1, 30, 130), [9, 5], [1, 1], [4, 2], True), ((1, 2, 112, 112), [5], [1], [2], False),
    ((1, 1, 64, 300), [3], [1], [1], True), ((1, 2, 28, 61), [13], [1], [6], False),
    # small planes, square windows of 5, 7, 9, 13 at a column stride of 1, four outputs per lane from 128-bit
    # row pieces: output rows that end 1, 2, 3 outputs into a quad, a row stride of 2 and 3, no padding,
    # overhanging windows; 11 wide: the same lanes cell by cell
    ((3, 5, 17, 17), [7], [2, 1], [3], True), ((2, 4, 21, 18), [9], [1], [4], False), ((2, 6, 15, 15), [5], [1], [0], False),
    ((5, 3, 12, 22), [13], [3, 1], [6], True), ((2, 3, 11, 11), [11], [1], [5], False), ((9, 2, 13, 13), [13], [1], [6], False),
]


@pytest.mark.parametrize("pool", [0, 1])
@pytest.mark.parametrize("shape,kernel,stride,pad,full", POOL_2D)
def test_pooling2d_op(ws, pool, shape, kernel, stride, pad, full):
    x = with_specials(normal(20, shape, 2.0), 20).reshape(shape)
    args = {"pool": pool, "kernel_size": kernel, "stride": stride, "pad": pad, "full_pooling": full}
    got = run(ws, "Pooling", [("x", x)], args)
    want = oracle.pooling_op(x, pool, kernel, stride, pad, full_pooling=full)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "pooling2d")


@pytest.mark.parametrize("pool", [0, 1])
@pytest.mark.parametrize("full", [False, True])
@pytest.mark.parametrize("shape,kernel,pad", [
    ((2, 3, 112, 112), 3, 0), ((2, 3, 112, 112), 3, 1), ((1, 2, 56, 64), 2, 0), ((3, 2, 33, 40), 3, 1),
    ((1, 2, 41, 72), 3, 0), ((1, 1, 3, 8), 3, 1), ((2, 2, 1, 16), 3, 1), ((1, 3, 50, 48), 2, 0),
    ((2, 1, 64, 256), 3, 1), ((1, 1, 30, 1024), 3, 0)])
def test_pooling_by_two_without_staging(ws, gpu, pool, full, shape, kernel, pad):
    """3x3 (pad 0 or 1) and 2x2 windows at stride 2 over rows of a multiple of eight columns: where the output
    is half as wide as the input (with either rounding of the output size) the kernel without staging runs --
    asked of the plan query -- and the results are those of the reference's walk, clipped windows, NaNs,
    infinities and equal cells included."""
    x = with_specials(normal(23, shape, 2.0), 23).reshape(shape)
    x[..., 0, :] = np.where(np.arange(shape[3]) % 3 == 0, -np.inf, x[..., 0, :])
    x[..., -1] = np.float32(-3.4028235e38)  # lowest(): equal to the fold's start value
    args = {"pool": pool, "kernel_size": [kernel], "stride": [2], "pad": [pad], "full_pooling": full}
    got = run(ws, "Pooling", [("x", x)], args)
    want = oracle.pooling_op(x, pool, [kernel], [2], [pad], full_pooling=full)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "pooling by two")
    path, variant, grid = ctypes.c_int(), ctypes.c_int(), ctypes.c_uint()
    assert shadow_amd.hip().shdw_hip_pooling2d_plan(shadow_amd.ints(list(shape)), pool, kernel, kernel, 2, 2, pad, pad,
                                                    shadow_amd.ints(list(want.shape)), ctypes.byref(path),
                                                    ctypes.byref(variant), ctypes.byref(grid)) == 0
    halves = want.shape[3] * 2 == shape[3]
    small = path.value == 23  # whole small planes in LDS keep their kernel
    assert small or (path.value == 26) == halves, (path.value, want.shape)


@pytest.mark.parametrize("pool", [0, 1])
@pytest.mark.parametrize("shape", [(2, 3, 40, 64), (1, 2, 33, 128), (1, 1, 5, 4), (2, 2, 1, 8), (1, 1, 70, 260),
                                   (3, 1, 2, 1028), (1, 4, 112, 112),
                                   (2, 8, 112, 112)])  # 196 workgroups: three whole runs of 64 and a rest of four
def test_pooling_3x3_stride_1_without_staging(ws, gpu, pool, shape):
    """3x3 at stride 1 with one cell of padding on rows of a multiple of four columns: the output is as large
    as the input, and planes too large for the whole-plane kernel take the kernel without staging (asked of
    the plan query).  Edge columns and rows, NaNs, infinities, signed zeros and lowest() are planted."""
    x = with_specials(normal(24, shape, 2.0), 24).reshape(shape)
    x[..., 0] = np.where(np.arange(shape[2])[:, None].repeat(1, 1)[:, 0] % 2 == 0, -0.0, 0.0).astype(np.float32)
    x[..., -1] = np.float32(-3.4028235e38)
    x[..., 0, 1:3] = np.inf
    args = {"pool": pool, "kernel_size": [3], "stride": [1], "pad": [1], "full_pooling": False}
    got = run(ws, "Pooling", [("x", x)], args)
    want = oracle.pooling_op(x, pool, [3], [1], [1], full_pooling=False)
    assert got.shape == want.shape == x.shape
    assert_bit_exact(got, want, "pooling 3x3 s1")
    path, variant, grid = ctypes.c_int(), ctypes.c_int(), ctypes.c_uint()
    assert shadow_amd.hip().shdw_hip_pooling2d_plan(shadow_amd.ints(list(shape)), pool, 3, 3, 1, 1, 1, 1,
                                                    shadow_amd.ints(list(shape)), ctypes.byref(path),
                                                    ctypes.byref(variant), ctypes.byref(grid)) == 0
    assert path.value in (23, 27), path.value  # whole small planes in LDS, or no staging


# The maximum keeps the earlier of equal cells and never takes a NaN: planes of signed
# zeros, -inf, lowest() and NaNs show whether an implementation that folds rows first
# returns the cell the row-major walk returns.
@pytest.mark.parametrize("shape,kernel,pad", [((3, 4, 13, 13), [5], [2]), ((2, 3, 14, 14), [13], [6]),
                                               ((2, 2, 19, 19), [9], [4]), ((1, 3, 56, 56), [5], [2]),
                                               ((1, 2, 40, 61), [7], [3]), ((1, 2, 45, 50), [3], [1]),
                                               ((2, 3, 15, 17), [7], [3])])
def test_max_pooling_ties_and_nans_in_wide_windows(ws, shape, kernel, pad):
    rng = np.random.default_rng(31)
    pick = rng.integers(0, 6, size=shape)
    x = np.choose(pick, [F(0.0), F(-0.0), F(-np.inf), F(np.finfo(F).min), F(np.nan), F(-1.0)]).astype(F)
    x[0, 0] = np.where(rng.random(shape[2:]) < 0.5, F(0.0), F(-0.0))
    x[-1, -1] = np.nan
    args = {"pool": 0, "kernel_size": kernel, "stride": [1], "pad": pad, "full_pooling": False}
    got = run(ws, "Pooling", [("x", x)], args)
    assert_bit_exact(got, oracle.pooling_op(x, 0, kernel, [1], pad, full_pooling=False), "max pooling ties")


@pytest.mark.parametrize("pool", [0, 1])
@pytest.mark.parametrize("shape,kernel,stride,pad", [((2, 2, 6, 7, 8), [3], [2], [1]),
                                                     ((1, 3, 4, 5, 5), [2, 3, 2], [1, 2, 2], [0, 1, 1]),
                                                     ((2, 2, 3, 4, 4), [3, 4, 4], [1], [0]),
                                                     ((1, 4, 8, 14, 14), [2], [2], [0])])
def test_pooling3d_op(ws, pool, shape, kernel, stride, pad):
    x = normal(21, shape, 2.0)
    got = run(ws, "Pooling", [("x", x)], {"pool": pool, "kernel_size": kernel, "stride": stride, "pad": pad})
    want = oracle.pooling_op(x, pool, kernel, stride, pad)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "pooling3d")


# whole-plane windows: both workgroup shapes, chunked and unchunked rows, ragged last group
@pytest.mark.parametrize("pool", [0, 1])
@pytest.mark.parametrize("shape", [(4, 128, 7, 7), (3, 5, 14, 14), (2, 3, 56, 56), (1, 70, 3, 3), (2, 2, 4, 2),
                                   (130, 2048, 7, 7), (2, 9, 10, 10), (1, 3, 2, 7, 7), (2, 65, 13, 15),
                                   # planes of 256 elements and more: the streaming average with 1, 2, 8, 32
                                   # and 64 rows per wave, one chunk and several, odd lengths, ragged last
                                   # wave and workgroup; the maximum by Reduce's row kernels or, with few rows,
                                   # by the plane kernel
                                   (20, 30, 17, 17), (8, 64, 70, 70), (13, 41, 129, 65), (40, 128, 16, 16),
                                   (64, 300, 18, 18), (71, 1023, 16, 17), (300, 1024, 16, 16), (1, 1, 16, 16)])
def test_global_pooling_op(ws, pool, shape):
    x = normal(22, shape, 2.0)
    got = run(ws, "Pooling", [("x", x)], {"pool": pool, "global_pooling": True})
    want = oracle.pooling_op(x, pool, global_pooling=True)
    assert got.shape == want.shape == tuple(shape[:2]) + (1,) * (len(shape) - 2)
    assert_bit_exact(got, want, "global pooling")


# Blobs start on allocator boundaries; pointers made of a blob and an offset, as the
# Blas face passes them, may start on any float.  One shape per kernel layout.
ODD_POINTER_COLUMNS = [(64, 1000, 1), (300, 4, 2), (5000, 21, 1), (1100, 333, 1), (2, 21, 63), (4, 8, 1024), (2, 150, 300),
                       (1, 512, 33), (2, 100, 100), (3, 4096, 7), (2, 1300, 30), (2, 600, 64), (1, 2048, 196)]


@pytest.mark.parametrize("offset", [1, 2, 3])
@pytest.mark.parametrize("outer,dim,inner", ODD_POINTER_COLUMNS)
def test_column_ops_on_pointers_off_the_vector_boundary(gpu, outer, dim, inner, offset):
    x = normal(29, outer * dim * inner, 3.0)
    assert_bit_exact(gpuops.softmax(x, outer, dim, inner, offset=offset), oracle.softmax(x, outer, dim, inner), "softmax")
    assert_bit_exact(gpuops.softmax(x, outer, dim, inner, inplace=True, offset=offset),
                     oracle.softmax(x, outer, dim, inner), "softmax in place")
    assert_bit_exact(gpuops.normalize(x, outer, dim, inner, 2.0, 1e-12, offset=offset),
                     oracle.normalize(x, outer, dim, inner, 2.0, 1e-12), "normalize")
    scale = uniform(30, dim, 0.5, 2.0)
    assert_bit_exact(gpuops.ssd_normalize(x, outer, dim, inner, False, False, 1e-5, scale, offset=offset),
                     oracle.ssd_normalize(x, outer, dim, inner, False, False, 1e-5, scale), "ssd normalize")


@pytest.mark.parametrize("offset", [1, 3])
@pytest.mark.parametrize("pool", [0, 1])
@pytest.mark.parametrize("shape,kernel,stride,pad", [
    ((2, 3, 12, 12), [3], [2], [1]), ((2, 16, 56, 56), [3], [2], [0]), ((1, 3, 112, 112), [3], [2], [1]),
    ((130, 64, 7, 7), [3], [1], [1]), ((2, 8, 13, 13), [5], [1], [2]), ((1, 1, 9, 2000), [3], [1], [1]),
    ((4, 128, 7, 7), [7], [1], [0]), ((3, 5, 14, 14), [14], [1], [0]), ((20, 30, 17, 17), [17], [1], [0]),
    ((40, 128, 16, 16), [16], [1], [0]), ((2, 3, 56, 56), [56], [1], [0]), ((2, 2, 6, 7, 8), [3], [2], [1]),
    ((1, 3, 64, 64), [5], [1], [2]), ((1, 2, 60, 44), [3], [1], [1])])
def test_pooling_on_pointers_off_the_vector_boundary(gpu, pool, shape, kernel, stride, pad, offset):
    x = normal(32, shape, 2.0)
    want = oracle.pooling_op(x, pool, kernel, stride, pad)
    nsp = len(shape) - 2
    got = gpuops.pooling(x, shape, pool, kernel * nsp, stride * nsp, pad * nsp, want.shape, offset=offset)
    assert_bit_exact(got, want.ravel(), "pooling")


def test_pooling_op_errors(ws):
    ws.set_blob("x", np.zeros((2, 3, 8, 8), F))
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("Pooling", ["x"], ["o"], {"pool": 2, "kernel_size": [2]})
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("Pooling", ["x"], ["x"], {"kernel_size": [2]}).run()  # in place is refused
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("Pooling", ["x"], ["o2"], {"kernel_size": [2, 2, 2]}).run()
    ws.set_blob("flat", np.zeros((2, 3, 8), F))
    with pytest.raises(ShadowError, match="2D or 3D"):
        ws.create_op("Pooling", ["flat"], ["o3"], {"kernel_size": [2]}).run()


def test_entry_point_argument_errors(gpu):
    lib = shadow_amd.hip()
    buf = shadow_amd.Buffer(1024)
    E = -1
    assert lib.shdw_hip_softmax(-1, 2, 2, buf.ptr, buf.ptr, None) == E
    assert lib.shdw_hip_softmax(2, 2, 2, None, buf.ptr, None) == E
    assert lib.shdw_hip_softmax(0, 5, 5, None, None, None) == 0
    assert lib.shdw_hip_normalize(65536, 65536, 2, 2.0, 0.0, buf.ptr, buf.ptr, None) == E
    assert lib.shdw_hip_batch_norm(8, 0, 1, buf.ptr, buf.ptr, buf.ptr, 1.0, 0.0, buf.ptr, None) == E
    assert lib.shdw_hip_axpy_rows(65536, 65536, buf.ptr, buf.ptr, buf.ptr, buf.ptr, None) == E
    sh = shadow_amd.ints([1, 1, 4, 4])
    assert lib.shdw_hip_pooling2d(sh, 2, 2, 2, 1, 1, 0, 0, sh, buf.ptr, buf.ptr, None) == E
    assert lib.shdw_hip_pooling2d(sh, 0, 0, 2, 1, 1, 0, 0, sh, buf.ptr, buf.ptr, None) == E
    assert lib.shdw_hip_pooling2d(sh, 0, 2, 2, 0, 1, 0, 0, sh, buf.ptr, buf.ptr, None) == E
    assert lib.shdw_hip_pooling2d(sh, 0, 2, 2, 1, 1, 0, 0, shadow_amd.ints([2, 1, 3, 3]), buf.ptr, buf.ptr, None) == E


# ------------------------------------------- group / instance / layer norm ---
# The fp64 row sums are associated differently on the GPU (per-lane partials
# combined through LDS) than in the oracle's serial loop.  Contract: 1e-5
# relative on every output; the tests also count differing bits, and every case
# here comes out identical.
@pytest.mark.parametrize("p", [1.0, 2.0])
@pytest.mark.parametrize("outer,dim,inner", [(2, 16, 100), (2, 100, 100), (1, 300, 37), (4, 30, 1), (1, 1000, 70)])
def test_normalize_extreme_magnitudes(gpu, p, outer, dim, inner):
    """Columns of tiny (1e-33, with denormal members), huge (1e30) and mixed
    magnitude, signed zeros, beside ordinary ones."""
    x = normal(20, (outer, dim, inner), 1.0)
    x[:, :, 0::7] *= F(1e-33)
    x[:, :, 1::7] *= F(1e30)
    x[:, ::3, 2::7] *= F(1e-36)
    x[:, 1::4, 3::7] = 0
    x[:, 0, 3::7] = -0.0
    x = x.reshape(-1)
    for eps in (1e-12, 0.0):
        assert_bit_exact(gpuops.normalize(x, outer, dim, inner, p, eps), oracle.normalize(x, outer, dim, inner, p, eps),
                         "normalize ranges eps=%g" % eps)
    got = gpuops.ssd_normalize(x, outer, dim, inner, False, True, 1e-10)
    assert_bit_exact(got, oracle.ssd_normalize(x, outer, dim, inner, False, True, 1e-10), "ssd ranges")


@pytest.mark.parametrize("outer,inner", [(16, 49), (9, 256), (5, 3136), (4, 25088), (4, 70000)])
def test_group_norm_rows_extreme_magnitudes(gpu, outer, inner):
    x = normal(41, (outer, inner), 1.0)
    x[0] *= F(1e-33)
    x[1] *= F(1e28)
    x[2, ::2] = x[2, 0]          # half of the row equal: zero or rounding-size deviations
    x[3, 5:] = F(1.5)            # one outlier, the rest a hair from the mean
    x = x.reshape(-1)
    for eps in (1e-5, 0.0):
        want = oracle.normalize_rows(x, outer, inner, eps)
        assert assert_rel_close(gpuops.group_norm(x, outer, inner, eps), want, 1e-5, "norm rows ranges") == 0


NORM_ROWS = [(6, 49), (4, 784), (8, 1024), (3, 2048), (5, 3136), (2, 4096), (2, 4100), (2, 25088), (7, 5),
             (300, 12), (1, 1), (3, 1000), (2, 8192), (2, 6002), (7, 400), (2100, 1200), (2051, 2048), (9, 256), (3, 16384), (2, 32768), (2, 32772), (1, 70000),
             # a thousand and more short rows: through LDS, 1 to 16 lanes per row
             (2000, 49), (1025, 127), (1500, 5), (4099, 56), (1024, 9), (3000, 66), (5000, 1), (3001, 2), (2048, 4),
             (1031, 12), (1024, 16), (1500, 28), (1111, 60), (1024, 124), (1030, 252), (1024, 255)]


@pytest.mark.parametrize("outer,inner", NORM_ROWS)
def test_group_norm_rows(gpu, outer, inner):
    x = normal(40, outer * inner, 3.0) + F(0.75)
    want = oracle.normalize_rows(x, outer, inner, 1e-5)
    for kw in ({}, {"inplace": True}, {"offset": 1}):
        got = gpuops.group_norm(x, outer, inner, 1e-5, **kw)
        assert assert_rel_close(got, want, 1e-5, "norm rows %s" % kw) == 0


# Long rows, few of them: with the caller's scratch memory every row is cut into slices
# (three launches); without it a workgroup walks a whole row.  Same results either way.
@pytest.mark.parametrize("outer,inner", [(1, 70000), (3, 32768), (2, 32770), (5, 100003), (40, 40000), (511, 32768),
                                         (1, 1000000), (512, 32768), (7, 4000)])
def test_group_norm_long_rows_with_scratch(gpu, outer, inner):
    x = normal(44, outer * inner, 3.0) + F(0.75)
    want = oracle.normalize_rows(x, outer, inner, 1e-5)
    need = shadow_amd.hip().shdw_hip_group_norm_workspace_bytes(outer, inner)
    assert (need > 0) == (outer < 512 and inner >= 32768)
    for kw in ({}, {"inplace": True}, {"offset": 1}):
        got = gpuops.group_norm(x, outer, inner, 1e-5, scratch=True, **kw)
        assert assert_rel_close(got, want, 1e-5, "sliced norm rows %s" % kw) == 0
    s, b = uniform(45, inner, 0.5, 2.0), normal(46, inner)   # LayerNorm's affine pair per position
    want2 = oracle.scale_bias(want, s, b, inner, 1)
    got = gpuops.group_norm(x, outer, inner, 1e-5, s, b, inner, 1, scratch=True)
    assert assert_rel_close(got, want2, 1e-5, "sliced norm rows, per-position affine") == 0
    if inner % 8 == 0:  # GroupNorm's: 8 channels per row
        s, b = uniform(47, 8 * outer, 0.5, 2.0), normal(48, 8 * outer)
        want3 = oracle.scale_bias(want, s, b, 8 * outer, inner // 8)
        got = gpuops.group_norm(x, outer, inner, 1e-5, s, b, 8 * outer, inner // 8, scratch=True)
        assert assert_rel_close(got, want3, 1e-5, "sliced norm rows, per-channel affine") == 0


@pytest.mark.parametrize("shape,group", [((2, 8, 5, 5), 1), ((2, 8, 5, 5), 4), ((4, 32, 14, 14), 8), ((2, 6, 7, 3), 6),
                                         ((4, 512, 7, 7), 512), ((8, 256, 3, 3), 128), ((2, 1024, 5, 5), 1024),
                                         ((1, 64, 56, 56), 32), ((2, 16, 64, 64), 1)])
def test_group_and_instance_norm_op(ws, shape, group):
    x = normal(41, shape, 2.0) + F(0.5)
    scale, bias = uniform(42, shape[1], 0.5, 2.0), normal(43, shape[1])
    got = run(ws, "GroupNorm", [("x", x)], {"group": group})
    assert got.shape == x.shape
    assert assert_rel_close(got, oracle.group_norm_op(x, group), 1e-5, "group norm") == 0
    got = run(ws, "GroupNorm", [("x", x), ("s", scale), ("b", bias)], {"group": group, "eps": 1e-3})
    assert assert_rel_close(got, oracle.group_norm_op(x, group, 1e-3, scale, bias), 1e-5, "group norm affine") == 0
    got = run(ws, "InstanceNorm", [("x", x), ("s", scale), ("b", bias)], {})
    assert assert_rel_close(got, oracle.instance_norm_op(x, 1e-5, scale, bias), 1e-5, "instance norm") == 0
    got = run(ws, "InstanceNorm", [("x", x)], {"eps": 1e-2})
    assert assert_rel_close(got, oracle.instance_norm_op(x, 1e-2), 1e-5, "instance norm plain") == 0


@pytest.mark.parametrize("shape,ns", [((4, 10, 32), [32]), ((2, 3, 6, 5), [6, 5]), ((64, 768), [768]), ((2, 3, 4), [3, 4]),
                                      ((3, 5000), [5000])])
def test_layer_norm_op(ws, shape, ns):
    x = normal(44, shape, 2.0)
    scale, bias = uniform(45, ns, 0.5, 2.0), normal(46, ns)
    got = run(ws, "LayerNorm", [("x", x)], {"normalized_shape": ns})
    assert got.shape == x.shape
    assert assert_rel_close(got, oracle.layer_norm_op(x, ns), 1e-5, "layer norm") == 0
    got = run(ws, "LayerNorm", [("x", x), ("s", scale), ("b", bias)], {"normalized_shape": ns, "eps": 1e-6})
    assert assert_rel_close(got, oracle.layer_norm_op(x, ns, 1e-6, scale, bias), 1e-5, "layer norm affine") == 0


def test_norm_special_values_and_errors(ws):
    # a NaN or inf poisons its own row only; constant rows give 0 / sqrt(eps)
    x = normal(47, (6, 64), 1.0)
    x[1, 3], x[2, 5], x[4, :] = np.nan, np.inf, 2.5
    got = run(ws, "LayerNorm", [("x", x)], {"normalized_shape": [64]})
    assert_bit_exact(got, oracle.layer_norm_op(x, [64]), "norm specials")
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("LayerNorm", ["x"], ["o1"], {})
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("LayerNorm", ["x"], ["o2"], {"normalized_shape": [32]}).run()
    ws.set_blob("img", np.zeros((2, 6, 4, 4), F))
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("GroupNorm", ["img"], ["o3"], {"group": 4}).run()
    ws.set_blob("s5", np.ones(5, F))
    ws.set_blob("b6", np.ones(6, F))
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("GroupNorm", ["img", "s5", "b6"], ["o4"], {"group": 2}).run()
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("InstanceNorm", ["img", "b6"], ["o5"], {}).run()
    lib = shadow_amd.hip()
    buf = shadow_amd.Buffer(1024)
    assert lib.shdw_hip_group_norm(2, 8, 1e-5, buf.ptr, buf.ptr, None, 1, 1, buf.ptr, None) == -1
    assert lib.shdw_hip_group_norm(-1, 8, 1e-5, buf.ptr, None, None, 1, 1, buf.ptr, None) == -1
    assert lib.shdw_hip_group_norm(0, 8, 1e-5, None, None, None, 1, 1, None, None) == 0
