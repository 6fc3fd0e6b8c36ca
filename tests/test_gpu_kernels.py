"""Parity of every C-ABI kernel entry point with the CPU oracle on the same
seeded inputs.  Bit-exact unless stated; fp64-accumulating reductions are held
to |gpu - cpu| <= 1e-5 |cpu| (their association order differs)."""
import ctypes

import numpy as np
import pytest

import oracle
import shadow_amd
from shadow_amd import Buffer
from tests import gpuops
from tests.helpers import (assert_bit_exact, assert_rel_close, normal, ulp_distance, uniform,
                           with_specials)

pytestmark = pytest.mark.gpu
F = np.float32

EXACT_UNARY = {0: "abs", 1: "square", 2: "sqrt", 3: "log", 4: "exp", 5: "sin", 6: "cos", 7: "tan",
               8: "asin", 9: "acos", 10: "atan", 11: "floor", 12: "ceil", 13: "neg", 14: "reciprocal"}

SIZES = [1, 3, 4, 5, 63, 64, 255, 1024, 1027, 4096 + 2, 100003, 1 << 20]


@pytest.mark.parametrize("n", SIZES)
def test_set(gpu, n):
    assert_bit_exact(gpuops.set_(n, -1.25), oracle.blas_set(n, -1.25), "set")


@pytest.mark.parametrize("op", sorted(EXACT_UNARY))
@pytest.mark.parametrize("n", [5, 1027, 100003])
def test_unary_exact(gpu, op, n):
    x = with_specials(normal(10 + op, n, 2.0), op)
    assert_bit_exact(gpuops.unary(op, x), oracle.unary(op, x), EXACT_UNARY[op])


@pytest.mark.parametrize("op", [0, 2, 4, 14])
def test_unary_inplace_and_misaligned(gpu, op):
    x = with_specials(normal(20 + op, 70001, 2.0), op)
    want = oracle.unary(op, x)
    assert_bit_exact(gpuops.unary(op, x, inplace=True), want, "in place")
    for off in (1, 2, 3):
        assert_bit_exact(gpuops.unary(op, x, offset=off), want, "offset %d" % off)


def _shifted(x, off):
    """x on the device, `off` floats past a 16-byte boundary."""
    buf = Buffer(4 * (x.size + off) + 16)
    buf.upload(x, 4 * off)
    return buf, buf.ptr + 4 * off


@pytest.mark.parametrize("offs", [(1, 2, 3), (0, 1, 0), (3, 3, 1), (2, 0, 2)])
def test_operands_on_different_dword_offsets(gpu, offs):
    """The 128-bit accesses of the streaming kernels take any float pointer: every
    operand shifted by its own number of floats off 16-byte alignment."""
    lib = shadow_amd.hip()
    n = 70003
    a, b = normal(30, n, 2.0), uniform(31, n, 0.5, 2.0)
    (ba, pa), (bb, pb), (by, py) = _shifted(a, offs[0]), _shifted(b, offs[1]), _shifted(np.zeros(n, F), offs[2])
    for op in (0, 3, 5):  # add, div, max
        gpuops.check(lib.shdw_hip_binary(op, n, pa, pb, py, None))
        assert_bit_exact(by.download(count=n, offset_bytes=4 * offs[2]), oracle.binary(op, a, b), "binary %d" % op)
    # Eltwise sum with coefficients, three inputs
    c = normal(32, n)
    (bc, pc) = _shifted(c, offs[0])
    ptrs = (ctypes.c_void_p * 3)(pa, pb, pc)
    co = (ctypes.c_float * 3)(0.5, -1.25, 2.0)
    gpuops.check(lib.shdw_hip_eltwise(1, 3, ptrs, co, n, py, None))
    assert_bit_exact(by.download(count=n, offset_bytes=4 * offs[2]), oracle.eltwise(1, [a, b, c], [0.5, -1.25, 2.0]),
                     "eltwise")
    # BatchNorm and Axpy rows: row parameters per 7 x 11 = 77 elements (rows never vector-aligned)
    rows, inner = 909, 77
    m = rows * inner
    mean, var = normal(33, rows), uniform(34, rows, 0.2, 3.0)
    dm, dv = Buffer.from_numpy(mean), Buffer.from_numpy(var)
    gpuops.check(lib.shdw_hip_batch_norm(m, rows, inner, pa, dm.ptr, dv.ptr, 0.999, 1e-5, py, None))
    assert_bit_exact(by.download(count=m, offset_bytes=4 * offs[2]),
                     oracle.batch_norm(a[:m], mean, var, rows, inner, F(0.999), F(1e-5)), "batch norm")
    alpha = Buffer.from_numpy(normal(35, rows))
    gpuops.check(lib.shdw_hip_axpy_rows(rows, inner, alpha.ptr, pa, pb, py, None))
    assert_bit_exact(by.download(count=m, offset_bytes=4 * offs[2]),
                     oracle.axpy_rows(normal(35, rows), a[:m], b[:m], inner), "axpy rows")


@pytest.mark.parametrize("op", [3, 5, 6, 7, 8, 9, 10])
@pytest.mark.parametrize("scale", [1.0, 100.0, 1e6, 1e30])
def test_unary_libm_wide_ranges(gpu, op, scale):
    """Argument-reduction paths of the trigonometric functions and the whole
    exponent range of log: still bit-exact."""
    x = with_specials(normal(30 + op, 150001, scale), op)
    assert_bit_exact(gpuops.unary(op, x), oracle.unary(op, x), EXACT_UNARY[op])


@pytest.mark.parametrize("op", [0, 1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("n", [7, 4099, 262144 + 1])
def test_binary_and_scalar(gpu, op, n):
    a = with_specials(normal(40 + op, n), op)
    b = with_specials(uniform(50 + op, n, 0.5, 2.0), op + 1)
    assert_bit_exact(gpuops.binary(op, a, b), oracle.binary(op, a, b), "binary %d" % op)
    assert_bit_exact(gpuops.binary(op, a, b, inplace=True), oracle.binary(op, a, b), "in place")
    for alpha in (1.5, -0.0, float("nan")):
        assert_bit_exact(gpuops.binary_scalar(op, a, alpha), oracle.binary_scalar(op, a, alpha),
                         "scalar %d" % op)


def test_binary_pow_exact(gpu):
    r = np.random.default_rng(60)
    a = with_specials(uniform(60, 300001, -4.0, 6.0), 7)
    b = with_specials(normal(61, 300001, 3.0), 8)
    b[::7] = np.round(b[::7])  # integer exponents make negative bases finite
    assert_bit_exact(gpuops.binary(4, a, b), oracle.binary(4, a, b), "pow")
    for alpha in (2.0, 0.5, -3.0, 0.0, float("inf")):
        assert_bit_exact(gpuops.binary_scalar(4, a, alpha), oracle.binary_scalar(4, a, alpha), "pow scalar")
    sa, sb = [64, 1, 33], [1, 5, 1]
    x, y = uniform(62, sa, 0.1, 4.0), normal(63, sb, 2.0)
    so = [64, 5, 33]
    assert_bit_exact(gpuops.broadcast_binary(4, x, sa, y, sb, so), oracle.broadcast_binary(4, x, sa, y, sb, so),
                     "pow broadcast")


def test_max_min_select_semantics(gpu):
    a = np.float32([0.0, -0.0, np.nan, 1.0, np.nan, -np.inf, 5.0])
    b = np.float32([-0.0, 0.0, 1.0, np.nan, np.nan, np.inf, 5.0])
    for op in (5, 6):
        got = gpuops.binary(op, a, b)
        assert_bit_exact(got, oracle.binary(op, a, b), "select")
        # ties and NaN in either position return the left operand
        assert np.signbit(got[0]) == False and np.signbit(got[1]) == True
        assert np.isnan(got[2]) and got[3] == 1.0


def test_level1(gpu):
    x = with_specials(normal(70, 30011), 1)
    y = normal(71, 30011)
    assert_bit_exact(gpuops.scal(0.37, x), oracle.scal(0.37, x), "scal")
    assert_bit_exact(gpuops.copy(x), oracle.copy(x), "copy")
    assert_bit_exact(gpuops.axpy(-1.3, x, y), oracle.axpy(-1.3, x, y), "axpy")
    z = normal(72, 1 << 20)
    assert_rel_close(gpuops.asum(z), oracle.asum(z), 1e-6, "asum")
    assert_rel_close(gpuops.asum(z[:77]), oracle.asum(z[:77]), 1e-6, "asum small")


def test_axpy_is_not_fused(gpu):
    """alpha*x + y with a product that needs rounding: an FMA would differ."""
    x = np.float32([1.0 + 2.0 ** -12] * 8)
    y = np.float32([-(1.0 + 2.0 ** -11)] * 8)
    alpha = float(np.float32(1.0 + 2.0 ** -12))
    want = oracle.axpy(alpha, x, y)
    assert_bit_exact(gpuops.axpy(alpha, x, y), want, "axpy")
    fused = np.float32(np.float64(alpha) * np.float64(x[0]) + np.float64(y[0]))
    assert want[0] != fused  # the case does discriminate


@pytest.mark.parametrize("act", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("n", [9, 66001])
def test_activate_exact(gpu, act, n):
    x = with_specials(normal(80 + act, n, 2.0), act)
    assert_bit_exact(gpuops.activate(x, act, 0.1), oracle.activate(x, act, 0.1), "act %d" % act)
    assert_bit_exact(gpuops.activate(x, act, 0.1, inplace=True), oracle.activate(x, act, 0.1), "in place")


@pytest.mark.parametrize("act", [3, 4, 5, 8])
def test_activate_libm_wide_range(gpu, act):
    x = with_specials(normal(90 + act, 200001, 30.0), act)
    assert_bit_exact(gpuops.activate(x, act), oracle.activate(x, act), "act %d" % act)


@pytest.mark.parametrize("shape,shared", [((2, 3, 5, 7), False), ((2, 3, 5, 7), True),
                                          ((4, 16, 12), False), ((3, 8), False), ((1, 64, 56, 56), False),
                                          ((5, 64, 2), False), ((3, 7, 3), False), ((2, 5, 7, 7), False)])
def test_prelu(gpu, shape, shared):
    x = with_specials(normal(100, shape), 3)
    slope = uniform(101, 1 if shared else shape[1], -0.5, 0.5)
    assert_bit_exact(gpuops.prelu(x, list(shape), shared, slope),
                     oracle.prelu(x, list(shape), shared, slope), "prelu")


@pytest.mark.parametrize("outer,num,inner", [(2, 3, 8), (4, 16, 196), (3, 5, 7), (1, 1, 1000),
                                             (8, 64, 3136), (5, 7, 1), (2, 256, 30),
                                             # vectors that end in the next row, the next row being parameter 0
                                             # again, rows shorter than a vector, a ragged end
                                             (3, 64, 2), (5, 3, 2), (7, 1000, 3), (9, 1, 3), (4, 3, 5), (2, 7, 49),
                                             (11, 2, 6), (1, 13, 2), (3, 4, 1), (5, 64, 1)])
@pytest.mark.parametrize("mode", ["sb", "s", "b"])
def test_scale_bias(gpu, outer, num, inner, mode):
    n = outer * num * inner
    x = with_specials(normal(110, n), 4)
    s = uniform(111, num, 0.5, 1.5) if "s" in mode else None
    b = uniform(112, num, -0.1, 0.1) if "b" in mode else None
    want = oracle.scale_bias(x, s, b, num, inner)
    assert_bit_exact(gpuops.scale_bias(x, s, b, num, inner), want, "scale")
    assert_bit_exact(gpuops.scale_bias(x, s, b, num, inner, inplace=True), want, "in place")
    assert_bit_exact(gpuops.scale_bias(x, s, b, num, inner, offset=1), want, "misaligned")
    relu = oracle.activate(want, 1)
    assert_bit_exact(gpuops.scale_bias(x, s, b, num, inner, relu=True), relu, "scale+relu")


def test_scale_is_not_fused(gpu):
    x = np.float32([1.0 + 2.0 ** -12] * 16)
    s = np.float32([1.0 + 2.0 ** -12])
    b = np.float32([-(1.0 + 2.0 ** -11)])
    want = oracle.scale_bias(x, s, b, 1, 16)
    assert_bit_exact(gpuops.scale_bias(x, s, b, 1, 16), want, "no fma")
    assert want[0] != np.float32(np.float64(x[0]) * np.float64(s[0]) + np.float64(b[0]))


BCAST_CASES = [
    ([8, 64, 12, 12], [1, 64, 1, 1]),
    ([16, 1, 8, 64], [1, 5, 8, 1]),
    ([4, 6, 1, 32], [1, 1, 6, 32]),
    ([128, 64], [1, 1]),
    ([2, 1], [1, 3]),
    ([3, 1, 5, 1, 7], [1, 4, 1, 6, 1]),
    ([2, 3, 1, 2, 1, 3, 1, 2], [1, 1, 4, 1, 5, 1, 2, 1]),
    ([1, 1], [1, 1]),
    ([5, 3], [5, 3]),
    ([1, 7], [9, 1]),
    ([6, 1, 10], [6, 4, 1]),
    ([33, 4], [1, 4]),
    # innermost extent not a multiple of 4: four outputs per lane across row ends
    ([6, 20, 7, 7], [1, 20, 1, 1]),
    ([5, 1, 13, 13], [1, 9, 13, 1]),
    ([3, 7, 1, 9], [1, 1, 5, 9]),
    ([1001, 3], [1, 3]),
    ([2, 3], [2, 3]),
    ([17, 1, 3], [1, 11, 1]),
    ([3, 1, 2, 1, 7], [1, 4, 1, 6, 1]),   # five dims after collapsing
    # a parameter per channel over rows of 2, 3, 5 and 6 elements: vectors that end in the next channel
    ([9, 64, 2], [1, 64, 1]), ([4, 5, 3], [1, 5, 1]), ([7, 3, 5], [1, 3, 1]), ([2, 11, 2, 3], [1, 11, 1, 1]),
]


@pytest.mark.parametrize("sa,sb", BCAST_CASES)
@pytest.mark.parametrize("op", [0, 1, 2, 3, 5, 6])
def test_broadcast_binary(gpu, sa, sb, op):
    so = [max(x, y) for x, y in zip(sa, sb)]
    a = with_specials(normal(120, sa), 5)
    b = with_specials(uniform(121, sb, 0.5, 2.0), 6)
    want = oracle.broadcast_binary(op, a, sa, b, sb, so)
    assert_bit_exact(gpuops.broadcast_binary(op, a, sa, b, sb, so), want, "bcast")


@pytest.mark.parametrize("op", [0, 1, 2, 3])
@pytest.mark.parametrize("k", [2, 3, 4, 5, 8, 9, 11])
def test_eltwise(gpu, op, k):
    n = 40003
    xs = [with_specials(normal(130 + j, n), j) for j in range(k)]
    coeff = [1.0, -0.5, 2.0, 0.25, 1.0, 3.0, -1.0, 0.5, 1.5, -2.0, 0.75][:k] if op == 1 else None
    want = oracle.eltwise(op, xs, coeff)
    assert_bit_exact(gpuops.eltwise(op, xs, coeff), want, "eltwise")


@pytest.mark.parametrize("op", [0, 1, 2, 3])
@pytest.mark.parametrize("k", [2, 4, 9])
def test_eltwise_relu(gpu, op, k):
    """shdw_hip_eltwise_relu is shdw_hip_eltwise followed by relu; with nine inputs the
    activation belongs to the second pass only."""
    n = 70003
    xs = [with_specials(normal(135 + j, n), j) for j in range(k)]
    coeff = [1.0, -0.5, 2.0, 0.25, 1.0, 1.0, -1.0, 3.0, 0.5][:k] if op == 1 else None
    want = oracle.activate(oracle.eltwise(op, xs, coeff if coeff else [1.0] * k), 1)
    got = gpuops.eltwise(op, xs, coeff, relu=True)
    assert_bit_exact(got, want, "eltwise + relu")


def test_eltwise_sum_signed_zero(gpu):
    a = np.float32([-0.0, 0.0, -0.0, 1.0])
    b = np.float32([-0.0, -0.0, 0.0, -1.0])
    got = gpuops.eltwise(1, [a, b])
    assert_bit_exact(got, oracle.eltwise(1, [a, b]), "sum zeros")
    assert not np.signbit(got).any()  # the accumulator starts at +0


@pytest.mark.parametrize("op", [0, 1, 2, 3])
@pytest.mark.parametrize("alias", [0, 1, 2])
def test_eltwise_aliased_output(gpu, op, alias):
    xs = [normal(140 + j, 5003) for j in range(3)]
    cpu_in = [x.copy() for x in xs]
    want = oracle.eltwise(op, cpu_in, None, out=cpu_in[alias]).copy()
    assert_bit_exact(gpuops.eltwise(op, xs, None, alias=alias), want, "aliased")


REDUCE_CASES = [
    ([4, 6, 7, 8], [2, 3]),      # rows, wave per row needs >= 256 rows: block path here
    ([16, 32, 7, 8], [2, 3]),    # rows, wave per row
    ([300, 9], [1]),             # rows, odd length
    ([3, 50, 20], [1]),          # strided, inner % 4 == 0
    ([3, 50, 21], [1]),          # strided, scalar lanes
    ([40, 300], [0]),            # strided with outer == 1
    ([5, 6, 7], []),             # no axes at kernel level: identity windows
    ([2, 3, 4, 5], [0, 1, 2, 3]),
    ([100003], [0]),             # full, split over blocks
    ([1 << 20], [0]),
    ([2, 3, 4, 5], [0, 2]),      # generic
    ([2, 3, 4, 5], [3, 1]),      # generic, list order differs from memory order
    ([6, 1, 5], [1]),            # reduced axis of extent 1
    ([1, 1, 1], [0, 1, 2]),
    ([2, 40000], [1]),           # rows, long, few
    ([2, 30000, 8], [1]),        # strided, 16 waves per tile and a second stage
    ([3, 200, 12], [1]),         # strided, 16 waves per tile, single stage
    ([1000, 49], [1]),           # rows of 49: unaligned 128-bit loads plus one tail element
    ([300, 6, 7, 7], [2, 3]),
    ([3, 40001], [1]),           # long rows that start on odd dwords
    ([500, 3], [1]),             # rows shorter than one vector
    # strided with 8..127 columns: the flat walk over [reduce][inner]
    ([5, 333, 49], [1]),         # odd columns: steps of 980 elements
    ([2, 4097, 127], [1]),       # steps of 508, second stage
    ([4, 1000, 126], [1]),       # steps of 1008
    ([3, 7, 100], [1]),          # less than one step
    ([2, 512, 7, 8], [1]),       # channels over a 7x8 map
    ([130, 64, 7, 7], [1]),
    ([3, 2, 9], [1]),
    # short rows of odd length through LDS, one lane per row
    ([700, 9], [1]), ([513, 127], [1]), ([260, 5], [1]), ([257, 5, 5], [1, 2]), ([1027, 66], [1]),
    # a reduced dim in front of the rows / strided view, folded by the second stage: channel statistics
    # over batch and plane with rows short, medium and sliced; [kept][lead][kept][reduce]; strided
    # views with short, narrow, vector and odd column counts
    ([6, 5, 7, 7], [0, 2, 3]), ([4, 300, 28, 28], [0, 2, 3]), ([3, 2, 300, 301], [0, 2, 3]), ([70, 3, 5], [0, 2]),
    ([3, 4, 5, 6], [1, 3]), ([2, 300, 3, 700], [1, 3]), ([5, 2, 9, 5000], [1, 3]), ([300, 2, 2, 9], [1, 3]),
    ([6, 5, 7, 9], [0, 2]), ([5, 3, 40, 64], [0, 2]), ([3, 2, 9, 256], [0, 2]), ([4, 3, 300, 130], [0, 2]),
    ([2, 3, 4000, 12], [0, 2]), ([7, 2, 33, 1001], [0, 2]), ([9, 4, 3, 7, 5], [0, 1, 3]), ([2, 3, 4, 5, 6], [1, 2, 4]),
    # a short reduced dim behind a long leading one: the leading dim first, the second stage folds slices and
    # the short dim (rows-like and strided-like, lane and workgroup per output, every first-stage kernel)
    ([40, 3, 7], [0, 2]), ([300, 5, 9], [0, 2]), ([3, 33, 4, 16], [1, 3]), ([5000, 2, 3], [0, 2]), ([64, 70, 63], [0, 2]),
    ([40, 6, 7, 5], [0, 2]), ([33, 300, 4, 8], [0, 2]), ([2000, 2, 5, 3], [0, 2]), ([32, 3, 31, 130], [0, 2]),
    ([100, 1030, 2], [0, 2]), ([9000, 1, 4, 1, 3], [0, 2]),
    # two to seven columns with slabs of a step and more: the flat walk
    ([3, 1024, 7], [1]), ([5, 700, 2], [1]), ([2, 9000, 3], [1]), ([4, 300, 5], [1]), ([2, 171, 6], [1]), ([3, 170, 6], [1]),
    ([2, 3, 600, 7], [0, 2]),
    # 4096 and more rows of 2 .. 7 (and 8, the first length past it): four rows per lane; row counts that end inside a lane's rows, a vector, a
    # wave's span; the same behind a reduced leading dim (partials, second stage)
    ([4096, 2], [1]), ([4099, 3], [1]), ([5001, 4], [1]), ([70001, 5], [1]), ([4097, 6], [1]), ([9999, 7], [1]),
    ([4098, 8], [1]), ([1300, 5, 2, 2], [2, 3]), ([3, 5000, 4], [0, 2]), ([2, 4100, 2, 3], [0, 2, 3]),
    # under eight rows over a strided axis whose rows are no whole vectors: four columns per lane on any
    # dword address, the row's cut end (1 to 3 columns) float by float; 63 and 64 columns either side of it
    ([3, 1001], [0]), ([2, 5, 66], [1]), ([7, 130003], [0]), ([4, 2, 65], [1]), ([3, 6, 63], [1]), ([2, 3, 64], [1]),
    ([5, 3, 777], [0, 1]), ([6, 4, 3, 67], [0, 2]),
]


@pytest.mark.parametrize("shape,axes", REDUCE_CASES)
@pytest.mark.parametrize("op", [0, 1, 2, 3, 4, 5, 6])
def test_reduce(gpu, shape, axes, op):
    x = normal(150, shape)
    if op == 0:
        x = uniform(151, shape, 0.9, 1.1)  # keep products in range
    want, _ = oracle.reduce(op, x, shape, axes)
    got, _ = gpuops.reduce(op, x, shape, axes)
    if op in (2, 3):
        assert_bit_exact(got, want, "reduce select")
    else:
        assert_rel_close(got, want, 1e-5, "reduce accumulate")


@pytest.mark.parametrize("shape,axes", [([70000, 8, 100], [1]),   # strided with more than 65535 outer slices
                                        ([66000, 4100], [1]),     # long rows, more than 65535 of them
                                        ([2, 9, 4200000], [1])])  # strided with more than 65535 column tiles
@pytest.mark.parametrize("op", [1, 2])
def test_reduce_beyond_the_second_grid_dimension(gpu, shape, axes, op):
    x = normal(152, shape)
    want, _ = oracle.reduce(op, x, shape, axes)
    got, _ = gpuops.reduce(op, x, shape, axes)
    if op == 2:
        assert_bit_exact(got, want, "reduce max")
    else:
        assert_rel_close(got, want, 1e-5, "reduce sum")


@pytest.mark.parametrize("shape,axes", [([64, 48], [1]), ([3, 64, 8], [1]), ([2, 3, 4, 5], [3, 1]),
                                        ([50000], [0]), ([300, 16], [1]), ([3, 500, 49], [1]), ([2, 6000, 12], [1]), ([300, 49], [1]),
                                        ([1000, 9], [1]),
                                        # the first zero of a window lies under another leading index
                                        ([6, 5, 7, 7], [0, 2, 3]), ([3, 2, 300, 301], [0, 2, 3]), ([5, 2, 9, 500], [1, 3]),
                                        ([6, 5, 7, 9], [0, 2]), ([4, 3, 300, 130], [0, 2]), ([7, 2, 33, 101], [0, 2]),
                                        ([3, 1024, 7], [1]), ([2, 9000, 3], [1]),
                                        ([300, 5, 9], [0, 2]), ([5000, 2, 3], [0, 2]), ([40, 6, 7, 5], [0, 2]), ([2000, 2, 5, 3], [0, 2])])
@pytest.mark.parametrize("op", [2, 3])
def test_reduce_select_special_values(gpu, shape, axes, op):
    """Zeros of both signs, NaNs and infinities: the first extremum in list
    order wins, NaNs are skipped, an all-NaN window returns the identity."""
    r = np.random.default_rng(160 + op)
    x = r.choice(np.float32([0.0, -0.0, np.nan, -1.0, 1.0, np.inf, -np.inf]),
                 size=int(np.prod(shape)), p=[0.3, 0.3, 0.2, 0.05, 0.05, 0.05, 0.05]).astype(np.float32)
    # windows made only of zeros / only of NaNs
    x = x.reshape(shape)
    if len(shape) == 2 and axes == [1]:
        x[0, :] = np.nan
        x[1, :] = np.where(r.random(shape[1]) < 0.5, 0.0, -0.0)
        x[2, :] = np.inf if op == 3 else -np.inf
    want, _ = oracle.reduce(op, x, shape, axes)
    got, _ = gpuops.reduce(op, x, shape, axes)
    assert_bit_exact(got, want, "reduce select specials")


@pytest.mark.parametrize("shape,axes", [([64, 48], [1]), ([300, 49], [1]), ([50000], [0]), ([3, 500, 49], [1]), ([2, 600, 784], [1]),
                                        ([3, 700, 256], [1]), ([2, 6000, 12], [1]), ([3, 1024, 7], [1]), ([300, 5, 9], [0, 2]),
                                        ([4, 300, 28, 28], [0, 2, 3]), ([9, 4100], [1]), ([4099, 3], [1]), ([7, 130003], [0])])
@pytest.mark.parametrize("op", [2, 3])
def test_reduce_select_signalling_nans(gpu, shape, axes, op):
    """Signalling and negative NaNs among ordinary values are skipped like quiet ones:
    the comparison `v < x` is false for every NaN, whatever the hardware's own maximum
    and minimum instructions make of a signalling one."""
    n = int(np.prod(shape))
    r = np.random.default_rng(165 + op)
    bits = normal(166, n).view(np.uint32).copy()
    where = r.random(n)
    bits[where < 0.02] = 0x7FA00000   # signalling NaN
    bits[(where >= 0.02) & (where < 0.03)] = 0xFFA00001  # negative signalling NaN
    bits[(where >= 0.03) & (where < 0.04)] = 0xFFC00000  # negative quiet NaN
    bits[(where >= 0.04) & (where < 0.05)] = 0x80000000  # -0
    bits[(where >= 0.05) & (where < 0.06)] = 0x00000000  # +0
    x = bits.view(np.float32).reshape(shape)
    want, _ = oracle.reduce(op, x, shape, axes)
    assert not np.isnan(want).any()
    got, _ = gpuops.reduce(op, x, shape, axes)
    assert_bit_exact(got, want, "reduce select with signalling NaNs")


def test_reduce_l2_and_avg_definition(gpu):
    x = np.float32([[3, 4], [6, 8]])
    got, _ = gpuops.reduce(6, x, [2, 2], [1])
    assert_bit_exact(got, np.float32([5, 10]), "l2")
    got, _ = gpuops.reduce(4, x, [2, 2], [1])
    assert_bit_exact(got, np.float32([3.5, 7]), "avg")


@pytest.mark.parametrize("outer,num,inner", [(2, 8, 196), (3, 5, 7), (1, 16, 1000), (4, 4, 4)])
def test_fused_tail(gpu, outer, num, inner):
    n = outer * num * inner
    x, r = normal(170, n), normal(171, n)
    s, b = uniform(172, num, 0.5, 1.5), uniform(173, num, -0.1, 0.1)
    t = oracle.scale_bias(x, s, b, num, inner)
    t = oracle.eltwise(1, [t, r], [1.0, 1.0])
    want_y = oracle.activate(t, 1)
    want_m, _ = oracle.reduce(4, want_y, [outer * num, inner], [1])
    y, m = gpuops.scale_residual_relu_rowmean(x, s, b, r, num, inner)
    assert_bit_exact(y, want_y, "fused y")
    assert_rel_close(m, want_m, 1e-5, "fused mean")
    _, m2 = gpuops.scale_residual_relu_rowmean(x, s, b, r, num, inner, want_y=False)
    assert_bit_exact(m2, m, "mean without y")


@pytest.mark.parametrize("form", ["scale", "bias", "both"])
@pytest.mark.parametrize("residual_first", [False, True])
# (101, 4, 12): 101 workgroups, three whole runs of 32 (which the kernel renumbers) and a rest of five
@pytest.mark.parametrize("outer,num,inner", [(2, 8, 196), (3, 5, 7), (2, 3, 1030), (101, 4, 12)])
def test_fused_tail_forms(gpu, form, residual_first, outer, num, inner):
    """The forms a network holds the sequence in: Scale with one parameter blob only, the
    residual as the first Eltwise input, no Reduce behind it."""
    n = outer * num * inner
    x, r = with_specials(normal(174, n), 3), with_specials(normal(175, n), 4)
    s = uniform(176, num, 0.5, 1.5) if form != "bias" else None
    b = uniform(177, num, -0.1, 0.1) if form != "scale" else None
    t = oracle.scale_bias(x, s, b, num, inner)
    t = oracle.eltwise(1, [r, t] if residual_first else [t, r], [1.0, 1.0])
    want_y = oracle.activate(t, 1)
    y, none = gpuops.scale_residual_relu(x, s, b, r, num, inner, residual_first, want_mean=False)
    assert none is None
    assert_bit_exact(y, want_y, "y")
    x, r = normal(174, n), normal(175, n)  # finite values for the mean
    y2, m = gpuops.scale_residual_relu(x, s, b, r, num, inner, residual_first)
    t = oracle.scale_bias(x, s, b, num, inner)
    clean = oracle.activate(oracle.eltwise(1, [r, t] if residual_first else [t, r], [1.0, 1.0]), 1)
    assert_bit_exact(y2, clean, "y with the mean")
    want_m, _ = oracle.reduce(4, clean, [outer * num, inner], [1])
    assert assert_rel_close(m, want_m, 1e-5, "mean") == 0


@pytest.mark.parametrize("form", ["scale", "bias", "both"])
@pytest.mark.parametrize("residual_first", [False, True])
@pytest.mark.parametrize("outer,num,inner", [(2, 8, 196), (3, 5, 7), (2, 3, 1030), (101, 4, 12)])
def test_fused_tail_behind_a_batch_norm(gpu, form, residual_first, outer, num, inner):
    """BatchNorm -> Scale -> Eltwise SUM -> ReLU [-> Reduce AVG] against the five operators of the oracle."""
    n = outer * num * inner
    stat_mean, stat_var = normal(181, num), uniform(182, num, 0.0, 30.0)
    s = uniform(176, num, 0.5, 1.5) if form != "bias" else None
    b = uniform(177, num, -0.1, 0.1) if form != "scale" else None
    factor, eps = np.float32(1 / 999.982), np.float32(1e-3)

    def five(x, r):
        t = oracle.batch_norm(x, stat_mean, stat_var, num, inner, factor, eps)
        t = oracle.scale_bias(t, s, b, num, inner)
        return oracle.activate(oracle.eltwise(1, [r, t] if residual_first else [t, r], [1.0, 1.0]), 1)

    x, r = with_specials(normal(174, n), 3), with_specials(normal(175, n), 4)
    y, none = gpuops.batch_norm_scale_residual_relu(x, stat_mean, stat_var, factor, eps, s, b, r, num, inner,
                                                    residual_first, want_mean=False)
    assert none is None
    assert_bit_exact(y, five(x, r), "y")
    x, r = normal(174, n), normal(175, n)  # finite values for the mean
    y2, m = gpuops.batch_norm_scale_residual_relu(x, stat_mean, stat_var, factor, eps, s, b, r, num, inner, residual_first)
    clean = five(x, r)
    assert_bit_exact(y2, clean, "y with the mean")
    want_m, _ = oracle.reduce(4, clean, [outer * num, inner], [1])
    assert assert_rel_close(m, want_m, 1e-5, "mean") == 0
    none, m2 = gpuops.batch_norm_scale_residual_relu(x, stat_mean, stat_var, factor, eps, s, b, r, num, inner,
                                                     residual_first, want_y=False)
    assert none is None
    assert_bit_exact(m2, m, "mean without y")


def test_argument_errors(gpu):
    import shadow_amd
    lib = gpu
    buf = shadow_amd.Buffer(64)
    assert lib.shdw_hip_unary(15, 4, buf.ptr, buf.ptr, None) == -1
    assert lib.shdw_hip_binary(7, 4, buf.ptr, buf.ptr, buf.ptr, None) == -1
    assert lib.shdw_hip_activate(0, 0.1, 4, buf.ptr, buf.ptr, None) == -1
    assert lib.shdw_hip_unary(0, 4, None, buf.ptr, None) == -1
    assert lib.shdw_hip_unary(0, 0, buf.ptr, buf.ptr, None) == 0
    sh = shadow_amd.ints([2, 3])
    assert lib.shdw_hip_broadcast_binary(0, 2, sh, shadow_amd.ints([2, 2]), sh, buf.ptr, buf.ptr,
                                         buf.ptr, None) == -1
    assert lib.shdw_hip_reduce(1, 2, sh, 1, shadow_amd.ints([-1]), buf.ptr, buf.ptr, None, 0, None) == -1
    big = shadow_amd.ints([1 << 20])
    assert lib.shdw_hip_reduce(1, 1, big, 1, shadow_amd.ints([0]), buf.ptr, buf.ptr, None, 0, None) == -3
    p = buf.ptr
    assert lib.shdw_hip_scale_residual_relu(16, 2, 8, p, None, None, p, 0, p, p, None) == -1  # no parameters
    assert lib.shdw_hip_scale_residual_relu(16, 2, 8, p, p, p, p, 0, None, None, None) == -1  # no output
    assert lib.shdw_hip_scale_residual_relu(16, 2, 8, p, p, p, None, 0, p, p, None) == -1     # no residual
    assert lib.shdw_hip_scale_residual_relu(15, 2, 8, p, p, p, p, 0, p, p, None) == -1        # not whole rows
    assert lib.shdw_hip_scale_residual_relu_rowmean(16, 2, 8, p, p, None, p, p, p, None) == -1
    assert lib.shdw_hip_batch_norm_scale_residual_relu(16, 2, 8, p, None, p, 1.0, 1e-5, p, p, p, 0, p, p, None) == -1
    assert lib.shdw_hip_batch_norm_scale_residual_relu(16, 2, 8, p, p, None, 1.0, 1e-5, p, p, p, 0, p, p, None) == -1
    assert lib.shdw_hip_batch_norm_scale_residual_relu(16, 2, 8, p, p, p, 1.0, 1e-5, None, None, p, 0, p, p, None) == -1
    assert lib.shdw_hip_batch_norm_scale_residual_relu(15, 2, 8, p, p, p, 1.0, 1e-5, p, p, p, 0, p, p, None) == -1
