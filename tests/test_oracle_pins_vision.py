"""Pins for the oracle's Axpy / BatchNorm / Softmax / Normalize / Pooling / LRN / GridSample
restatements.  The reference holds no vectors for these either, so each is
checked against an independent numpy formulation (axis operations and slicing,
never the oracle's flat pointer walks), against exactly representable data with
one right answer, and against hand-computed special cases.  numpy's float32
`add.accumulate` is a front-to-back running sum, which is what pins the
summation ORDER; expf/powf digits are taken from the already pinned unary and
binary oracle functions, so only the composition is under test here."""
import numpy as np
import pytest

import oracle
from tests.helpers import assert_bit_exact, bits, normal, uniform, with_specials

F = np.float32


def running_sum(a, axis, dtype):
    acc = np.add.accumulate(a.astype(dtype), axis=axis, dtype=dtype)
    return np.take(acc, -1, axis=axis)


# ------------------------------------------------------------------- axpy ---
def test_axpy_rows_closed_form():
    alpha, x, y = normal(1, (6, 5)), normal(2, (6, 5, 7, 3)), normal(3, (6, 5, 7, 3))
    want = y + alpha[:, :, None, None] * x  # two rounded numpy operations
    assert_bit_exact(oracle.axpy_op(alpha, x, y), want, "axpy")
    assert_bit_exact(oracle.axpy_op(alpha.reshape(6, 5, 1, 1), x, y), want, "axpy 4-d alpha")
    # a fused multiply-add would differ on some of these
    fused = (y.astype(np.float64) + alpha[:, :, None, None].astype(np.float64) * x).astype(F)
    assert (bits(fused) != bits(want)).any()


def test_axpy_op_checks():
    x = np.zeros((2, 3, 4, 4), F)
    with pytest.raises(oracle.OracleCheckError):
        oracle.axpy_op(np.zeros((2, 4), F), x, x)
    with pytest.raises(oracle.OracleCheckError):
        oracle.axpy_op(np.zeros((2, 3, 2, 1), F), x, x)
    with pytest.raises(oracle.OracleCheckError):
        oracle.axpy_op(np.zeros((2, 3), F), x, np.zeros((2, 3, 4, 5), F))


# ------------------------------------------------------------- batch norm ---
@pytest.mark.parametrize("scale", [None, 0.0, 1.0, 999.982])
def test_batch_norm_closed_form(scale):
    x = with_specials(normal(4, (3, 8, 5, 5), 3.0), 4).reshape(3, 8, 5, 5)
    mean, var = normal(5, 8), uniform(6, 8, -0.5, 4.0)  # negative variances exercise the abs
    eps = F(1e-5)
    sf = F(1) if scale is None else (F(0) if scale == 0 else F(1) / F(scale))
    with np.errstate(all="ignore"):
        m = (mean * sf)[None, :, None, None]
        d = np.sqrt(np.abs(var * sf) + eps)[None, :, None, None]
        want = (x - m) / d
    got = oracle.batch_norm_op(x, mean, var, None if scale is None else F([scale]), eps=1e-5)
    assert_bit_exact(got, want, "batch_norm")


def test_batch_norm_known_values_and_checks():
    # (x - 1) / sqrt(4 + 0) with eps = 0: exact halves
    got = oracle.batch_norm_op(F([[[[1, 3, 5]]]]), F([1]), F([4]), eps=0.0)
    assert got.ravel().tolist() == [0.0, 1.0, 2.0]
    with pytest.raises(oracle.OracleCheckError):
        oracle.batch_norm_op(np.zeros((1, 2, 2, 2), F), F([0]), F([1, 1]))
    with pytest.raises(oracle.OracleCheckError):
        oracle.batch_norm_op(np.zeros((1, 2, 2, 2), F), F([0, 0]), F([1, 1]), scale=F([1, 2]))


# ---------------------------------------------------------------- softmax ---
def softmax_numpy(x, axis):
    mx = np.max(x, axis=axis, keepdims=True)
    e = oracle.unary(4, (x - mx).ravel()).reshape(x.shape)  # host expf, pinned elsewhere
    s = np.expand_dims(running_sum(e, axis, F), axis)
    return e / s


@pytest.mark.parametrize("shape,axis", [((4, 10), 1), ((3, 5, 7, 2), 1), ((2, 6, 9), 2), ((5, 3, 4), 0),
                                        ((2, 1000), -1), ((2, 21, 17, 19), 1)])
def test_softmax_against_axis_formulation(shape, axis):
    x = normal(7, shape, 4.0)
    assert_bit_exact(oracle.softmax_op(x, axis), softmax_numpy(x, axis % len(shape)), "softmax")


def test_softmax_sum_is_front_to_back_fp32():
    # Terms chosen so that fp32 running sums in other orders (or in fp64) differ.
    x = np.log(np.array([[1.0, 2.0 ** -24, 2.0 ** -24, 2.0 ** -24, 2.0 ** -24]])).astype(F)
    out = oracle.softmax_op(x, 1)
    # front to back: 1 + 2^-24 rounds back to 1 every time, so the sum stays 1
    assert out[0, 0] == F(1.0)
    y = x[:, ::-1].copy()  # back to front the small terms add up first
    out_r = oracle.softmax_op(y, 1)
    assert out_r[0, -1] < F(1.0)


def test_softmax_known_values():
    assert_bit_exact(oracle.softmax_op(np.full((2, 8), 3.25, F)), np.full((2, 8), 0.125, F), "uniform")
    assert_bit_exact(oracle.softmax_op(F([[5.0]]), 1), F([[1.0]]), "single")
    out = oracle.softmax_op(F([[0.0, -np.inf, 0.0]]))
    assert out.ravel().tolist() == [0.5, 0.0, 0.5]
    # any NaN poisons its column; a column of -inf keeps the finite identity and ends 0/0
    assert np.isnan(oracle.softmax_op(F([[np.nan, 1, 2], [1, 2, np.nan]]))).all()
    assert np.isnan(oracle.softmax_op(F([[-np.inf, -np.inf]]))).all()
    # shift by a power of two keeps x - max exact
    x = normal(8, (3, 40))
    x = np.round(x * 64) / 64
    assert_bit_exact(oracle.softmax_op(x + F(8)), oracle.softmax_op(x), "shift invariance")


# -------------------------------------------------------------- normalize ---
def normalize_numpy(x, p, axis, eps):
    a = np.abs(x)
    if p == 1:
        val = running_sum(a, axis, np.float64).astype(F)
    elif p == 2:
        val = np.sqrt(running_sum(a * a, axis, np.float64).astype(F))  # fp32 squares
    else:
        t = oracle.binary_scalar(4, a.ravel(), p).reshape(x.shape)  # host powf
        s = running_sum(t, axis, np.float64).astype(F)
        val = oracle.binary_scalar(4, s.ravel(), F(1) / F(p)).reshape(s.shape)
    val = np.where(val < F(eps), F(eps), val)
    return x / np.expand_dims(val, axis)


@pytest.mark.parametrize("p", [1.0, 2.0, 3.0, 0.5])
@pytest.mark.parametrize("shape,axis", [((6, 128), 1), ((2, 16, 5, 5), 1), ((3, 4, 50), -1), ((7, 3), 0)])
def test_normalize_against_axis_formulation(p, shape, axis):
    x = normal(9, shape, 2.0)
    got = oracle.normalize_op(x, p, axis, 1e-12)
    assert_bit_exact(got, normalize_numpy(x, p, axis % len(shape), 1e-12), "normalize p=%g" % p)


def test_normalize_known_values():
    q = F(3) / F(5), F(4) / F(5)
    assert oracle.normalize_op(F([[3, 4]]), 2, 1).ravel().tolist() == [q[0], q[1]]
    assert oracle.normalize_op(F([[3, -4, 1]]), 1, 1).ravel().tolist() == [F(3) / F(8), F(-4) / F(8), F(1) / F(8)]
    # zero column: 0 / eps
    assert oracle.normalize_op(np.zeros((1, 4), F), 2, 1).ravel().tolist() == [0.0] * 4
    # eps takes over when the norm is below it
    out = oracle.normalize_op(F([[1e-3, 0]]), 2, 1, eps=1.0)
    assert out.ravel().tolist() == [F(1e-3), 0.0]
    # the square is taken in fp32: 1e-30^2 underflows to 0 there, not in fp64
    with np.errstate(all="ignore"):
        assert np.isinf(oracle.normalize_op(F([[1e-30]]), 2, 1, eps=0.0)).all()
    out = oracle.normalize_op(F([[1e-30, 1e-30]]), 2, 1, eps=1e-12)
    assert out.ravel().tolist() == [F(1e-30) / F(1e-12)] * 2


# ----------------------------------------------------------- SSDNormalize ---
def ssd_numpy(x, scale, across_spatial, channel_shared, eps):
    """Array formulation with numpy's own rounded operations."""
    eps = F(eps)
    sq = x * x  # fp32 squares
    if across_spatial:
        flat = sq.reshape(x.shape[0], -1)
        total = running_sum(flat, 1, np.float64).astype(F)        # Sasum: fp64 fold, fp32 result
        factor = F(1) / np.sqrt(total + eps, dtype=F)             # fp32 add, sqrt, divide
        out = x * factor.reshape((-1,) + (1,) * (x.ndim - 1))
    else:
        total = running_sum(sq, 1, np.float64)                    # stays fp64
        val = np.sqrt(total + np.float64(eps)).astype(F)          # fp64 add and sqrt
        out = x / np.expand_dims(val, 1)
    if scale is not None:
        sc = scale.ravel()
        out = out * sc[0] if channel_shared else out * sc[:x.shape[1]].reshape((1, -1) + (1,) * (x.ndim - 2))
    return out.astype(F)


@pytest.mark.parametrize("across", [False, True])
@pytest.mark.parametrize("scale_kind", ["none", "shared", "channel"])
@pytest.mark.parametrize("shape", [(2, 5, 3, 4), (3, 7, 1, 1), (1, 33, 6, 2), (2, 3, 9)])
def test_ssd_normalize_against_array_formulation(across, scale_kind, shape):
    x = normal(40, shape, 3.0)
    scale = {"none": None, "shared": F([20.0]), "channel": normal(41, (shape[1],)) + F(20)}[scale_kind]
    got = oracle.ssd_normalize_op(x, scale, across, scale_kind != "channel", 1e-5)
    assert_bit_exact(got, ssd_numpy(x, scale, across, scale_kind != "channel", 1e-5), "ssd %s" % scale_kind)


def test_ssd_normalize_known_values():
    # per position: four equal channels, 1.5 / sqrt(4 * 2.25) = 0.5 exactly
    x = np.full((1, 4, 2, 2), 1.5, F)
    assert (oracle.ssd_normalize_op(x, None, False, True, 0.0) == F(0.5)).all()
    # per item: 16 values of 1.5, 1 / sqrt(36) rounded, times 1.5, times the shared scale
    want = F(1.5) * (F(1) / np.sqrt(F(36), dtype=F)) * F(20)
    assert (oracle.ssd_normalize_op(x, F([20]), True, True, 0.0) == want).all()
    # eps sits inside the square root, not under a max: a zero item gives 0 * (1 / sqrt(eps))
    z = np.zeros((1, 2, 2, 2), F)
    assert (oracle.ssd_normalize_op(z, None, True, True, 1e-5) == 0).all()
    assert (oracle.ssd_normalize_op(z, None, False, True, 1e-5) == 0).all()
    with np.errstate(all="ignore"):
        assert np.isnan(oracle.ssd_normalize_op(z, None, False, True, 0.0)).all()  # 0 / 0
    # the per-position root is taken in fp64 and rounded once: an fp32 root of the fp32
    # sum is a different number for some columns
    x = normal(42, (1, 16, 64, 64), 2.0)
    got = oracle.ssd_normalize_op(x, None, False, True, 1e-5)
    sq = x * x
    total32 = running_sum(sq, 1, np.float64).astype(F)
    other = x / np.expand_dims(np.sqrt(total32 + F(1e-5), dtype=F), 1)
    assert (got.view(np.uint32) != other.view(np.uint32)).any()
    # both arguments default to true in the operator (ssd_normalize_op.cpp:11-12)
    assert_bit_exact(oracle.ssd_normalize_op(x, F([3])), oracle.ssd_normalize_op(x, F([3]), True, True, 1e-5), "defaults")


def test_ssd_normalize_unit_norm_and_scale_checks():
    x = normal(43, (3, 8, 5, 5), 4.0)
    per_item = oracle.ssd_normalize_op(x, None, True, True, 0.0).astype(np.float64)
    np.testing.assert_allclose((per_item ** 2).reshape(3, -1).sum(1), 1.0, rtol=1e-5)
    per_pos = oracle.ssd_normalize_op(x, None, False, True, 0.0).astype(np.float64)
    np.testing.assert_allclose((per_pos ** 2).sum(1), 1.0, rtol=1e-5)
    with pytest.raises(oracle.OracleCheckError):
        oracle.ssd_normalize_op(x, F([1, 2]), True, True)   # shared scale holds one value
    with pytest.raises(oracle.OracleCheckError):
        oracle.ssd_normalize_op(x, F([1, 2]), True, False)  # fewer values than channels


# ---------------------------------------------------------------- pooling ---
def pooling_numpy(x, pool, kernel, stride, pad, out_shape):
    """Window by slicing; running fp32 sum over the flattened window."""
    nsp = len(kernel)
    out = np.empty(out_shape, F)
    for idx in np.ndindex(*out_shape[2:]):
        lo = [i * s - p for i, s, p in zip(idx, stride, pad)]
        hi = [min(l + k, d + p) for l, k, d, p in zip(lo, kernel, x.shape[2:], pad)]
        size = int(np.prod([h - l for h, l in zip(hi, lo)]))
        sl = tuple(slice(max(l, 0), min(h, d)) for l, h, d in zip(lo, hi, x.shape[2:]))
        win = x[(slice(None), slice(None)) + sl].reshape(x.shape[0], x.shape[1], -1)
        if pool == 0:
            m = np.full(win.shape[:2], np.finfo(F).min, F)
            for j in range(win.shape[2]):
                m = np.where(m < win[:, :, j], win[:, :, j], m)
            res = m
        else:
            s = np.zeros(win.shape[:2], F)
            for j in range(win.shape[2]):
                s = s + win[:, :, j]
            with np.errstate(all="ignore"):
                res = s / F(size)
        out[(slice(None), slice(None)) + idx] = res
    return out


CASES_2D = [
    ((2, 3, 12, 12), [3], [2], [0], True), ((2, 3, 12, 12), [3], [2], [1], True),
    ((2, 3, 12, 12), [3], [2], [1], False), ((1, 2, 7, 9), [2, 3], [2, 1], [1, 0], True),
    ((2, 4, 7, 7), [7], [1], [0], True), ((1, 1, 5, 5), [5], [3], [2], True),
    ((3, 2, 8, 8), [2], [2], [0], False), ((1, 2, 6, 6), [3], [3], [2], True),
]


@pytest.mark.parametrize("pool", [0, 1])
@pytest.mark.parametrize("shape,kernel,stride,pad,full", CASES_2D)
def test_pooling2d_against_slicing(pool, shape, kernel, stride, pad, full):
    x = normal(10, shape, 2.0)
    got = oracle.pooling_op(x, pool, kernel, stride, pad, full_pooling=full)
    k, s, p = [v * 2 if len(v) == 1 else v for v in (kernel, stride, pad)]
    assert_bit_exact(got, pooling_numpy(x, pool, k, s, p, got.shape), "pool2d")


@pytest.mark.parametrize("pool", [0, 1])
@pytest.mark.parametrize("shape,kernel,stride,pad", [((2, 2, 6, 7, 8), [3], [2], [1]),
                                                     ((1, 3, 4, 5, 5), [2, 3, 2], [1, 2, 2], [0, 1, 1]),
                                                     ((2, 2, 3, 4, 4), [3, 4, 4], [1], [0])])
def test_pooling3d_against_slicing(pool, shape, kernel, stride, pad):
    x = normal(11, shape, 2.0)
    got = oracle.pooling_op(x, pool, kernel, stride, pad)
    k, s, p = [v * 3 if len(v) == 1 else v for v in (kernel, stride, pad)]
    assert_bit_exact(got, pooling_numpy(x, pool, k, s, p, got.shape), "pool3d")


def test_pooling_known_values():
    x = np.arange(25, dtype=F).reshape(1, 1, 5, 5)
    # 3x3 stride 2, no pad: maxima are the window corners, means the centres
    assert oracle.pooling_op(x, 0, [3], [2], [0]).ravel().tolist() == [12, 14, 22, 24]
    assert oracle.pooling_op(x, 1, [3], [2], [0]).ravel().tolist() == [6, 8, 16, 18]
    # global pooling ignores kernel/stride/pad arguments
    assert oracle.pooling_op(x, 1, [2], [5], [3], global_pooling=True).ravel().tolist() == [12]
    assert oracle.pooling_op(x, 0, global_pooling=True).shape == (1, 1, 1, 1)
    # the average divides by the window clipped to input + pad, not to the input:
    # top-left 2x2 window with pad 1 holds one real value but counts 4 cells
    got = oracle.pooling_op(np.full((1, 1, 2, 2), 8, F), 1, [2], [2], [1], full_pooling=False)
    assert got.ravel().tolist() == [2.0, 2.0, 2.0, 2.0]
    # max ignores NaN (NaN never compares greater) and starts from the finite identity
    assert oracle.pooling_op(F([[[[np.nan, 1], [2, np.nan]]]]), 0, [2], [2], [0]).ravel().tolist() == [2.0]
    assert bits(oracle.pooling_op(F([[[[-np.inf] * 2] * 2]]), 0, [2], [2], [0]))[0, 0, 0, 0] == 0xff7fffff
    # first zero wins the sign
    assert bits(oracle.pooling_op(F([[[[-0.0, 0.0], [0.0, 0.0]]]]), 0, [2], [2], [0])).ravel()[0] == 0x80000000


def test_pooling_out_size_formula():
    # ceil / floor of an fp32 quotient, plus one; no clipping of the last window
    assert oracle.pooling_out_size(112, 3, 2, 0, True) == 56
    assert oracle.pooling_out_size(112, 3, 2, 0, False) == 55
    assert oracle.pooling_out_size(112, 3, 2, 1, True) == 57
    assert oracle.pooling_out_size(112, 3, 2, 1, False) == 56
    assert oracle.pooling_out_size(7, 7, 1, 0, True) == 1
    assert oracle.pooling_out_size(5, 2, 2, 0, True) == 3
    assert oracle.pooling_out_size(5, 2, 2, 0, False) == 2


def test_pooling_op_checks():
    with pytest.raises(oracle.OracleCheckError):
        oracle.pooling_op(np.zeros((2, 3, 4), F), 0, [2])
    with pytest.raises(oracle.OracleCheckError):
        oracle.pooling_op(np.zeros((2, 3, 4, 4), F), 2, [2])
    with pytest.raises(oracle.OracleCheckError):
        oracle.pooling_op(np.zeros((2, 3, 4, 4), F), 0, [2, 2, 2])


# --------------------------------------------------- group / instance / layer norm ---
def normalize_rows_numpy(x2, eps):
    """x2: [outer, inner].  fp32 products, fp64 front-to-back sums, one rounding each."""
    alpha = F(1) / F(x2.shape[1])
    mean = running_sum(alpha * x2, 1, np.float64).astype(F)
    val = x2 - mean[:, None]
    var = running_sum(alpha * (val * val), 1, np.float64).astype(F)
    return val / np.sqrt(var + F(eps))[:, None]


@pytest.mark.parametrize("shape,group", [((2, 8, 5, 5), 1), ((2, 8, 5, 5), 4), ((3, 6, 7, 3), 6), ((1, 4, 1, 1), 2)])
def test_group_norm_against_axis_formulation(shape, group):
    x = normal(30, shape, 3.0) + F(1.5)
    want = normalize_rows_numpy(x.reshape(shape[0] * group, -1), 1e-5).reshape(shape)
    assert_bit_exact(oracle.group_norm_op(x, group), want, "group norm")
    scale, bias = uniform(31, shape[1], 0.5, 2.0), normal(32, shape[1])
    want_affine = want * scale[None, :, None, None] + bias[None, :, None, None]
    assert_bit_exact(oracle.group_norm_op(x, group, scale=scale, bias=bias), want_affine, "group norm affine")
    if group == shape[1]:
        assert_bit_exact(oracle.instance_norm_op(x, scale=scale, bias=bias), want_affine, "instance norm")


@pytest.mark.parametrize("shape,ns", [((4, 10, 32), [32]), ((2, 3, 6, 5), [6, 5]), ((5, 7), [7]), ((2, 3, 4), [3, 4])])
def test_layer_norm_against_axis_formulation(shape, ns):
    x = normal(33, shape, 2.0)
    inner = int(np.prod(ns))
    want = normalize_rows_numpy(x.reshape(-1, inner), 1e-5).reshape(shape)
    assert_bit_exact(oracle.layer_norm_op(x, ns), want, "layer norm")
    scale, bias = uniform(34, ns, 0.5, 2.0), normal(35, ns)
    assert_bit_exact(oracle.layer_norm_op(x, ns, scale=scale, bias=bias), want * scale + bias, "layer norm affine")


def test_norm_known_values_and_checks():
    # mean 2, deviations -1/+1, variance 1, eps 0
    assert oracle.layer_norm_op(F([[1, 3]]), [2], eps=0.0).ravel().tolist() == [-1.0, 1.0]
    # constant row: 0 / sqrt(eps)
    assert oracle.group_norm_op(np.full((1, 2, 2, 2), 7, F), 1).ravel().tolist() == [0.0] * 8
    # the 1/inner factor is applied per element in fp32, before the fp64 sum:
    # 3 * fl(fl(1/3) * 1) = 1.0000000298 in fp64, which rounds to 1 in fp32
    assert oracle.layer_norm_op(F([[1, 1, 1]]), [3], eps=1.0).ravel().tolist() == [0.0] * 3
    big = F([[16777216.0, 1.0, 1.0, 1.0]])  # an fp32 running sum would drop the ones
    m = running_sum(F(0.25) * big, 1, np.float64).astype(F)
    assert m[0] == F(4194304.75)
    assert_bit_exact(oracle.layer_norm_op(big, [4]), normalize_rows_numpy(big, 1e-5), "fp64 accumulate")
    with pytest.raises(oracle.OracleCheckError):
        oracle.group_norm_op(np.zeros((1, 6, 2, 2), F), 4)
    with pytest.raises(oracle.OracleCheckError):
        oracle.group_norm_op(np.zeros((1, 6, 2, 2), F), 3, scale=np.ones(5, F), bias=np.ones(6, F))
    with pytest.raises(oracle.OracleCheckError):
        oracle.layer_norm_op(np.zeros((2, 3, 4), F), [4, 3])
    with pytest.raises(oracle.OracleCheckError):
        oracle.layer_norm_op(np.zeros((2, 3, 4), F), [])
    with pytest.raises(oracle.OracleCheckError):
        oracle.layer_norm_op(np.zeros((2, 3, 4), F), [4], scale=np.ones(4, F))


# -------------------------------------------------------------------- lrn ---
def lrn_by_planes(x, size, alpha, beta, k):
    """The channel walk on whole [batch, h, w] planes at once: every step is one rounded fp32 numpy
    operation, entering square added before the leaving one is subtracted."""
    x = x.astype(F)
    c_in, post = x.shape[1], (size - 1) // 2
    sq = x * x
    aos = F(alpha) / F(size)
    accum = np.zeros(x[:, 0].shape, F)
    scale = np.empty_like(x)
    for head in range(c_in + post):
        if head < c_in:
            accum = accum + sq[:, head]
        if head >= size:
            accum = accum - sq[:, head - size]
        if head >= post:
            scale[:, head - post] = F(k) + accum * aos
    power = oracle.binary(4, scale, np.full(scale.shape, -F(beta), F)).reshape(x.shape)  # the pinned powf
    return x * power, scale


@pytest.mark.parametrize("shape,size", [((2, 7, 3, 5), 5), ((1, 2, 4, 4), 5), ((3, 16, 1, 1), 3), ((2, 6, 2, 3), 1),
                                        ((2, 5, 2, 2), 9), ((1, 40, 3, 3), 11)])
@pytest.mark.parametrize("alpha,beta,k", [(1e-4, 0.75, 1.0), (1.0, 0.75, 1.0), (0.5, 2.0, 2.0)])
def test_lrn_against_plane_formulation(shape, size, alpha, beta, k):
    x = normal(61, shape, 3.0)
    want, want_scale = lrn_by_planes(x, size, alpha, beta, k)
    got, scale = oracle.lrn(x, shape, size, alpha, beta, k)
    assert_bit_exact(scale.reshape(shape), want_scale, "lrn scale")
    assert_bit_exact(got.reshape(shape), want, "lrn")
    assert_bit_exact(oracle.lrn_op(x, size, alpha, beta, 0, k), want, "lrn op")


def test_lrn_sum_is_a_running_one():
    """The window sum formed afresh for every channel rounds differently from add-then-subtract."""
    shape, size = (4, 64, 5, 5), 5
    x = normal(62, shape, 3.0)
    _, scale = oracle.lrn(x, shape, size, 1.0, 0.75, 1.0)
    sq = (x * x).astype(F)
    fresh = np.empty_like(x)
    for c in range(shape[1]):
        lo, hi = max(0, c - 2), min(shape[1], c + 3)
        fresh[:, c] = F(1) + running_sum(sq[:, lo:hi], 1, F) * (F(1) / F(size))
    assert (bits(fresh) != bits(scale.reshape(shape))).any()
    assert np.allclose(fresh, scale.reshape(shape), rtol=1e-5)


def test_lrn_exact_data_and_known_values():
    # small integers and alpha / size a power of two: every operation is exact, one right answer
    shape, size = (2, 9, 3, 3), 5
    x = (np.arange(np.prod(shape)) % 7 - 3).astype(F).reshape(shape)
    _, scale = oracle.lrn(x, shape, size, 5 * 2.0 ** -3, 0.75, 1.0)
    sq = x.astype(np.float64) ** 2
    want = np.empty(shape)
    for c in range(shape[1]):
        want[:, c] = 1.0 + sq[:, max(0, c - 2):c + 3].sum(1) * 2.0 ** -3
    assert_bit_exact(scale.reshape(shape), want.astype(F), "exact scale")
    # two channels of ones, window 3, alpha / size = 1, k = 2: both scales are 4
    ones = np.ones((1, 2, 1, 1), F)
    assert_bit_exact(oracle.lrn_op(ones, 3, 3.0, 1.0, 0, 2.0), np.full((1, 2, 1, 1), 0.25, F), "4^-1")
    assert_bit_exact(oracle.lrn_op(ones, 3, 3.0, 0.5, 0, 2.0), np.full((1, 2, 1, 1), 0.5, F), "4^-1/2")
    x = normal(63, (2, 4, 3, 3))
    assert_bit_exact(oracle.lrn_op(x, 3, 1.0, 0.0, 0, 1.0), x, "beta 0")
    # a window of one channel: scale = k + x^2 * alpha in the first channel; further on the sum is
    # (previous + entering) - previous, which need not be the entering square again
    got, scale = oracle.lrn(x, x.shape, 1, 0.5, 0.75, 1.0)
    assert_bit_exact(scale.reshape(x.shape)[:, 0], F(1) + (x * x)[:, 0] * F(0.5), "window of one")


def test_lrn_op_checks():
    x = np.zeros((2, 3, 4, 4), F)
    with pytest.raises(oracle.OracleCheckError):
        oracle.lrn_op(x, 4)
    with pytest.raises(oracle.OracleCheckError):
        oracle.lrn_op(x, 5, norm_region=1)
    with pytest.raises(oracle.OracleCheckError):
        oracle.lrn_op(np.zeros((2, 3, 4), F), 5)
    with pytest.raises(oracle.OracleCheckError):
        oracle.lrn_op(x, 9)  # three channels, four behind the centre
    oracle.lrn_op(x, 7)


# ------------------------------------------------------------ grid sample ---
def grid_sample_by_arrays(x, grid, mode, padding_mode):
    """Whole-array numpy: coordinates, masks, gathers with take_along_axis-free fancy indexing and the
    reference's order of float32 operations; finite coordinates that fit an int."""
    x, grid = x.astype(F), grid.astype(F)
    b, c, in_h, in_w = x.shape
    gx, gy = grid[..., 0], grid[..., 1]                      # [b, out_h, out_w]
    fh = (gy + F(1)) / F(2) * F(in_h - 1)
    fw = (gx + F(1)) / F(2) * F(in_w - 1)
    bi = np.arange(b)[:, None, None, None]
    ci = np.arange(c)[None, :, None, None]
    if mode == 0:
        away = lambda v: np.where(v >= 0, np.floor(v + F(0.5)), np.ceil(v - F(0.5)))  # half away from zero
        h, w = away(fh.astype(np.float64)).astype(np.int64), away(fw.astype(np.float64)).astype(np.int64)
        outside = (h < 0) | (w < 0) | (h > in_h - 1) | (w > in_w - 1)
        h, w = np.clip(h, 0, in_h - 1), np.clip(w, 0, in_w - 1)
        out = x[bi, ci, h[:, None], w[:, None]]
        return np.where(outside[:, None] & (padding_mode == 0), F(0), out).astype(F)
    outside = (fh < 0) | (fw < 0) | (fh > in_h - 1) | (fw > in_w - 1)
    if padding_mode == 1:
        fh, fw = np.clip(fh, F(0), F(in_h - 1)), np.clip(fw, F(0), F(in_w - 1))
    safe_h, safe_w = np.clip(fh, 0, in_h - 1), np.clip(fw, 0, in_w - 1)  # masked out below where it matters
    h0, h1 = np.floor(safe_h).astype(np.int64), np.ceil(safe_h).astype(np.int64)
    w0, w1 = np.floor(safe_w).astype(np.int64), np.ceil(safe_w).astype(np.int64)
    sh, sw = (safe_h - h0.astype(F))[:, None], (safe_w - w0.astype(F))[:, None]
    pick = lambda hh, ww: x[bi, ci, hh[:, None], ww[:, None]]
    one = F(1)
    out = ((one - sh) * (one - sw) * pick(h0, w0) + sh * (one - sw) * pick(h1, w0) + (one - sh) * sw * pick(h0, w1)
           + sh * sw * pick(h1, w1))
    if padding_mode == 0:
        out = np.where(outside[:, None], F(0), out)
    return out.astype(F)


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("padding_mode", [0, 1])
@pytest.mark.parametrize("shape,out_hw", [((2, 3, 5, 7), (4, 6)), ((1, 2, 1, 9), (3, 3)), ((3, 1, 8, 1), (2, 5)),
                                          ((2, 4, 6, 6), (11, 13))])
def test_grid_sample_against_array_formulation(mode, padding_mode, shape, out_hw):
    x = normal(71, shape, 2.0)
    grid = uniform(72, (shape[0],) + out_hw + (2,), -1.3, 1.3)  # a fifth of the coordinates outside the input
    want = grid_sample_by_arrays(x, grid, mode, padding_mode)
    assert_bit_exact(oracle.grid_sample_op(x, grid, mode, padding_mode), want, "grid sample")


def test_grid_sample_known_values():
    x = np.arange(15, dtype=F).reshape(1, 1, 5, 3)  # extents whose cell centres are exact coordinates
    gy, gx = np.meshgrid(np.linspace(-1, 1, 5), np.linspace(-1, 1, 3), indexing="ij")
    centres = np.stack([gx, gy], -1).astype(F)[None]
    for mode in (0, 1):
        assert_bit_exact(oracle.grid_sample_op(x, centres, mode, 0), x, "the grid of the cell centres gives the input back")
    # half way between cells 0 and 1 of the first row, and between rows 0 and 1 of the first column
    mid = np.array([[[[-0.5, -1.0], [-1.0, -0.75]]]], F)
    assert_bit_exact(oracle.grid_sample_op(x, mid, 1, 0), F([[[[0.5, 1.5]]]]), "averages")
    # outside: zeros, or the border cell
    far = np.array([[[[-2.0, -1.0], [3.0, 1.0], [0.0, 40.0]]]], F)
    assert_bit_exact(oracle.grid_sample_op(x, far, 1, 0), np.zeros((1, 1, 1, 3), F), "zeros outside")
    assert_bit_exact(oracle.grid_sample_op(x, far, 0, 0), np.zeros((1, 1, 1, 3), F), "zeros outside, nearest")
    assert_bit_exact(oracle.grid_sample_op(x, far, 0, 1), F([[[[0, 14, 13]]]]), "border, nearest")
    assert_bit_exact(oracle.grid_sample_op(x, far, 1, 1), F([[[[0, 14, 13]]]]), "border, bilinear")
    # a tie goes away from zero: coordinate 0.5 of a row of two is cell 1
    two = F([[[[5, 7]]]])
    assert_bit_exact(oracle.grid_sample_op(two, F([[[[0.0, 0.0]]]]), 0, 0), F([[[[7]]]]), "round half away from zero")


def test_grid_sample_coordinates_that_fit_no_int_and_checks():
    x = np.arange(6, dtype=F).reshape(1, 1, 2, 3)
    huge = np.array([[[[1e30, 0.0], [-1e30, 0.0], [np.inf, -1.0], [np.nan, 1.0]]]], F)
    # nearest: the conversion of the reference's x86-64 build gives INT_MIN: zero, or clamped to cell 0
    assert_bit_exact(oracle.grid_sample_op(x, huge, 0, 0), np.zeros((1, 1, 1, 4), F), "nearest, zeros")
    assert_bit_exact(oracle.grid_sample_op(x, huge, 0, 1), F([[[[3, 3, 0, 3]]]]), "nearest, border")
    # bilinear: clamped or rejected before any conversion; a NaN coordinate gives NaN
    got = oracle.grid_sample_op(x, huge, 1, 1).ravel()
    assert_bit_exact(got[:3], F([3.5, 1.5, 2]), "bilinear, border")  # rows 0 and 1 half and half in the border column
    assert np.isnan(got[3])
    got = oracle.grid_sample_op(x, huge, 1, 0).ravel()
    assert_bit_exact(got[:3], F([0, 0, 0]), "bilinear, zeros")
    assert np.isnan(got[3])
    grid = np.zeros((1, 2, 2, 2), F)
    for bad in (dict(mode=2), dict(padding_mode=2)):
        with pytest.raises(oracle.OracleCheckError):
            oracle.grid_sample_op(x, grid, **bad)
    with pytest.raises(oracle.OracleCheckError):
        oracle.grid_sample_op(x, np.zeros((2, 2, 2, 2), F))
    with pytest.raises(oracle.OracleCheckError):
        oracle.grid_sample_op(x, np.zeros((1, 2, 2, 3), F))
