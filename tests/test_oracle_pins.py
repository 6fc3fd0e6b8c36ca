"""Pins for the CPU oracle (oracle/shadow_cpu.c + oracle/__init__.py).

The reference has no tests or golden vectors for this path, and its own build
needs a cmake-generated header, so the oracle is pinned by:
  * IEEE closed forms evaluated independently with numpy float32 arithmetic
    (numpy never fuses multiply-add across ufunc calls);
  * brute-force N-d broadcast / reduce written with numpy indexing, not with the
    oracle's flat-index arithmetic;
  * exactly representable data where an fp64 sum has one right answer;
  * the special-value behaviour observed on the compiled reference when the
    path was surveyed (signed zeros, NaN, identities leaking out of max/min);
  * libm-backed functions against an fp64 evaluation, within 1 ulp -- enough to
    catch a wrong function, sign or argument, which is what a restatement can
    get wrong (the digits themselves are the host libm's, as in the reference).
"""
import itertools
import math

import numpy as np
import pytest

import oracle
from tests.helpers import (assert_bit_exact, bits, normal, ulp_distance, uniform, with_specials)

F = np.float32


def sel_max(a, b):
    return np.where(a < b, b, a)


def sel_min(a, b):
    return np.where(b < a, b, a)


# ------------------------------------------------------------------ unary ---
def test_unary_closed_forms():
    x = with_specials(normal(1, 5000, 2.0), 1)
    with np.errstate(all="ignore"):
        assert_bit_exact(oracle.unary(0, x), np.abs(x), "abs")
        assert_bit_exact(oracle.unary(1, x), x * x, "square")
        assert_bit_exact(oracle.unary(2, x), np.sqrt(x), "sqrt")
        assert_bit_exact(oracle.unary(11, x), np.floor(x), "floor")
        assert_bit_exact(oracle.unary(12, x), np.ceil(x), "ceil")
        assert_bit_exact(oracle.unary(13, x), -x, "neg")
        assert_bit_exact(oracle.unary(14, x), F(1) / x, "reciprocal")


@pytest.mark.parametrize("op,fn,lo,hi", [
    (3, np.log, 1e-3, 50.0), (4, np.exp, -20.0, 20.0), (5, np.sin, -6.0, 6.0),
    (6, np.cos, -6.0, 6.0), (7, np.tan, -1.5, 1.5), (8, np.arcsin, -1.0, 1.0),
    (9, np.arccos, -1.0, 1.0), (10, np.arctan, -50.0, 50.0)])
def test_unary_libm_against_fp64(op, fn, lo, hi):
    x = uniform(2 + op, 20000, lo, hi)
    want = fn(x.astype(np.float64)).astype(F)
    assert ulp_distance(oracle.unary(op, x), want).max() <= 1


def test_unary_rejects_unknown_operation():
    with pytest.raises(oracle.OracleCheckError):
        oracle.unary_op(np.zeros(4, F), 15)
    with pytest.raises(oracle.OracleCheckError):
        oracle.unary_op(np.zeros(4, F), -1)


# ----------------------------------------------------------------- binary ---
def test_binary_closed_forms():
    a = with_specials(normal(10, 4000), 2)
    b = with_specials(uniform(11, 4000, 0.5, 2.0), 3)
    with np.errstate(all="ignore"):
        expect = {0: a + b, 1: a - b, 2: a * b, 3: a / b, 5: sel_max(a, b), 6: sel_min(a, b)}
        for op, want in expect.items():
            assert_bit_exact(oracle.binary(op, a, b), want, "binary %d" % op)
            assert_bit_exact(oracle.binary_scalar(op, a, 1.5),
                             {0: a + F(1.5), 1: a - F(1.5), 2: a * F(1.5), 3: a / F(1.5),
                              5: sel_max(a, F(1.5)), 6: sel_min(a, F(1.5))}[op], "scalar %d" % op)
    p = oracle.binary(4, uniform(12, 3000, 0.1, 4.0), uniform(13, 3000, -3, 3))
    q = np.power(uniform(12, 3000, 0.1, 4.0).astype(np.float64), uniform(13, 3000, -3, 3).astype(np.float64))
    assert ulp_distance(p, q.astype(F)).max() <= 1


def test_max_min_reference_observations():
    """(+0,-0) -> +0, (-0,+0) -> -0, (NaN,1) -> NaN, (1,NaN) -> 1 for both max and min."""
    a = F([0.0, -0.0, np.nan, 1.0])
    b = F([-0.0, 0.0, 1.0, np.nan])
    for op in (5, 6):
        got = oracle.binary(op, a, b)
        assert bits(got)[0] == 0x00000000 and bits(got)[1] == 0x80000000
        assert np.isnan(got[2]) and got[3] == 1.0


@pytest.mark.parametrize("sa,sb", [([2, 1], [3]), ([8, 6, 5, 4], [1, 6, 1, 1]), ([4, 1, 3, 5], [1, 7, 3, 1]),
                                   ([2, 3, 1, 4], [3, 4]), ([6, 5], [1]), ([1, 1, 2], [3, 2, 1])])
@pytest.mark.parametrize("op", [0, 1, 2, 3, 5, 6])
def test_broadcast_against_numpy(sa, sb, op):
    a, b = normal(20, sa), uniform(21, sb, 0.5, 2.0)
    A, B = np.broadcast_arrays(a, b)
    want = {0: A + B, 1: A - B, 2: A * B, 3: A / B, 5: sel_max(A, B), 6: sel_min(A, B)}[op]
    got = oracle.binary_op(a, b, operation=op)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "broadcast")


def test_binary_op_shape_errors_and_scalar_form():
    with pytest.raises(oracle.OracleCheckError):
        oracle.binary_op(np.zeros((2, 3), F), np.zeros((2,), F), operation=0)
    with pytest.raises(oracle.OracleCheckError):
        oracle.binary_op(np.zeros((2, 3), F), np.zeros((2, 3), F), operation=7)
    x = normal(22, (3, 4))
    assert_bit_exact(oracle.binary_op(x, operation=1, scalar=0.25), x - F(0.25), "scalar form")
    # observed on the reference: [2,1] - [3] -> [2,3], bottom[0] - bottom[1]
    got = oracle.binary_op(F([[1], [2]]), F([1, 2, 3]), operation=1)
    assert_bit_exact(got, F([[0, -1, -2], [1, 0, -1]]), "sub broadcast")


# --------------------------------------------------------------- activate ---
def test_activate_closed_forms():
    x = with_specials(normal(30, 6000, 2.5), 4)
    with np.errstate(all="ignore"):
        assert_bit_exact(oracle.activate(x, 1), np.where(x > 0, x, F(0)), "relu")
        assert_bit_exact(oracle.activate(x, 2, 0.1), np.where(x > 0, x, F(0.1) * x), "leaky")
        assert_bit_exact(oracle.activate(x, 6), np.where(x < 0, F(0), np.where(x > 6, F(6), x)), "relu6")
        hs = np.where(x < -3, F(0), np.where(x > 3, x, (x * (x + F(3))) / F(6)))
        assert_bit_exact(oracle.activate(x, 7), hs, "hardswish")
        # sigmoid is fp32 arithmetic around the oracle's own expf
        e = oracle.unary(4, -x)
        assert_bit_exact(oracle.activate(x, 3), F(1) / (F(1) + e), "sigmoid composition")


def test_activate_libm_against_fp64():
    x = uniform(31, 20000, -9.0, 9.0)
    xd = x.astype(np.float64)
    assert ulp_distance(oracle.activate(x, 5), np.tanh(xd).astype(F)).max() <= 2  # fdlibm tanhf: < 2 ulp
    assert ulp_distance(oracle.activate(x, 3), (1 / (1 + np.exp(-xd))).astype(F)).max() <= 2
    assert ulp_distance(oracle.activate(x, 4), np.log1p(np.exp(xd)).astype(F)).max() <= 2
    erf = np.vectorize(math.erf)
    gelu = 0.5 * xd * (1 + erf(np.float64(F(0.707107)) * xd))
    # 1 + erf(.) cancels in the negative tail, so bound the absolute error
    assert np.abs(oracle.activate(x, 8).astype(np.float64) - gelu).max() <= 1e-6


def test_activate_reference_observations():
    got = oracle.activate(F([-0.0, np.nan, -np.inf, 1e-45]), 1)
    assert list(bits(got)) == [0, 0, 0, 1]  # relu: -0, NaN, -inf -> +0; denormal kept
    s = oracle.activate(F([-np.inf, np.inf, 0.0, -100.0, 100.0]), 3)
    assert_bit_exact(s, F([0.0, 1.0, 0.5, 0.0, 1.0]), "sigmoid limits")
    assert np.isnan(oracle.activate(F([np.nan]), 3)[0])


@pytest.mark.parametrize("shape,shared", [((2, 3, 4, 5), False), ((2, 3, 4, 5), True), ((3, 6), False)])
def test_prelu_against_numpy(shape, shared):
    x = normal(32, shape)
    slope = uniform(33, 1 if shared else shape[1], -0.5, 0.5)
    s = slope.reshape([1, -1] + [1] * (len(shape) - 2)) if not shared else slope[0]
    want = np.where(x > 0, x, x * s)
    assert_bit_exact(oracle.activate_op(x, 0, slope_blob=slope), want, "prelu")


# ------------------------------------------------------------------ scale ---
@pytest.mark.parametrize("shape,axis,pshape", [((2, 5, 3, 4), 1, (5,)), ((2, 5, 3, 4), 1, (5, 3)),
                                               ((4, 6), 1, (6,)), ((3, 4, 5), 0, (3,)), ((2, 3, 4), 2, (4,))])
def test_scale_blob_form_against_numpy(shape, axis, pshape):
    x = normal(40, shape)
    s, b = uniform(41, pshape, 0.5, 1.5), uniform(42, pshape, -0.1, 0.1)
    view = [1] * axis + list(pshape) + [1] * (len(shape) - axis - len(pshape))
    S, B = s.reshape(view), b.reshape(view)
    t = x * S
    assert_bit_exact(oracle.scale_op(x, axis, scale=s, bias=b), t + B, "scale+bias (two roundings)")
    assert_bit_exact(oracle.scale_op(x, axis, scale=s), t, "scale")
    assert_bit_exact(oracle.scale_op(x, axis, bias=b), x + B, "bias")


def test_scale_value_form_and_no_fma():
    x = normal(43, (2, 3, 4))
    got = oracle.scale_op(x, 1, scale_value=[2.0], bias_value=[1.0, 2.0, 3.0])
    want = x * F(2.0) + F([1, 2, 3]).reshape(1, 3, 1)
    assert_bit_exact(got, want, "value form, size-1 value replicated")
    with pytest.raises(oracle.OracleCheckError):
        oracle.scale_op(x, 1, scale_value=[1.0, 2.0])
    # a product that needs rounding: fused evaluation would give another result
    xx = F([1.0 + 2.0 ** -12])
    got = oracle.scale_bias(xx, F([1.0 + 2.0 ** -12]), F([-(1.0 + 2.0 ** -11)]), 1, 1)
    assert got[0] == F(F(xx[0] * xx[0]) + F(-(1.0 + 2.0 ** -11)))
    assert got[0] != F(np.float64(xx[0]) ** 2 - (1.0 + 2.0 ** -11))


# ---------------------------------------------------------------- eltwise ---
def test_eltwise_against_numpy():
    xs = [normal(50 + j, 3000) for j in range(4)]
    co = [1.0, -0.5, 2.0, 0.25]
    acc = np.zeros(3000, F)
    for c, x in zip(co, xs):
        acc = acc + F(c) * x
    assert_bit_exact(oracle.eltwise(1, xs, co), acc, "sum: 0 + c0*x0 + c1*x1 ...")
    assert_bit_exact(oracle.eltwise(0, xs), ((xs[0] * xs[1]) * xs[2]) * xs[3], "prod")
    assert_bit_exact(oracle.eltwise(2, xs), sel_max(sel_max(sel_max(xs[0], xs[1]), xs[2]), xs[3]), "max")
    assert_bit_exact(oracle.eltwise(3, xs), sel_min(sel_min(sel_min(xs[0], xs[1]), xs[2]), xs[3]), "min")


def test_eltwise_reference_observations_and_checks():
    got = oracle.eltwise(1, [F([-0.0, 0.0]), F([-0.0, -0.0])])
    assert list(bits(got)) == [0, 0]  # (-0)+(-0) and (+0)+(-0) both give +0
    with pytest.raises(oracle.OracleCheckError):
        oracle.eltwise_op([np.zeros(3, F), np.zeros(4, F)], 1)
    with pytest.raises(oracle.OracleCheckError):
        oracle.eltwise_op([np.zeros(3, F), np.zeros(3, F)], 2, coeff=[1, 1])
    with pytest.raises(oracle.OracleCheckError):
        oracle.eltwise_op([np.zeros(3, F), np.zeros(3, F)], 1, coeff=[1])


# ----------------------------------------------------------------- reduce ---
def brute_reduce(x, axes, op):
    """Window-by-window evaluation with numpy indexing; windows are visited with
    the last listed axis fastest, values folded sequentially."""
    out_shape = [1 if n in axes else d for n, d in enumerate(x.shape)]
    out = np.empty(out_shape, F)
    for idx in itertools.product(*[range(d) for d in out_shape]):
        vals = []
        for r in itertools.product(*[range(x.shape[a]) for a in axes]):
            full = list(idx)
            for a, v in zip(axes, r):
                full[a] = v
            vals.append(x[tuple(full)])
        if op == 0:
            v = np.float64(1)
            for t in vals:
                v = v * np.float64(t)
            res = F(v)
        elif op in (1, 4, 5):
            v = np.float64(0)
            for t in vals:
                v = v + np.float64(abs(t) if op == 5 else t)
            res = F(v / len(vals)) if op == 4 else F(v)
        elif op == 6:
            v = np.float64(0)
            for t in vals:
                a = np.abs(F(t))
                v = v + np.float64(F(a * a))
            res = np.sqrt(F(v))
        elif op == 2:
            v = F(-3.4028235e38)
            for t in vals:
                v = t if v < t else v
            res = v
        else:
            v = F(3.4028235e38)
            for t in vals:
                v = t if t < v else v
            res = v
        out[idx] = res
    return out


@pytest.mark.parametrize("shape,axes", [((3, 4, 5), [1]), ((3, 4, 5), [0, 2]), ((2, 3, 4, 2), [2, 3]),
                                        ((2, 3, 4, 2), [3, 1]), ((6,), [0]), ((2, 3), [0, 1])])
@pytest.mark.parametrize("op", range(7))
def test_reduce_against_brute_force(shape, axes, op):
    x = normal(60, shape)
    with np.errstate(all="ignore"):
        want = brute_reduce(x, axes, op)
    got = oracle.reduce_op(x, op, axes, True)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "reduce op %d" % op)


def test_reduce_exact_integer_sums_and_shapes():
    x = np.arange(1, 7, dtype=F).reshape(2, 3)
    got = oracle.reduce_op(x, 1, [], False)
    assert got.shape == () and got == 21  # observed on the reference: value 21, rank-0 shape
    assert oracle.reduce_op(x, 1, [], True).shape == (1, 1)
    big = (np.arange(200000) % 1000).astype(F).reshape(200, 1000)
    assert_bit_exact(oracle.reduce_op(big, 1, [1]), np.full((200, 1), 499500, F), "row sums")
    assert_bit_exact(oracle.reduce_op(big, 4, [1]), np.full((200, 1), 499.5, F), "row means")
    assert_bit_exact(oracle.reduce_op(F([[3, 4]]), 6, [1]), F([[5]]), "L2 of [3,4]")
    k = oracle.reduce_op(normal(61, (2, 3, 4, 5)), 2, [1, 3], False)
    assert k.shape == (2, 4)


def test_reduce_select_reference_observations():
    assert oracle.reduce_op(F([[1, np.nan, 3]]), 2, [1])[0, 0] == 3  # NaNs skipped
    assert bits(oracle.reduce_op(F([[np.nan, np.nan]]), 2, [1]))[0, 0] == 0xff7fffff  # identity leaks
    assert bits(oracle.reduce_op(F([[np.nan, np.nan]]), 3, [1]))[0, 0] == 0x7f7fffff
    # first zero in list order decides the sign
    assert bits(oracle.reduce_op(F([[-0.0, 0.0]]), 2, [1]))[0, 0] == 0x80000000
    assert bits(oracle.reduce_op(F([[0.0, -0.0]]), 2, [1]))[0, 0] == 0x00000000
    assert bits(oracle.reduce_op(F([[-0.0, 0.0]]), 3, [1]))[0, 0] == 0x80000000
    # identities are finite: +inf cannot beat FLT_MAX in a min, nor -inf in a max
    assert bits(oracle.reduce_op(F([[np.inf, np.inf]]), 3, [1]))[0, 0] == 0x7f7fffff
    assert bits(oracle.reduce_op(F([[-np.inf]]), 2, [1]))[0, 0] == 0xff7fffff


def test_reduce_sum_close_to_exact():
    x = normal(62, (64, 784))
    got = oracle.reduce_op(x, 1, [1]).ravel()
    exact = np.array([math.fsum(map(float, row)) for row in x])
    assert ulp_distance(got, exact.astype(F)).max() <= 1


# ------------------------------------------------------------------ blas ----
def test_level1():
    x, y = normal(70, 1000), normal(71, 1000)
    assert_bit_exact(oracle.scal(0.37, x), x * F(0.37), "scal")
    assert_bit_exact(oracle.copy(x), x, "copy")
    assert_bit_exact(oracle.axpy(-1.3, x, y), y + F(-1.3) * x, "axpy")
    assert oracle.asum(F([1, -2, 3.5])) == F(6.5)
    assert_bit_exact(oracle.blas_set(5, 2.5), np.full(5, 2.5, F), "set")
