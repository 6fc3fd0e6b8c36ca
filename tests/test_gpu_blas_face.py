"""The inner free-function layer, Blas::X<kGPU, float> and Vision::X<kGPU, float>,
driven the way the reference's kernels outside this path call it: with element
offsets (`offa`, `offb`, `offy`), in place, and in the call sequences of the
convolution epilogue (kernels/conv.hpp:122-131), of Eltwise (kernels/
eltwise.hpp:37-44) and of SSDNormalize (kernels/ssd_normalize.hpp:47-75).  Every
result is compared with the oracle; elementwise results bit for bit."""
import ctypes

import numpy as np
import pytest

import oracle
import shadow_amd
from tests.helpers import assert_bit_exact, assert_rel_close, normal, uniform

pytestmark = pytest.mark.gpu
F32P = ctypes.POINTER(ctypes.c_float)
SENTINEL = np.float32(-777.25)


def _p(a):
    return a.ctypes.data_as(F32P) if a is not None else None


@pytest.fixture(scope="module")
def ws(gpu):
    with shadow_amd.Workspace("Native", 0) as w:
        yield w


def blas(ws, name, n, a=None, offa=0, b=None, offb=0, alpha=0.0, y=None, offy=0, y_count=None):
    """Returns the whole y buffer after the call (cells outside [offy, offy + n) keep what was uploaded)."""
    a = None if a is None else np.ascontiguousarray(a, np.float32)
    if y is None:
        y = np.full(y_count if y_count is not None else offy + n + 5, SENTINEL, np.float32)
    y = np.ascontiguousarray(y, np.float32).copy()
    bb = None if b is None else np.ascontiguousarray(b, np.float32)
    rc = ws.lib.shdw_host_face_blas(ws.ptr, name.encode(), n, _p(a), 0 if a is None else a.size, offa, _p(bb),
                                    0 if bb is None else bb.size, offb, alpha, _p(y), y.size, offy)
    shadow_amd.host_check(rc == 0)
    return y


def untouched(y, offy, n):
    return (y[:offy] == SENTINEL).all() and (y[offy + n:] == SENTINEL).all()


UNARY = {"Abs": 0, "Square": 1, "Sqrt": 2, "Log": 3, "Exp": 4, "Sin": 5, "Cos": 6, "Tan": 7, "Asin": 8,
         "Acos": 9, "Atan": 10, "Floor": 11, "Ceil": 12, "Neg": 13, "Reciprocal": 14}
BINARY = {"Add": 0, "Sub": 1, "Mul": 2, "Div": 3, "Pow": 4, "Max": 5, "Min": 6}


@pytest.mark.parametrize("name", sorted(UNARY))
@pytest.mark.parametrize("n,offa,offy", [(1001, 3, 7), (64, 0, 1), (5, 2, 0)])
def test_unary_with_offsets(ws, name, n, offa, offy):
    a = normal(40, n + offa + 3)
    if name in ("Asin", "Acos"):
        a = uniform(41, n + offa + 3, -1, 1)
    y = blas(ws, name, n, a, offa, offy=offy)
    assert untouched(y, offy, n)
    assert_bit_exact(y[offy:offy + n], oracle.unary(UNARY[name], a[offa:offa + n]), name)


@pytest.mark.parametrize("name", sorted(BINARY))
@pytest.mark.parametrize("n,offa,offb,offy", [(1003, 5, 9, 2), (128, 1, 0, 3)])
def test_binary_tensor_and_scalar_with_offsets(ws, name, n, offa, offb, offy):
    a, b = normal(42, n + offa + 1), uniform(43, n + offb + 2, 0.5, 2.0)
    if name == "Pow":
        a = np.abs(a) + np.float32(0.1)
    y = blas(ws, name, n, a, offa, b, offb, offy=offy)
    assert untouched(y, offy, n)
    assert_bit_exact(y[offy:offy + n], oracle.binary(BINARY[name], a[offa:offa + n], b[offb:offb + n]), name)
    y = blas(ws, name, n, a, offa, alpha=1.75, offy=offy)
    assert untouched(y, offy, n)
    assert_bit_exact(y[offy:offy + n], oracle.binary_scalar(BINARY[name], a[offa:offa + n], 1.75), name + " scalar")


def test_level1_with_offsets(ws):
    n, offa, offy = 997, 6, 11
    x, y0 = normal(44, n + offa + 2), normal(45, n + offy + 4)
    y = blas(ws, "Set", n, alpha=2.5, offy=offy)
    assert untouched(y, offy, n) and (y[offy:offy + n] == np.float32(2.5)).all()
    y = blas(ws, "Scopy", n, x, offa, offy=offy)
    assert untouched(y, offy, n)
    assert_bit_exact(y[offy:offy + n], x[offa:offa + n], "Scopy")
    y = blas(ws, "Sscal", n, alpha=-0.3, y=y0, offy=offy)
    want = y0.copy()
    want[offy:offy + n] = oracle.scal(-0.3, y0[offy:offy + n])
    assert_bit_exact(y, want, "Sscal")
    y = blas(ws, "Saxpy", n, x, offa, alpha=0.7, y=y0, offy=offy)
    want = y0.copy()
    want[offy:offy + n] = oracle.axpy(0.7, x[offa:offa + n], y0[offy:offy + n])
    assert_bit_exact(y, want, "Saxpy")
    for count, off in ((n, offa), (5, 1), (300000, 3)):
        big = normal(46, count + off)
        got = blas(ws, "Sasum", count, big, off, y_count=4)[0]
        assert_rel_close(np.float32([got]), np.float32([oracle.asum(big[off:off + count])]), 1e-5, "Sasum")


def test_in_place_through_the_face(ws):
    """a is None: the y buffer is the first operand too, as in Blas::Mul(count, out_data, 0,
    inputs[n]->data(), 0, out_data, 0, ...) (kernels/eltwise.hpp:31-33)."""
    n, off = 515, 4
    x, b = normal(47, n + off + 3), normal(48, n)
    y = blas(ws, "Abs", n, None, off, y=x, offy=off)
    want = x.copy()
    want[off:off + n] = np.abs(x[off:off + n])
    assert_bit_exact(y, want, "Abs in place")
    y = blas(ws, "Mul", n, None, off, b, 0, y=x, offy=off)
    want = x.copy()
    want[off:off + n] = oracle.binary(2, x[off:off + n], b)
    assert_bit_exact(y, want, "Mul in place")
    y = blas(ws, "Max", n, None, off, alpha=0.25, y=x, offy=off)
    want = x.copy()
    want[off:off + n] = oracle.binary_scalar(5, x[off:off + n], 0.25)
    assert_bit_exact(y, want, "Max scalar in place")


@pytest.mark.parametrize("num_output,spatial,batch", [(16, 49, 3), (7, 1, 5), (64, 3136, 2)])
@pytest.mark.parametrize("bias_term,act", [(1, 1), (1, 0), (0, 1)])
def test_conv_epilogue(ws, num_output, spatial, batch, bias_term, act):
    count = batch * num_output * spatial
    out, bias = normal(50, count), normal(51, num_output)
    got = out.copy()
    rc = ws.lib.shdw_host_face_conv_epilogue(ws.ptr, _p(got), count, _p(bias), num_output, spatial, bias_term, act)
    shadow_amd.host_check(rc == 0)
    want = out
    if bias_term:
        want = oracle.scale_bias(want, None, bias, num_output, spatial)
    if act == 1:
        want = oracle.activate(want, 1, 0.0)
    assert_bit_exact(got, want, "conv epilogue")


@pytest.mark.parametrize("k", [2, 3, 5])
def test_eltwise_sum_as_set_plus_saxpy(ws, k):
    n = 10007
    xs = [normal(60 + j, n) for j in range(k)]
    coeff = np.float32([1.0, -0.5, 2.25, 0.125, 3.0][:k])
    ptrs = (F32P * k)(*[_p(x) for x in xs])
    got = np.empty(n, np.float32)
    shadow_amd.host_check(ws.lib.shdw_host_face_eltwise_sum(ws.ptr, k, ptrs, _p(coeff), n, _p(got)) == 0)
    assert_bit_exact(got, oracle.eltwise(1, xs, coeff), "Set + Saxpy")


@pytest.mark.parametrize("across_spatial", [0, 1])
@pytest.mark.parametrize("scale_kind", ["none", "shared", "channel"])
@pytest.mark.parametrize("batch,channel,spatial", [(3, 8, 49), (2, 20, 361), (5, 3, 1)])
def test_ssd_normalize_run_sequence(ws, across_spatial, scale_kind, batch, channel, spatial):
    x = normal(70, batch * channel * spatial)
    scale = None
    if scale_kind == "shared":
        scale = np.float32([20.0])
    elif scale_kind == "channel":
        scale = uniform(71, channel, 10.0, 30.0)
    got = np.empty_like(x)
    rc = ws.lib.shdw_host_face_ssd_normalize(ws.ptr, _p(x), batch, channel, spatial, across_spatial,
                                             int(scale_kind == "shared"), 1e-5, _p(scale), _p(got))
    shadow_amd.host_check(rc == 0)
    want = oracle.ssd_normalize(x, batch, channel, spatial, across_spatial, scale_kind == "shared", 1e-5, scale)
    if across_spatial:
        assert_rel_close(got, want, 1e-5, "per item (fp64 sums associate differently)")
    else:
        assert_bit_exact(got, want, "per position")


def test_unknown_function_is_an_error(ws):
    with pytest.raises(shadow_amd.ShadowError):
        blas(ws, "Sgemm", 4, normal(1, 8))
