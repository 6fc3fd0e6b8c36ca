"""The six operators through Operator::Run() (C++ layer behind its C facade),
against the operator-level oracle: values, output shapes, argument handling and
the errors the reference raises through CHECK."""
import numpy as np
import pytest

import oracle
import shadow_amd
from shadow_amd import ShadowError
from tests.helpers import assert_bit_exact, assert_rel_close, normal, uniform, with_specials

pytestmark = pytest.mark.gpu


@pytest.fixture()
def ws(gpu):
    w = shadow_amd.Workspace("Native", 0)
    yield w
    w.close()


def run(ws, op_type, inputs, args, top="out", bottoms=None):
    names = []
    for k, (name, arr) in enumerate(inputs):
        ws.set_blob(name, arr)
        names.append(name)
    op = ws.create_op(op_type, bottoms or names, [top], args)
    op.run()
    return ws.get_blob(top)


@pytest.mark.parametrize("operation", range(15))
def test_unary_op(ws, operation):
    x = normal(1, (3, 5, 7, 11), 2.0)
    if operation in (8, 9):
        x = np.clip(x, -1, 1)
    got = run(ws, "Unary", [("x", x)], {"operation": operation})
    want = oracle.unary_op(x, operation)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "unary %d" % operation)


def test_unary_op_argument_errors(ws):
    ws.set_blob("x", np.zeros((2, 2), np.float32))
    for bad in (15, -1):
        with pytest.raises(ShadowError, match="Check Failed"):
            ws.create_op("Unary", ["x"], ["y"], {"operation": bad})
    with pytest.raises(ShadowError):  # operation is mandatory (default -1)
        ws.create_op("Unary", ["x"], ["y"], {})
    with pytest.raises(ShadowError, match="not registered"):
        ws.create_op("NoSuchOp", ["x"], ["y"], {})


@pytest.mark.parametrize("operation", [0, 1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("sa,sb", [((2, 3, 4), (2, 3, 4)), ((2, 1), (3,)), ((8, 64, 12, 12), (1, 64, 1, 1)),
                                   ((16, 1, 8, 32), (1, 5, 8, 1)), ((4, 6, 1, 32), (6, 32)), ((12, 10), (1,)),
                                   ((3,), (2, 4, 3))])
def test_binary_op(ws, operation, sa, sb):
    a = with_specials(normal(2, sa), 1).reshape(sa)
    b = with_specials(uniform(3, sb, 0.5, 2.0), 2).reshape(sb)
    got = run(ws, "Binary", [("a", a), ("b", b)], {"operation": operation})
    want = oracle.binary_op(a, b, operation=operation)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "binary")
    # the input blobs keep their own shapes after the rank alignment
    assert tuple(ws.blob_shape("a")) == tuple(sa) and tuple(ws.blob_shape("b")) == tuple(sb)


def test_binary_scalar_form_and_errors(ws):
    x = normal(4, (5, 6))
    for operation in (0, 1, 2, 3, 5, 6):
        got = run(ws, "Binary", [("x", x)], {"operation": operation, "scalar": 0.75}, top="o%d" % operation)
        assert_bit_exact(got, oracle.binary_op(x, operation=operation, scalar=0.75), "scalar form")
    ws.set_blob("p", np.zeros((2, 3), np.float32))
    ws.set_blob("q", np.zeros((2,), np.float32))
    op = ws.create_op("Binary", ["p", "q"], ["r"], {"operation": 0})
    with pytest.raises(ShadowError, match="Check Failed"):
        op.run()  # [2,3] + [2] does not broadcast
    assert ws.blob_shape("p") == [2, 3] and ws.blob_shape("q") == [2]
    with pytest.raises(ShadowError):
        ws.create_op("Binary", ["p", "q"], ["r2"], {"operation": 7})
    one = ws.create_op("Binary", ["p"], ["r3"], {"operation": 0})
    with pytest.raises(ShadowError):
        one.run()  # two inputs expected without `scalar`


@pytest.mark.parametrize("operation", [0, 1, 2, 3])
@pytest.mark.parametrize("k", [2, 3, 5])
def test_eltwise_op(ws, operation, k):
    xs = [normal(10 + j, (4, 3, 14, 14)) for j in range(k)]
    args = {"operation": operation}
    coeff = []
    if operation == 1:
        coeff = [1.0, -0.5, 2.0, 0.25, 1.5][:k]
        args["coeff"] = coeff
    got = run(ws, "Eltwise", [("x%d" % j, x) for j, x in enumerate(xs)], args)
    assert_bit_exact(got, oracle.eltwise_op(xs, operation, coeff), "eltwise")


def test_eltwise_op_errors(ws):
    ws.set_blob("a", np.zeros((2, 3), np.float32))
    ws.set_blob("b", np.zeros((2, 3), np.float32))
    ws.set_blob("c", np.zeros((3, 2), np.float32))
    with pytest.raises(ShadowError):
        ws.create_op("Eltwise", ["a", "c"], ["o1"], {"operation": 1}).run()
    with pytest.raises(ShadowError, match="only takes coefficients for summation"):
        ws.create_op("Eltwise", ["a", "b"], ["o2"], {"operation": 2, "coeff": [1.0, 1.0]}).run()
    with pytest.raises(ShadowError, match="one coefficient per input"):
        ws.create_op("Eltwise", ["a", "b"], ["o3"], {"operation": 1, "coeff": [1.0]}).run()
    with pytest.raises(ShadowError):
        ws.create_op("Eltwise", ["a"], ["o4"], {"operation": 1}).run()
    with pytest.raises(ShadowError):
        ws.create_op("Eltwise", ["a", "b"], ["o5"], {"operation": 4})


@pytest.mark.parametrize("shape,axes", [((4, 8, 7, 7), [2, 3]), ((4, 8, 7, 7), [1]), ((4, 8, 7, 7), []),
                                        ((2, 3, 4, 5), [0, 2]), ((6, 10), [0]), ((5,), [0]),
                                        # two stages through the Workspace's temp buffer: channel statistics,
                                        # the leading dim first, sliced rows behind a leading dim
                                        ((6, 8, 9, 9), [0, 2, 3]), ((40, 6, 7, 5), [0, 2]), ((3, 2, 300, 301), [0, 2, 3])])
@pytest.mark.parametrize("operation", range(7))
@pytest.mark.parametrize("keep_dims", [True, False])
def test_reduce_op(ws, shape, axes, operation, keep_dims):
    x = uniform(20, shape, 0.9, 1.1) if operation == 0 else normal(20, shape)
    args = {"operation": operation, "keep_dims": keep_dims}
    if axes:
        args["axes"] = axes
    got = run(ws, "Reduce", [("x", x)], args)
    want = oracle.reduce_op(x, operation, axes, keep_dims)
    assert list(got.shape) == list(want.shape)
    if operation in (2, 3):
        assert_bit_exact(got, want, "reduce")
    else:
        assert_rel_close(got, want, 1e-5, "reduce")


def test_reduce_op_observed_reference_cases(ws):
    x = np.arange(1, 7, dtype=np.float32).reshape(2, 3)
    got = run(ws, "Reduce", [("x", x)], {"operation": 1, "keep_dims": False})
    assert got.shape == () and got == 21  # all axes, rank-0 shape vector
    ws.set_blob("y", x)
    with pytest.raises(ShadowError):
        ws.create_op("Reduce", ["y"], ["y"], {"operation": 1}).run()  # never in place
    with pytest.raises(ShadowError, match="negative axes"):
        ws.create_op("Reduce", ["y"], ["z"], {"operation": 1, "axes": [-1]}).run()
    with pytest.raises(ShadowError):
        ws.create_op("Reduce", ["y"], ["z2"], {"operation": 7})
    l2 = run(ws, "Reduce", [("v", np.float32([[3, 4]]))], {"operation": 6, "axes": [1]}, top="l2")
    assert_bit_exact(l2, np.float32([[5]]), "L2 of [3,4]")
    mx = run(ws, "Reduce", [("w", np.float32([[1, np.nan, 3], [np.nan, np.nan, np.nan]]))],
             {"operation": 2, "axes": [1]}, top="mx")
    assert mx[0, 0] == 3 and mx.view(np.uint32)[1, 0] == 0xff7fffff


@pytest.mark.parametrize("act", [1, 2, 3, 4, 5, 6, 7, 8])
def test_activate_op(ws, act):
    x = with_specials(normal(30, (2, 6, 9, 9), 2.0), 3).reshape(2, 6, 9, 9)
    got = run(ws, "Activate", [("x", x)], {"type": act, "slope": 0.2})
    assert_bit_exact(got, oracle.activate_op(x, act, 0.2), "activate")


def test_activate_defaults_prelu_and_in_place(ws):
    x = normal(31, (2, 6, 5, 5))
    assert_bit_exact(run(ws, "Activate", [("x", x)], {}), oracle.activate_op(x, 1), "default type is relu")
    assert_bit_exact(run(ws, "Activate", [("x", x)], {"type": 2}, top="lk"), oracle.activate_op(x, 2, 0.1),
                     "default slope 0.1")
    for slope in (uniform(32, 6, -0.5, 0.5), np.float32([0.25])):
        got = run(ws, "Activate", [("x", x), ("s", slope)], {"type": 0}, top="pr%d" % slope.size)
        assert_bit_exact(got, oracle.activate_op(x, 0, slope_blob=slope), "prelu")
    # top == bottom, as converters emit it
    ws.set_blob("io", x)
    ws.create_op("Activate", ["io"], ["io"], {"type": 3}).run()
    assert_bit_exact(ws.get_blob("io"), oracle.activate_op(x, 3), "in place")
    with pytest.raises(ShadowError):
        ws.create_op("Activate", ["x"], ["bad"], {"type": 9})
    with pytest.raises(ShadowError):
        ws.create_op("Activate", ["x"], ["bad2"], {"type": 0}).run()  # PRelu needs the slope blob
    ws.set_blob("s5", np.zeros(5, np.float32))
    with pytest.raises(ShadowError):
        ws.create_op("Activate", ["x", "s5"], ["bad3"], {"type": 0}).run()  # 5 slopes for 6 channels


@pytest.mark.parametrize("shape,axis,pshape", [((4, 16, 14, 14), 1, (16,)), ((2, 5, 3, 4), 1, (5, 3)),
                                               ((3, 4, 5), 0, (3,)), ((2, 3, 8), 2, (8,)), ((6, 7), 1, (7,))])
def test_scale_op_blob_form(ws, shape, axis, pshape):
    x = normal(40, shape)
    s, b = uniform(41, pshape, 0.5, 1.5), uniform(42, pshape, -0.1, 0.1)
    base = {"axis": axis}
    got = run(ws, "Scale", [("x", x), ("s", s), ("b", b)], dict(base, has_scale=True, has_bias=True), top="o1")
    assert_bit_exact(got, oracle.scale_op(x, axis, scale=s, bias=b), "scale+bias")
    got = run(ws, "Scale", [("x", x), ("s", s)], dict(base, has_scale=True), top="o2")
    assert_bit_exact(got, oracle.scale_op(x, axis, scale=s), "scale only")
    got = run(ws, "Scale", [("x", x), ("b", b)], dict(base, has_bias=True), top="o3")
    assert_bit_exact(got, oracle.scale_op(x, axis, bias=b), "bias only")


def test_scale_op_value_form_in_place_and_errors(ws):
    x = normal(43, (2, 3, 4, 4))
    sv, bv = [0.5, 1.5, -2.0], [0.25]
    got = run(ws, "Scale", [("x", x)], {"scale_value": sv, "bias_value": bv}, top="v1")
    assert_bit_exact(got, oracle.scale_op(x, 1, scale_value=sv, bias_value=bv), "value form")
    got = run(ws, "Scale", [("x", x)], {"bias_value": [1.0, 2.0, 3.0]}, top="v2")
    assert_bit_exact(got, oracle.scale_op(x, 1, bias_value=[1.0, 2.0, 3.0]), "bias values only")
    ws.set_blob("io", x)
    op = ws.create_op("Scale", ["io"], ["io"], {"scale_value": sv, "bias_value": [0.0, 1.0, 2.0]})
    op.run()
    assert_bit_exact(ws.get_blob("io"), oracle.scale_op(x, 1, scale_value=sv, bias_value=[0.0, 1.0, 2.0]),
                     "in place")
    with pytest.raises(ShadowError):
        ws.create_op("Scale", ["x"], ["e1"], {"scale_value": [1.0, 2.0]}).run()
    with pytest.raises(ShadowError):
        ws.create_op("Scale", ["x"], ["e2"], {}).run()
    ws.set_blob("s", np.ones(3, np.float32))
    with pytest.raises(ShadowError):
        ws.create_op("Scale", ["x", "s"], ["e3"], {"has_scale": True, "has_bias": True}).run()


def test_output_blob_reuse_is_grow_only(ws):
    """One operator run on a big then a small then a big input: results stay right
    while the output blob keeps its allocation (Blob::reshape is grow-only)."""
    op = None
    for n in (4096, 16, 3000):
        x = normal(50 + n, (n,))
        ws.set_blob("x", x)
        if op is None:
            op = ws.create_op("Unary", ["x"], ["y"], {"operation": 1})
        op.run()
        assert_bit_exact(ws.get_blob("y"), x * x, "square n=%d" % n)


def test_chain_scale_eltwise_relu_pool(ws):
    """Config 5 as four operators sharing one workspace and stream, no sync in between."""
    shape = (4, 32, 14, 14)
    x, r = normal(60, shape), normal(61, shape)
    g, b = uniform(62, 32, 0.5, 1.5), uniform(63, 32, -0.1, 0.1)
    for name, arr in (("x", x), ("r", r), ("g", g), ("b", b)):
        ws.set_blob(name, arr)
    ops = [ws.create_op("Scale", ["x", "g", "b"], ["s"], {"axis": 1, "has_scale": True, "has_bias": True}),
           ws.create_op("Eltwise", ["s", "r"], ["e"], {"operation": 1}),
           ws.create_op("Activate", ["e"], ["e"], {"type": 1}),
           ws.create_op("Reduce", ["e"], ["p"], {"operation": 4, "axes": [2, 3]})]
    for op in ops:
        op.run()
    s = oracle.scale_op(x, 1, scale=g, bias=b)
    e = oracle.activate_op(oracle.eltwise_op([s, r], 1), 1)
    assert_bit_exact(ws.get_blob("e"), e, "tail")
    p = ws.get_blob("p")
    assert list(p.shape) == [4, 32, 1, 1]
    assert_rel_close(p, oracle.reduce_op(e, 4, [2, 3]), 1e-5, "pooled")
    assert "Scale" in ops[0].debug_log() and "x(4,32,14,14)" in ops[0].debug_log()


def test_workspace_rejects_cpu_backend(gpu):
    with pytest.raises(ShadowError, match="GPU-only"):
        shadow_amd.Workspace("CPU", 0)
