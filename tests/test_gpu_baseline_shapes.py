"""The five BASELINE workloads at their full shapes and seeds, HIP path against
the CPU oracle on the same buffers (the oracle needs a few seconds per config).
Elementwise, broadcast, max: bit-exact.  Sum / mean: |gpu - cpu| <= 1e-5 |cpu|,
plus a size-independent cross-check (sum of row sums == full sum in fp64)."""
import numpy as np
import pytest

import oracle
from tests import gpuops
from tests.helpers import assert_bit_exact, assert_rel_close, bits, normal, uniform

pytestmark = pytest.mark.gpu


def test_cfg1_binary_add_channel_broadcast(gpu):
    sa, sb = [8, 64, 112, 112], [1, 64, 1, 1]
    a, b = uniform(101, sa, -1, 1), uniform(102, sb, -1, 1)
    got = gpuops.broadcast_binary(0, a, sa, b, sb, sa)
    assert_bit_exact(got, oracle.broadcast_binary(0, a, sa, b, sb, sa), "cfg1")
    assert_bit_exact(got, (a + b).ravel(), "cfg1 vs numpy broadcast")


@pytest.fixture(scope="module")
def cfg2_x():
    return normal(201, 64 * 256 * 56 * 56, 2.0)


@pytest.mark.parametrize("name,kind,code", [("relu", "act", 1), ("sigmoid", "act", 3), ("tanh", "act", 5),
                                            ("exp", "unary", 4), ("abs", "unary", 0)])
def test_cfg2_single_ops(gpu, cfg2_x, name, kind, code):
    if kind == "act":
        got, want = gpuops.activate(cfg2_x, code), oracle.activate(cfg2_x, code)
    else:
        got, want = gpuops.unary(code, cfg2_x), oracle.unary(code, cfg2_x)
    assert_bit_exact(got, want, "cfg2 " + name)


def test_cfg2_sqrt_of_abs_and_scale_relu(gpu, cfg2_x):
    a = gpuops.unary(0, cfg2_x)
    assert_bit_exact(gpuops.unary(2, a), oracle.unary(2, oracle.unary(0, cfg2_x)), "sqrt(abs)")
    g, b = uniform(202, 256, 0.5, 1.5), uniform(203, 256, -0.1, 0.1)
    want = oracle.activate(oracle.scale_bias(cfg2_x, g, b, 256, 3136), 1)
    assert_bit_exact(gpuops.scale_bias(cfg2_x, g, b, 256, 3136, relu=True), want, "fused scale+relu")
    unfused = gpuops.activate(gpuops.scale_bias(cfg2_x, g, b, 256, 3136), 1)
    assert_bit_exact(unfused, want, "scale then relu")


def test_cfg3_reductions(gpu):
    shape = [32, 512, 28, 28]
    x = normal(301, shape)
    for op in (1, 4):
        got, _ = gpuops.reduce(op, x, shape, [2, 3])
        want, _ = oracle.reduce(op, x, shape, [2, 3])
        differing = assert_rel_close(got, want, 1e-5, "cfg3 {2,3} op %d" % op)
        assert differing == 0  # fp64 accumulation: same float after the single rounding
    got, _ = gpuops.reduce(2, x, shape, [1])
    assert_bit_exact(got, oracle.reduce(2, x, shape, [1])[0], "cfg3 max over channels")
    assert_bit_exact(got, x.max(axis=1).ravel(), "cfg3 max vs numpy")
    full, _ = gpuops.reduce(1, x, shape, [0, 1, 2, 3])
    want, _ = oracle.reduce(1, x, shape, [0, 1, 2, 3])
    assert_rel_close(full, want, 1e-5, "cfg3 full sum")
    # size-independent: the full sum is the sum of the row sums
    rows, _ = gpuops.reduce(1, x, shape, [2, 3])
    exact = np.sum(x.astype(np.float64))
    assert abs(float(full[0]) - exact) <= 1e-5 * abs(exact) + 1e-3
    assert abs(np.sum(rows.astype(np.float64)) - exact) <= 1e-4 * np.sum(np.abs(rows.astype(np.float64)))


@pytest.mark.parametrize("sa,sb,seeds", [([16, 1, 128, 256], [1, 32, 128, 1], (401, 402)),
                                         ([4, 64, 1, 512], [1, 1, 64, 512], (403, 404)),
                                         ([128, 1024], [1, 1], (405, 406))])
def test_cfg4_general_broadcast(gpu, sa, sb, seeds):
    so = [max(p, q) for p, q in zip(sa, sb)]
    a, b = normal(seeds[0], sa), uniform(seeds[1], sb, 0.5, 2.0)
    for op in (2, 1, 3, 5):
        got = gpuops.broadcast_binary(op, a, sa, b, sb, so)
        assert_bit_exact(got, oracle.broadcast_binary(op, a, sa, b, sb, so), "cfg4 op %d" % op)
    if sb == [1, 1]:  # pair (iii) also through the scalar-argument form
        for op in (2, 1, 3, 5):
            assert_bit_exact(gpuops.binary_scalar(op, a, float(b.ravel()[0])),
                             oracle.binary_scalar(op, a, float(b.ravel()[0])), "cfg4 scalar form")


def test_cfg5_resnet_tail(gpu):
    n, C, inner = 64 * 1024 * 14 * 14, 1024, 196
    x, r = normal(501, n), normal(504, n)
    g, b = uniform(502, C, 0.5, 1.5), uniform(503, C, -0.1, 0.1)
    s = oracle.scale_bias(x, g, b, C, inner)
    e = oracle.eltwise(1, [s, r], [1.0, 1.0])
    y = oracle.activate(e, 1)
    m, _ = oracle.reduce(4, y, [64 * 1024, inner], [1])
    # four separate launches
    gs = gpuops.scale_bias(x, g, b, C, inner)
    assert_bit_exact(gs, s, "cfg5 scale")
    ge = gpuops.eltwise(1, [gs, r])
    assert_bit_exact(ge, e, "cfg5 eltwise sum")
    gy = gpuops.activate(ge, 1)
    assert_bit_exact(gy, y, "cfg5 relu")
    gm, _ = gpuops.reduce(4, gy, [64, 1024, 14, 14], [2, 3])
    assert assert_rel_close(gm, m, 1e-5, "cfg5 pooled") == 0
    # one launch
    fy, fm = gpuops.scale_residual_relu_rowmean(x, g, b, r, C, inner)
    assert_bit_exact(fy, y, "cfg5 fused y")
    assert assert_rel_close(fm, m, 1e-5, "cfg5 fused mean") == 0
