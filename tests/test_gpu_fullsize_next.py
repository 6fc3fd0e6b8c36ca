"""The neighbouring operators and the data movers at the size of the headline
tensor (fp32 [64,256,56,56] = 205 MB, or the ResNet shape that feeds them),
through Operator::Run against the oracle on the same buffers.  Same bars as at
small sizes: bit-exact, except the fp64-summing norms (1e-5, observed 0)."""
import numpy as np
import pytest

import oracle
import shadow_amd
from tests.helpers import assert_bit_exact, assert_rel_close, normal, uniform

pytestmark = pytest.mark.gpu
F = np.float32
SHAPE = (64, 256, 56, 56)


@pytest.fixture(scope="module")
def big():
    return normal(901, SHAPE, 2.0)


@pytest.fixture()
def ws(gpu):
    w = shadow_amd.Workspace("Native", 0)
    yield w
    w.close()


def run(ws, op_type, inputs, args, tops=("out",)):
    names = []
    for name, arr in inputs:
        ws.set_blob(name, arr)
        names.append(name)
    op = ws.create_op(op_type, names, list(tops), args)
    op.run()
    got = [ws.get_blob(t) for t in tops]
    return got[0] if len(got) == 1 else got


def test_batch_norm_and_axpy(ws, big):
    mean, var = normal(902, 256), uniform(903, 256, 0.2, 3.0)
    got = run(ws, "BatchNorm", [("x", big), ("m", mean), ("v", var)], {"eps": 1e-5})
    assert_bit_exact(got, oracle.batch_norm_op(big, mean, var), "batch norm")
    alpha = uniform(904, (64, 256), -1.0, 1.0)
    got = run(ws, "Axpy", [("alpha", alpha), ("x", big), ("y", got)], {}, tops=["ax"])
    assert_bit_exact(got, oracle.axpy_op(alpha, big, oracle.batch_norm_op(big, mean, var)), "axpy")


def test_stem_pooling(ws):
    x = normal(905, (64, 64, 112, 112), 2.0)
    for pool in (0, 1):
        got = run(ws, "Pooling", [("x", x)], {"pool": pool, "kernel_size": [3], "stride": [2], "pad": [0]},
                  tops=["p%d" % pool])
        want = oracle.pooling_op(x, pool, [3], [2], [0])
        assert got.shape == want.shape == (64, 64, 56, 56)
        assert_bit_exact(got, want, "stem pooling %d" % pool)


def test_global_pooling_and_softmax(ws, big):
    feat = big.reshape(512, 2048, 7, 7)
    got = run(ws, "Pooling", [("x", feat)], {"pool": 1, "global_pooling": True})
    want = oracle.pooling_op(feat, 1, global_pooling=True)
    assert_bit_exact(got, want, "global average pooling")
    dense = big.reshape(64, 49, 128, 128)
    got = run(ws, "Softmax", [("d", dense)], {"axis": 1}, tops=["sm"])
    want = oracle.softmax_op(dense, 1)
    assert_bit_exact(got, want, "channel softmax")
    # columns sum to one within a few ulp (size-independent property)
    assert np.abs(got.sum(axis=1, dtype=np.float64) - 1).max() < 1e-6
    got = run(ws, "Normalize", [("d", dense)], {"axis": 1}, tops=["nz"])
    assert_bit_exact(got, oracle.normalize_op(dense, 2.0, 1), "channel L2 normalize")


def test_norms(ws, big):
    scale, bias = uniform(906, 256, 0.5, 1.5), normal(907, 256, 0.1)
    got = run(ws, "InstanceNorm", [("x", big), ("s", scale), ("b", bias)], {})
    assert assert_rel_close(got, oracle.instance_norm_op(big, 1e-5, scale, bias), 1e-5, "instance norm") == 0
    got = run(ws, "GroupNorm", [("x", big), ("s", scale), ("b", bias)], {"group": 32}, tops=["gn"])
    assert assert_rel_close(got, oracle.group_norm_op(big, 32, 1e-5, scale, bias), 1e-5, "group norm") == 0
    rows = big.reshape(65536, 784)
    ls, lb = uniform(908, 784, 0.5, 1.5), normal(909, 784, 0.1)
    got = run(ws, "LayerNorm", [("r", rows), ("ls", ls), ("lb", lb)], {"normalized_shape": [784]}, tops=["ln"])
    assert assert_rel_close(got, oracle.layer_norm_op(rows, [784], 1e-5, ls, lb), 1e-5, "layer norm") == 0


def test_movers(ws, big):
    got = run(ws, "Permute", [("x", big)], {"order": [0, 2, 3, 1]})
    assert_bit_exact(got, big.transpose(0, 2, 3, 1), "NCHW -> NHWC")
    # a permutation followed by its inverse is the identity (size-independent property)
    back = run(ws, "Permute", [("nhwc", got)], {"order": [0, 3, 1, 2]}, tops=["back"])
    assert_bit_exact(back, big, "permute round trip")
    got = run(ws, "ShuffleChannel", [("x", big)], {"group": 2}, tops=["sh"])
    assert_bit_exact(got, oracle.shuffle_channel_op(big, 2), "shuffle")
    a, b = run(ws, "Slice", [("x", big)], {"axis": 1}, tops=["lo", "hi"])
    assert_bit_exact(a, big[:, :128], "slice low")
    assert_bit_exact(b, big[:, 128:], "slice high")
    got = run(ws, "Concat", [("lo", a), ("hi", b)], {"axis": 1}, tops=["cat"])
    assert_bit_exact(got, big, "slice then concat")
    small = big.reshape(64, 64, 112, 112)[:, :, :56, :56].copy()
    got = run(ws, "Resize", [("s", small)], {"scale": [2.0]}, tops=["up"])
    assert_bit_exact(got, oracle.resize_op(small, scale=[2.0]), "bilinear x2")
    got = run(ws, "Reorg", [("x4", big.reshape(64, 64, 112, 112))], {"type": 1, "stride": 2}, tops=["ro"])
    assert_bit_exact(got, oracle.reorg_op(big.reshape(64, 64, 112, 112), 1, 2), "reorg")
    got = run(ws, "Pad", [("x", big)], {"paddings": [1, 1, 1, 1], "value": 0.5}, tops=["pd"])
    assert_bit_exact(got, np.pad(big, ((0, 0), (0, 0), (1, 1), (1, 1)), constant_values=F(0.5)), "pad")


def test_lrn_and_grid_sample(ws, big):
    got = run(ws, "LRN", [("x", big)], {"local_size": 5, "alpha": 1e-4, "beta": 0.75, "k": 1.0}, tops=["lrn"])
    assert_bit_exact(got, oracle.lrn_op(big, 5, 1e-4, 0.75, 0, 1.0), "lrn")
    gy, gx = np.meshgrid(np.linspace(-1, 1, 56), np.linspace(-1, 1, 56), indexing="ij")
    grid = np.stack([gx, gy], -1).astype(F)[None] + uniform(906, (64, 56, 56, 2), -0.08, 0.08)  # leaves the input at the rim
    for mode in (0, 1):
        got = run(ws, "GridSample", [("x", big), ("grid", grid)], {"mode": mode, "padding_mode": mode}, tops=["gs%d" % mode])
        assert_bit_exact(got, oracle.grid_sample_op(big, grid, mode, mode), "grid sample %d" % mode)
