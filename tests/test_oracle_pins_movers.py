"""Pins for the oracle's data movers: every one is an index map, so numpy's own
indexing (concatenate, split, stack, take, pad, transpose, reshape) is an
independent statement of the expected result.  Resize is pinned by hand-computed
cases, exact identities (integer scale factors, constant images) and an fp32
numpy restatement of the coordinate rule on whole arrays."""
import numpy as np
import pytest

import oracle
from tests.helpers import assert_bit_exact, normal

F = np.float32


def ramp(shape):
    return np.arange(int(np.prod(shape)), dtype=F).reshape(shape)


@pytest.mark.parametrize("axis", [0, 1, 2, 3, -1, -3])
def test_concat_slice_stack(axis):
    a, b, c = normal(1, (2, 3, 4, 5)), normal(2, (2, 3, 4, 5)), normal(3, (2, 3, 4, 5))
    ax = axis % 4
    wide = np.concatenate([a, b, c], ax)
    assert_bit_exact(oracle.concat_op([a, b, c], axis), wide, "concat")
    parts = oracle.slice_op(wide, 3, axis)
    for got, want in zip(parts, (a, b, c)):
        assert_bit_exact(got, want, "slice equal")
    assert_bit_exact(oracle.stack_op([a, b, c], axis), np.stack([a, b, c], axis), "stack")
    assert_bit_exact(oracle.stack_op([a, b], 4), np.stack([a, b], 4), "stack last")


def test_concat_uneven_and_slice_points():
    a, b = normal(4, (2, 3, 4)), normal(5, (2, 7, 4))
    assert_bit_exact(oracle.concat_op([a, b], 1), np.concatenate([a, b], 1), "concat uneven")
    x = normal(6, (3, 10, 2))
    got = oracle.slice_op(x, 3, 1, [2, 7])
    for g, w in zip(got, np.split(x, [2, 7], 1)):
        assert g.shape == w.shape
        assert_bit_exact(g, w, "slice points")
    for bad in (lambda: oracle.concat_op([a], 1), lambda: oracle.concat_op([a, normal(7, (2, 3, 5))], 1),
                lambda: oracle.slice_op(x, 3, 1), lambda: oracle.slice_op(x, 3, 1, [7, 2]),
                lambda: oracle.slice_op(x, 3, 1, [2, 10]), lambda: oracle.stack_op([a, a], 4)):
        with pytest.raises(oracle.OracleCheckError):
            bad()


@pytest.mark.parametrize("axis,idx", [(0, [2, 0]), (1, [4, 4, 1, 0, 3]), (2, [1]), (-1, [0, 2, 1])])
def test_gather(axis, idx):
    x = normal(8, (3, 5, 2, 3))
    assert_bit_exact(oracle.gather_op(x, axis, idx), np.take(x, idx, axis), "gather")


@pytest.mark.parametrize("pads", [[1, 2, 3, 4], [0, 0, 0, 1], [-1, 2, 0, -2], [-1, -1, -1, -1], [2, -1, -2, 3],
                                  [0, 0, 0, 0]])
def test_pad(pads):
    x = normal(9, (2, 3, 6, 7))
    t, b, l, r = pads
    crop = x[:, :, max(-t, 0):6 - max(-b, 0), max(-l, 0):7 - max(-r, 0)]
    want = np.pad(crop, ((0, 0), (0, 0), (max(t, 0), max(b, 0)), (max(l, 0), max(r, 0))), constant_values=F(-2.5))
    got = oracle.pad_op(x, pads, -2.5)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "pad")


@pytest.mark.parametrize("shape,order", [((2, 3, 4, 5), [0, 2, 3, 1]), ((2, 3, 4, 5), [0, 3, 1, 2]),
                                         ((2, 3, 4, 5), [3, 2, 1, 0]), ((4, 6), [1, 0]), ((2, 3, 4), [0, 1, 2]),
                                         ((2, 3, 4, 5, 6), [4, 0, 3, 1, 2]), ((7,), [0]), ((2, 1, 3), [2, 1, 0])])
def test_permute(shape, order):
    x = normal(10, shape)
    assert_bit_exact(oracle.permute_op(x, order), x.transpose(order), "permute")


def test_reorg():
    x = normal(11, (2, 8, 6, 4))
    s = 2
    # natural: out[b, (c2*s + oh)*s + ow, h, w] = in[b, c2, h*s + oh, w*s + ow]
    want = x.reshape(2, 8, 3, s, 2, s).transpose(0, 1, 3, 5, 2, 4).reshape(2, 32, 3, 2)
    assert_bit_exact(oracle.reorg_op(x, 1, s), want, "reorg natural")
    # Darknet: the flat result equals in viewed as [b, c/ss, h*s, w*s], read as
    # out_flat[b, c, h, w] = view[b, c % oc, h*s + (c/oc)/s, w*s + (c/oc)%s]
    oc = 8 // (s * s)
    view = x.reshape(2, oc, 6 * s, 4 * s)
    flat = np.empty((2, 8, 6, 4), F)
    for c in range(8):
        off = c // oc
        flat[:, c] = view[:, c % oc, off // s::s, off % s::s]
    got = oracle.reorg_op(x, 0, s)
    assert got.shape == (2, 32, 3, 2)
    assert_bit_exact(got, flat, "reorg darknet")
    with pytest.raises(oracle.OracleCheckError):
        oracle.reorg_op(normal(12, (1, 6, 4, 4)), 0, 2)
    with pytest.raises(oracle.OracleCheckError):
        oracle.reorg_op(normal(12, (1, 4, 5, 4)), 1, 2)


@pytest.mark.parametrize("group", [1, 2, 3, 6])
def test_shuffle_channel(group):
    x = normal(13, (2, 6, 3, 5))
    want = x.reshape(2, group, 6 // group, 3, 5).transpose(0, 2, 1, 3, 4).reshape(x.shape)
    assert_bit_exact(oracle.shuffle_channel_op(x, group), want, "shuffle")


# ----------------------------------------------------------------- resize ---
def bilinear_numpy(x, out_h, out_w, align):
    """The reference's rule on whole arrays, every product and sum a rounded fp32 operation."""
    in_h, in_w = x.shape[2:]

    def axis(out, inn):
        o = np.arange(out, dtype=F)
        if align:
            f = F(inn - 1) / F(out - 1)
            src = o * f
        else:
            f = F(inn) / F(out)
            src = (o + F(0.5)) * f - F(0.5)
            src = np.where(src < 0, F(0), src)
        lo = src.astype(np.int32)
        hi = lo + 1
        edge = lo >= inn - 1
        lo = np.where(edge, inn - 1, lo)
        hi = np.where(edge, inn - 1, hi)
        return lo, hi, (src - lo.astype(F)).astype(F)

    hl, hh, sh = axis(out_h, in_h)
    wl, wh, sw = axis(out_w, in_w)
    sh, sw = sh[:, None], sw[None, :]
    one = F(1)
    v0, v1 = x[:, :, hl][:, :, :, wl], x[:, :, hh][:, :, :, wl]
    v2, v3 = x[:, :, hl][:, :, :, wh], x[:, :, hh][:, :, :, wh]
    return (((one - sh) * (one - sw)) * v0 + (sh * (one - sw)) * v1 + ((one - sh) * sw) * v2) + (sh * sw) * v3


@pytest.mark.parametrize("align", [False, True])
@pytest.mark.parametrize("in_hw,out_hw", [((5, 7), (10, 14)), ((8, 8), (3, 5)), ((4, 6), (9, 7)), ((2, 2), (5, 5)),
                                          ((7, 3), (7, 9))])
def test_resize_bilinear_against_array_formulation(align, in_hw, out_hw):
    x = normal(14, (2, 3) + in_hw, 2.0)
    got = oracle.resize_op(x, size=list(out_hw), type=1, align_corners=align)
    assert_bit_exact(got, bilinear_numpy(x, out_hw[0], out_hw[1], align), "bilinear")


def test_resize_known_values():
    x = ramp((1, 1, 2, 2))  # [[0, 1], [2, 3]]
    # align_corners to 3x3: corners kept, midpoints are exact averages
    got = oracle.resize_op(x, size=[3, 3], type=1, align_corners=True)
    assert got.ravel().tolist() == [0, 0.5, 1, 1, 1.5, 2, 2, 2.5, 3]
    # half-pixel centres to 4x4: source coords -0.25 -> 0, 0.25, 0.75, 1.25 -> clamped to the last row
    got = oracle.resize_op(x, scale=[2.0], type=1)
    assert got[0, 0, 0].tolist() == [0, 0.25, 0.75, 1]
    assert got[0, 0, :, 0].tolist() == [0, 0.5, 1.5, 2]
    # nearest with integer factors repeats pixels; source index is floor(o * in / out)
    assert_bit_exact(oracle.resize_op(x, scale=[2.0], type=0), np.repeat(np.repeat(x, 2, 2), 2, 3), "nearest x2")
    y = ramp((1, 1, 4, 6))
    assert_bit_exact(oracle.resize_op(y, size=[2, 3], type=0), y[:, :, ::2, ::2], "nearest /2")
    assert oracle.resize_op(y, size=[3, 4], type=0)[0, 0, :, 0].tolist() == [0, 6, 12]
    # a constant image stays constant (weights sum to 1 exactly for dyadic fractions)
    const = np.full((1, 2, 4, 4), 3.0, F)
    assert_bit_exact(oracle.resize_op(const, scale=[2.0]), np.full((1, 2, 8, 8), 3.0, F), "constant")
    # same size is a copy; the scale form truncates
    assert_bit_exact(oracle.resize_op(y, size=[4, 6]), y, "copy")
    assert oracle.resize_op(y, scale=[1.4, 0.5]).shape == (1, 1, 5, 3)
    for bad in (lambda: oracle.resize_op(y, size=[1, 2, 3]), lambda: oracle.resize_op(y, type=2),
                lambda: oracle.resize_op(y, scale=[0.1]), lambda: oracle.resize_op(ramp((2, 3, 4)))):
        with pytest.raises(oracle.OracleCheckError):
            bad()
