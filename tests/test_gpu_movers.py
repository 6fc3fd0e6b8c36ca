"""GPU parity of the data movers through Operator::Run: bit for bit against the
oracle (pure index maps, and Resize whose fp32 weights are computed in the
reference's operation order)."""
import numpy as np
import pytest

import oracle
import shadow_amd
from shadow_amd import ShadowError
from tests.helpers import assert_bit_exact, normal, with_specials

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture()
def ws(gpu):
    w = shadow_amd.Workspace("Native", 0)
    yield w
    w.close()


def run(ws, op_type, inputs, args, tops=("out",)):
    names = []
    for name, arr in inputs:
        ws.set_blob(name, arr, dtype="int32" if np.asarray(arr).dtype.kind == "i" else "float")
        names.append(name)
    op = ws.create_op(op_type, names, list(tops), args)
    op.run()
    got = [ws.get_blob(t) for t in tops]
    return got[0] if len(got) == 1 else got


@pytest.mark.parametrize("shapes,axis", [
    ([(2, 3, 4, 5), (2, 7, 4, 5)], 1), ([(2, 3, 4, 8), (2, 3, 4, 4), (2, 3, 4, 12)], 3),
    ([(3, 5), (2, 5), (4, 5)], 0), ([(2, 3, 7), (2, 3, 1)], -1), ([(4, 16, 14, 14), (4, 32, 14, 14)], 1),
    ([(2, 3, 5, 5), (2, 3, 5, 5)], 2),
    # chunks and pitches that are no whole vectors: 128-bit accesses on any dword address with the chunk's cut
    # end float by float (chunks of 49, 5, 75 and 1001 floats), chunks under four floats
    ([(3, 1, 7, 7), (3, 2, 7, 7)], 1), ([(40, 5), (40, 9), (40, 2)], 1), ([(6, 3, 25), (6, 4, 25)], 1),
    ([(5, 1001), (5, 1003)], 1), ([(4, 7, 3), (4, 7, 1)], 2)])
def test_concat_op(ws, shapes, axis):
    xs = [normal(10 + k, s) for k, s in enumerate(shapes)]
    got = run(ws, "Concat", [("x%d" % k, x) for k, x in enumerate(xs)], {"axis": axis})
    want = oracle.concat_op(xs, axis)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "concat")


@pytest.mark.parametrize("shape,axis,points,n", [((2, 12, 4, 4), 1, [], 3), ((2, 12, 4, 4), 1, [4, 5], 3),
                                                 ((6, 5), 0, [], 2), ((2, 3, 10), -1, [3], 2),
                                                 ((4, 48, 7, 7), 1, [16, 32], 3),
                                                 ((3, 5, 7, 7), 1, [1, 3], 3), ((30, 21), 1, [5, 14], 3),
                                                 ((4, 2004), 1, [1001], 2), ((6, 9, 5), 1, [2], 2)])
def test_slice_op(ws, shape, axis, points, n):
    x = normal(20, shape)
    args = {"axis": axis}
    if points:
        args["slice_point"] = points
    got = run(ws, "Slice", [("x", x)], args, tops=["o%d" % k for k in range(n)])
    want = oracle.slice_op(x, n, axis, points)
    for g, w in zip(got, want):
        assert g.shape == w.shape
        assert_bit_exact(g, w, "slice")


@pytest.mark.parametrize("shape,axis,k", [((2, 3, 4), 0, 2), ((2, 3, 4), 1, 3), ((2, 3, 4), 3, 2), ((2, 3, 4), -1, 2),
                                          ((5, 8), -2, 4), ((16, 64), 1, 3), ((7, 49), 1, 3), ((3, 5, 13), 1, 2)])
def test_stack_op(ws, shape, axis, k):
    xs = [normal(30 + j, shape) for j in range(k)]
    got = run(ws, "Stack", [("x%d" % j, x) for j, x in enumerate(xs)], {"axis": axis})
    want = oracle.stack_op(xs, axis)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "stack")


@pytest.mark.parametrize("shape,axis,idx", [((5, 8), 0, [4, 0, 0, 2]), ((3, 6, 4), 1, [5, 1]), ((2, 3, 7), -1, [6, 0, 3]),
                                            ((4, 10, 16), 1, [9, 8, 7, 0, 1, 2, 2]),
                                            ((3, 6, 7), 1, [5, 1]), ((2, 9, 7, 7), 1, [8, 8, 0]),  # rows of 7 and 49 floats
                                            ((5, 3), 0, [4, 1, 1])])
def test_gather_op(ws, shape, axis, idx):
    x = normal(40, shape)
    want = oracle.gather_op(x, axis, idx)
    got = run(ws, "Gather", [("x", x)], {"axis": axis, "indexes": idx})
    assert got.shape == want.shape
    assert_bit_exact(got, want, "gather by argument")
    got = run(ws, "Gather", [("x", x), ("idx", np.asarray(idx, np.int32))], {"axis": axis}, tops=["out2"])
    assert_bit_exact(got, want, "gather by blob")


def test_gather_index_checks(ws):
    x = normal(41, (4, 6))
    ws.set_blob("x", x)
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("Gather", ["x"], ["o"], {"axis": 0, "indexes": [4]}).run()
    with pytest.raises(ShadowError, match="Check Failed"):
        ws.create_op("Gather", ["x"], ["o1"], {"axis": 0}).run()
    # a bad index in a device blob cannot be checked on the host: that row comes out as zeros
    got = run(ws, "Gather", [("x", x), ("idx", np.asarray([1, 9, -1, 3], np.int32))], {"axis": 0}, tops=["o2"])
    assert_bit_exact(got, np.stack([x[1], np.zeros(6, F), np.zeros(6, F), x[3]]), "out-of-range rows")


@pytest.mark.parametrize("pads", [[1, 2, 3, 4], [0, 0, 0, 1], [-1, 2, 0, -2], [-1, -1, -1, -1], [2, -1, -2, 3],
                                  [0, 0, 0, 0]])
@pytest.mark.parametrize("shape", [(2, 3, 6, 7), (1, 2, 16, 16), (1, 3, 33, 29)])
def test_pad_op(ws, pads, shape):
    x = normal(50, shape)
    got = run(ws, "Pad", [("x", x)], {"paddings": pads, "value": -2.5})
    want = oracle.pad_op(x, pads, -2.5)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "pad")


@pytest.mark.parametrize("shape,order", [
    ((2, 3, 4, 5), [0, 2, 3, 1]), ((2, 3, 4, 5), [0, 3, 1, 2]), ((2, 3, 4, 5), [3, 2, 1, 0]), ((4, 6), [1, 0]),
    ((2, 3, 4), [0, 1, 2]), ((2, 3, 4, 5, 6), [4, 0, 3, 1, 2]), ((7,), [0]), ((2, 1, 3), [2, 1, 0]),
    ((3, 130, 70), [0, 2, 1]), ((200, 131), [1, 0]), ((2, 64, 28, 28), [0, 2, 3, 1]), ((2, 5, 6, 7), [1, 0, 2, 3]),
    ((2, 3, 4, 5), [0, 1, 3, 2]), ((1, 1, 9), [2, 0, 1]),
    # one thin side (interleaved <-> planar images): whole and ragged tiles, odd lengths, batches
    ((1000, 3), [1, 0]), ((3, 1000), [1, 0]), ((2, 37, 41, 3), [0, 3, 1, 2]), ((2, 3, 37, 41), [0, 2, 3, 1]),
    ((3, 777, 5), [0, 2, 1]), ((2, 16, 9001), [0, 2, 1]), ((9001, 16), [1, 0]), ((1, 6000, 1), [1, 0, 2]),
    ((4, 260, 1, 2), [0, 3, 2, 1]), ((5462, 3), [1, 0]), ((2, 257, 13), [0, 2, 1]), ((17, 300), [1, 0]),
    # thin sides up to 128 (a detection head's [anchors][85][cells] -> [anchors][cells][85]); multiples of
    # eight take the padded tile
    ((3, 85, 1444), [0, 2, 1]), ((3, 1444, 85), [0, 2, 1]), ((2, 8, 1000), [0, 2, 1]), ((2, 1001, 8), [0, 2, 1]),
    ((64, 300), [1, 0]), ((300, 64), [1, 0]), ((2, 24, 5000), [0, 2, 1]), ((5000, 120), [1, 0]),
    ((120, 4999), [1, 0]), ((127, 257), [1, 0]), ((256, 128), [1, 0]), ((128, 256), [1, 0]), ((100, 333), [1, 0]),
    ((1, 3, 85, 19, 19), [0, 1, 3, 4, 2])])
def test_permute_op(ws, shape, order):
    x = normal(60, shape)
    got = run(ws, "Permute", [("x", x)], {"order": order})
    want = oracle.permute_op(x, order)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "permute")


@pytest.mark.parametrize("type_", [0, 1])
# rows that are whole vectors and rows that are not (26, 38, 6 and 9 floats: a lane's four source floats run
# over the end of a row, a channel and an image), strides 1 to 4, a tensor that is no whole vectors
@pytest.mark.parametrize("shape,stride", [((2, 8, 6, 4), 2), ((1, 9, 6, 9), 3), ((2, 64, 26, 26), 2), ((1, 4, 2, 2), 1),
                                          ((3, 16, 38, 38), 2), ((2, 4, 6, 6), 2), ((3, 9, 3, 3), 3), ((2, 16, 8, 12), 4),
                                          ((1, 4, 2, 6), 2), ((5, 4, 10, 2), 2)])
def test_reorg_op(ws, type_, shape, stride):
    x = normal(70, shape)
    got = run(ws, "Reorg", [("x", x)], {"type": type_, "stride": stride})
    want = oracle.reorg_op(x, type_, stride)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "reorg")


@pytest.mark.parametrize("align", [False, True])
@pytest.mark.parametrize("shape,size", [
    ((3, 5, 56, 56), [112, 112]),    # several bands per plane, 128-bit both sides
    ((2, 3, 57, 33), [114, 66]),     # rows that are not a multiple of four floats
    ((1, 2, 120, 64), [17, 40]),     # reduction by 7: a band spans many input rows
    ((1, 1, 300, 5), [2, 10]),       # two output rows 150 input rows apart
    ((1, 1, 4, 6000), [8, 9000]),    # rows too wide for the staged kernel: gather kernel
    ((2, 2, 9, 2100), [5, 4100]),    # one-row bands with a large tile
    ((1, 3, 200, 31), [333, 77]),    # odd output width: a lane's four outputs span two rows
    ((2, 3, 75, 75), [150, 150]),    # x2 of odd maps: bands start on any dword
    ((2, 2, 13, 13), [26, 26]),
    ((2, 3, 19, 19), [38, 38]),
    ((1, 5, 7, 3), [9, 2]),          # rows shorter than a lane's four outputs
    ((1, 4, 10, 10), [23, 2]),
    ((64, 64, 13, 13), [26, 26]),    # small maps, many planes: two whole planes per workgroup
    ((96, 128, 5, 3), [10, 6]),      # five planes per workgroup, three in the last
    ((65, 64, 7, 5), [10, 9])])      # odd rows across the planes of a group
def test_resize_bilinear_bands(ws, shape, size, align):
    x = normal(91, shape, 2.0)
    got = run(ws, "Resize", [("x", x)], {"size": size, "align_corners": align})
    want = oracle.resize_op(x, size, [1.0], 1, align)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "resize %s -> %s" % (shape, size))


@pytest.mark.parametrize("shape,size", [((3, 5, 56, 56), [112, 112]), ((2, 3, 75, 75), [150, 150]),
                                        ((2, 2, 13, 13), [26, 26]), ((2, 3, 19, 19), [38, 38]), ((1, 5, 7, 3), [9, 2]),
                                        ((1, 4, 10, 10), [23, 1]), ((3, 2, 33, 21), [50, 47]), ((1, 1, 50, 47), [33, 21]),
                                        ((1, 1, 1, 1), [3, 3]), ((64, 64, 13, 13), [26, 26]),
                                        ((96, 128, 5, 3), [10, 6]), ((65, 64, 7, 5), [10, 9]),
                                        ((1, 1, 4, 6000), [8, 9000])])  # rows too wide to stage: gathers
def test_resize_nearest_any_width(ws, shape, size):
    """Output rows of any length: four consecutive outputs per lane, across row
    ends where the width is not a multiple of four."""
    x = normal(92, shape, 2.0)
    got = run(ws, "Resize", [("x", x)], {"size": size, "type": 0})
    want = oracle.resize_op(x, size, [1.0], 0, False)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "nearest %s -> %s" % (shape, size))


@pytest.mark.parametrize("typ", [0, 1])
@pytest.mark.parametrize("shape", [(1, 1, 1, 4), (2, 3, 1, 6), (1, 2, 2, 4), (3, 1, 3, 8), (2, 2, 57, 6), (1, 3, 5, 130),
                                   (3, 5, 56, 56), (2, 2, 38, 38), (1, 1, 9, 4096)])
def test_resize_by_two_of_even_rows(ws, typ, shape):
    """Exactly x2 on rows of an even number (>= 4) of positions: the kernels without staging.  Infinities and NaNs
    are planted (a weight of zero times an infinity is a NaN, as in the reference's sum), also in the edge
    columns and rows."""
    x = with_specials(normal(93, shape, 2.0), 93).reshape(shape)
    x[..., 0, 1] = np.inf
    x[..., -1, -1] = -np.inf
    x[0, 0, 0, 0] = np.nan
    got = run(ws, "Resize", [("x", x)], {"scale": [2.0], "type": typ})
    want = oracle.resize_op(x, [0], [2.0], typ, False)
    assert got.shape == want.shape
    assert_bit_exact(got, want, "x2 type %d %s" % (typ, shape))


@pytest.mark.parametrize("typ", [0, 1])
@pytest.mark.parametrize("x_off,y_off", [(1, 0), (2, 0), (3, 0), (0, 1), (2, 2), (1, 3)])
def test_resize_by_two_on_pointers_off_the_vector_boundary(gpu, typ, x_off, y_off):
    """x2 through the C ABI with the input and the output 1 to 3 floats off 16-byte alignment: whichever kernel
    the alignment leaves (the one without staging needs y on 16 bytes and, for nearest, x on 8), same bits."""
    shape = (2, 3, 19, 24)
    x = with_specials(normal(94, shape, 2.0), 94).reshape(shape)
    want = oracle.resize_op(x, [0], [2.0], typ, False)
    lib = shadow_amd.hip()
    dx = shadow_amd.Buffer(x.nbytes + 16)
    dx.upload(x, 4 * x_off)
    dy = shadow_amd.Buffer(want.nbytes + 16)
    shadow_amd.check(lib.shdw_hip_resize(shadow_amd.ints(list(shape)), shadow_amd.ints(list(want.shape)), typ, 0,
                                         dx.ptr + 4 * x_off, dy.ptr + 4 * y_off, None))
    shadow_amd.check(lib.shdw_hip_stream_sync(None))
    got = dy.download(count=want.size, offset_bytes=4 * y_off).reshape(want.shape)
    assert_bit_exact(got, want, "x2 type %d, x + %d, y + %d floats" % (typ, x_off, y_off))


@pytest.mark.parametrize("shape,group", [((2, 6, 3, 5), 2), ((2, 6, 3, 5), 3), ((1, 12, 4, 4), 4), ((3, 8, 1, 1), 8),
                                         ((2, 116, 28, 28), 2), ((2, 6, 3, 5), 1), ((2, 116, 7, 7), 2), ((3, 4, 1, 3), 2),
                                         # rows of 7, 1, 2, 5 and 49 floats: a lane's four outputs from up to four rows
                                         ((9, 12, 1, 7), 4), ((33, 10, 1, 1), 5), ((7, 6, 1, 2), 3), ((5, 9, 5, 1), 3),
                                         ((3, 232, 7, 7), 2), ((1, 3, 1, 1), 3)])
def test_shuffle_channel_op(ws, shape, group):
    x = normal(80, shape)
    got = run(ws, "ShuffleChannel", [("x", x)], {"group": group})
    assert_bit_exact(got, oracle.shuffle_channel_op(x, group), "shuffle")


@pytest.mark.parametrize("args", [
    {"scale": [2.0]}, {"scale": [2.0], "align_corners": True}, {"size": [9, 7]}, {"size": [9, 7], "align_corners": True},
    {"size": [3, 5], "type": 0}, {"scale": [2.0], "type": 0}, {"scale": [0.5, 1.5]}, {"size": [4, 6]},
    {"size": [2, 2], "align_corners": True}, {"size": [1, 5]}, {"scale": [3.0]}, {"size": [13], "type": 0}])
@pytest.mark.parametrize("shape", [(2, 3, 4, 6), (1, 2, 17, 9)])
def test_resize_op(ws, args, shape):
    x = with_specials(normal(90, shape, 2.0), 90).reshape(shape)
    got = run(ws, "Resize", [("x", x)], args)
    want = oracle.resize_op(x, args.get("size", [0]), args.get("scale", [1.0]), args.get("type", 1),
                            args.get("align_corners", False))
    assert got.shape == want.shape
    assert_bit_exact(got, want, "resize %s" % args)


def test_mover_argument_errors(ws):
    ws.set_blob("x", np.zeros((2, 6, 4, 4), F))
    ws.set_blob("y", np.zeros((2, 6, 4, 5), F))
    bad = [("Concat", ["x"], ["o0"], {}), ("Concat", ["x", "y"], ["o1"], {"axis": 1}),
           ("Slice", ["x"], ["a", "b", "c", "d"], {"axis": 1}), ("Slice", ["x"], ["a2"], {"axis": 1}),
           ("Slice", ["x"], ["a3", "b3"], {"axis": 1, "slice_point": [6]}),
           ("Stack", ["x", "x"], ["o2"], {"axis": 5}), ("Stack", ["x", "y"], ["o3"], {"axis": 0}),
           ("Pad", ["x"], ["o4"], {"paddings": [-2, -2, 0, 0]}), ("Permute", ["x"], ["o5"], {"order": [0, 1, 2]}),
           ("Permute", ["x"], ["o6"], {"order": [0, 1, 1, 2]}), ("Reorg", ["x"], ["o7"], {"type": 0, "stride": 2}),
           ("Reorg", ["x"], ["o8"], {"type": 2, "stride": 2}), ("Reorg", ["y"], ["o9"], {"type": 1, "stride": 2}),
           ("ShuffleChannel", ["x"], ["o10"], {"group": 4}), ("Resize", ["x"], ["o11"], {"size": [1, 2, 3]}),
           ("Resize", ["x"], ["o12"], {"scale": [0.1]}), ("Resize", ["x"], ["o13"], {"size": [1, 8], "align_corners": True}),
           ("Permute", ["x"], ["x"], {"order": [0, 1, 2, 3]})]
    for op_type, bottoms, tops, args in bad:
        with pytest.raises(ShadowError):
            ws.create_op(op_type, bottoms, tops, args).run()
    for op_type, args in (("Pad", {"paddings": [1, 1]}), ("ShuffleChannel", {}), ("Resize", {"type": 2})):
        with pytest.raises(ShadowError, match="Check Failed"):
            ws.create_op(op_type, ["x"], ["oo"], args)
