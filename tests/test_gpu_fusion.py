"""The Native backend's fusion pass: Scale -> Activate(relu),
Scale -> Eltwise(SUM) -> Activate(relu) [-> Reduce(AVG)], Eltwise -> Activate(relu) and
BatchNorm -> Scale [-> Activate(relu)] run as one launch each.
Every network here runs three ways: fused (the default), with fuse=False, and
through oracle.net.run (the operators one by one on the CPU).  The blobs a fused
run still writes must carry the same bits as the unfused run's, and the oracle's
too, except the mean, which the device sums in fp64 either way: fused and
unfused agree bit for bit there and both are within 1e-5 of the oracle.  Blobs
that have another reader, or that the network hands out, must block the fusion
that would stop writing them."""
import numpy as np
import pytest

import shadow_amd
from oracle import net as onet
from tests.helpers import assert_bit_exact, assert_rel_close, normal, uniform, with_specials

pytestmark = pytest.mark.gpu
F = np.float32


def arg_i(name, v):
    return (name, "s_i", int(v))


def op(typ, name, bottom, top, *args):
    return {"type": typ, "name": name, "bottom": list(bottom), "top": list(top), "arg": list(args)}


def scale_op(bottom, top, has_scale=True, has_bias=True, name="bn", axis=1):
    params = (["gamma"] if has_scale else []) + (["beta"] if has_bias else [])
    return op("Scale", name, [bottom] + params, [top], arg_i("axis", axis), arg_i("has_scale", has_scale),
              arg_i("has_bias", has_bias))


SHAPE = (3, 6, 5, 7)  # rows of 35 floats: not whole 128-bit vectors


def make(ops, out, shape=SHAPE, inputs=("x",), params=("gamma", "beta"), param_shape=None):
    c = shape[1]
    pshape = list(param_shape or [c])
    return {"name": "fusion", "arg": [("out_blob", "v_s", list(out))],
            "blob": [(p, "float", pshape) for p in params],
            "op": [op("Input", "in", [], list(inputs), *[(n, "v_i", list(shape)) for n in inputs])] + list(ops)}


def data(shape=SHAPE, inputs=("x",), seed=0, specials=True, nparams=2, param_shape=None):
    pshape = tuple(param_shape or [shape[1]])
    weights = [uniform(seed + 1, pshape, 0.5, 1.5), normal(seed + 2, pshape, 0.3)][:nparams]
    feed = {}
    for k, name in enumerate(inputs):
        a = normal(seed + 10 + k, shape, 2.0)
        if specials:
            a = with_specials(a, seed + k).reshape(shape)
        feed[name] = a
    return weights, feed


def run_all(net, weights, feed, written, fp64=(), expect_fused=None, reshape=False, against_oracle=True):
    """Fused and unfused runs against each other (bit for bit) and against the oracle."""
    text = onet.write_text(net)
    want = onet.run(net, weights, feed) if against_oracle else None
    with shadow_amd.Network(text, weights, fuse=False) as plain:
        assert plain.fused == []
        plain.forward(feed, reshape=reshape)
        ref = {name: plain.blob(name) for name in written}
    with shadow_amd.Network(text, weights) as nw:
        if expect_fused is not None:
            assert nw.fused == expect_fused
        for _ in range(2):  # a second forward finds the blobs already shaped
            nw.forward(feed, reshape=reshape)
            for name in written:
                got = nw.blob(name)
                assert list(got.shape) == list(ref[name].shape), name
                assert_bit_exact(got, ref[name], name + " fused against unfused")
                if want is None:
                    continue
                assert list(got.shape) == list(want[name].shape), name
                if name in fp64:
                    assert assert_rel_close(got, want[name], 1e-5, name) == 0
                else:
                    assert_bit_exact(got, want[name], name + " against the oracle")
        return nw.fused


@pytest.mark.parametrize("in_place", [False, True])
@pytest.mark.parametrize("has_scale,has_bias", [(True, True), (True, False), (False, True)])
def test_scale_relu(gpu, in_place, has_scale, has_bias):
    """has_bias alone is the Bias -> Activate pair of the convolution epilogue."""
    top = "s" if in_place else "y"
    params = (["gamma"] if has_scale else []) + (["beta"] if has_bias else [])
    net = make([scale_op("x", "s", has_scale, has_bias), op("Activate", "relu", ["s"], [top], arg_i("type", 1)),
                op("Unary", "neg", [top], ["out"], arg_i("operation", 13))], ["out"], params=params)
    weights, feed = data()
    weights = [w for w, keep in zip(weights, (has_scale, has_bias)) if keep]
    run_all(net, weights, feed, [top, "out"], expect_fused=["bn(Scale) + relu(Activate) -> " + top])


def test_scale_relu_with_parameters_over_two_axes_and_a_long_tensor(gpu):
    shape = (2, 4, 6, 64)
    net = make([scale_op("x", "s"), op("Activate", "relu", ["s"], ["s"])], ["s"], shape=shape, param_shape=[4, 6])
    weights, feed = data(shape, param_shape=[4, 6])
    assert run_all(net, weights, feed, ["s"]) == ["bn(Scale) + relu(Activate) -> s"]


TAIL = ["bn(Scale) + add(Eltwise) + relu(Activate) + gap(Reduce) -> e, pool"]


def tail_ops(relu_top="e", residual_first=False, keep_dims=True, axes=(2, 3), scale_in="x", scale_top="s"):
    return [scale_op(scale_in, scale_top),
            op("Eltwise", "add", ["r", scale_top] if residual_first else [scale_top, "r"], ["e"], arg_i("operation", 1)),
            op("Activate", "relu", ["e"], [relu_top], arg_i("type", 1)),
            op("Reduce", "gap", [relu_top], ["pool"], arg_i("operation", 4), ("axes", "v_i", list(axes)),
               arg_i("keep_dims", keep_dims))]


@pytest.mark.parametrize("shape", [SHAPE, (2, 8, 4, 8), (5, 3, 1, 1), (2, 5, 14, 14)])
@pytest.mark.parametrize("residual_first", [False, True])
@pytest.mark.parametrize("keep_dims", [True, False])
def test_residual_tail_with_mean(gpu, shape, residual_first, keep_dims):
    net = make(tail_ops(residual_first=residual_first, keep_dims=keep_dims), ["e", "pool"], shape=shape, inputs=("x", "r"))
    weights, feed = data(shape, ("x", "r"), seed=3, specials=False)
    run_all(net, weights, feed, ["e", "pool"], fp64=("pool",), expect_fused=TAIL)


def test_residual_tail_with_special_values(gpu):
    """Signed zeros, infinities and NaNs go through x*s + b, 0 + t, + r and the select
    exactly as through the four operators; the means of rows that hold them follow."""
    net = make(tail_ops()[:3], ["e"], inputs=("x", "r"))
    weights, feed = data(SHAPE, ("x", "r"), seed=5, specials=True)
    feed["r"][0, 0, 0, :4] = [0.0, -0.0, np.inf, -np.inf]
    feed["x"][0, 0, 0, :4] = [-0.0, -0.0, -np.inf, 1.0]
    run_all(net, weights, feed, ["e"], expect_fused=["bn(Scale) + add(Eltwise) + relu(Activate) -> e"])


def test_residual_tail_relu_into_another_blob_and_scale_in_place(gpu):
    net = make(tail_ops(relu_top="a", scale_in="x", scale_top="x"), ["a", "pool"], inputs=("x", "r"))
    weights, feed = data(SHAPE, ("x", "r"), seed=7, specials=False)
    run_all(net, weights, feed, ["a", "pool"], fp64=("pool",),
            expect_fused=["bn(Scale) + add(Eltwise) + relu(Activate) + gap(Reduce) -> a, pool"])


def test_tail_whose_reduce_covers_other_axes_runs_its_members_one_by_one(gpu):
    """The group is found from the operator list; whether the reduced axes are the run
    one parameter applies to is known when the blobs have their shapes."""
    for axes in ([3], [1, 2, 3], [0], []):
        net = make(tail_ops(axes=axes), ["e", "pool"], inputs=("x", "r"))
        weights, feed = data(SHAPE, ("x", "r"), seed=9, specials=False)
        run_all(net, weights, feed, ["e", "pool"], fp64=("pool",), expect_fused=TAIL)


def test_a_later_reader_of_the_activated_sum_keeps_the_mean_out_of_the_group(gpu):
    ops = tail_ops()
    ops.insert(3, op("Unary", "abs", ["e"], ["m"], arg_i("operation", 0)))
    net = make(ops, ["m", "pool"], inputs=("x", "r"))
    weights, feed = data(SHAPE, ("x", "r"), seed=11, specials=False)
    run_all(net, weights, feed, ["e", "m", "pool"], fp64=("pool",),
            expect_fused=["bn(Scale) + add(Eltwise) + relu(Activate) -> e"])


def test_an_operator_between_the_members_that_touches_nothing_of_theirs_is_stepped_over(gpu):
    ops = tail_ops()
    ops.insert(1, op("Unary", "abs", ["r"], ["m"], arg_i("operation", 0)))  # reads an input of the group: harmless
    net = make(ops, ["m", "pool"], inputs=("x", "r"))
    weights, feed = data(SHAPE, ("x", "r"), seed=13, specials=False)
    run_all(net, weights, feed, ["e", "m", "pool"], fp64=("pool",), expect_fused=TAIL)


ADD_RELU = ["add(Eltwise) + relu(Activate) -> e"]
# what keeps the Scale out of a group, and what is fused all the same: (operators, out_blob, blobs written, groups)
BLOCKED = {
    "the Scale output is an output of the network":
        (tail_ops(), ["s", "pool"], ["s", "e", "pool"], ADD_RELU),
    "the Scale output has a second reader":
        (tail_ops() + [op("Unary", "abs", ["s"], ["m"], arg_i("operation", 0))], ["m", "pool"], ["s", "e", "m", "pool"],
         ADD_RELU),
    "an operator in between rewrites the residual":
        (tail_ops()[:1] + [op("Unary", "neg", ["r"], ["r"], arg_i("operation", 13))] + tail_ops()[1:], ["pool"],
         ["s", "e", "pool"], ADD_RELU),
    "the sum has coefficients":
        ([scale_op("x", "s"), op("Eltwise", "add", ["s", "r"], ["e"], arg_i("operation", 1), ("coeff", "v_f", [F(1), F(0.5)])),
          op("Activate", "relu", ["e"], ["e"], arg_i("type", 1))], ["e"], ["s", "e"], ADD_RELU),
    "the Eltwise is a maximum":
        ([scale_op("x", "s"), op("Eltwise", "add", ["s", "r"], ["e"], arg_i("operation", 2)),
          op("Activate", "relu", ["e"], ["e"], arg_i("type", 1))], ["e"], ["s", "e"], ADD_RELU),
    "the activation is not relu":
        ([scale_op("x", "s"), op("Activate", "act", ["s"], ["y"], arg_i("type", 6))], ["y"], ["s", "y"], []),
    "the sum is read before it is activated elsewhere":
        ([scale_op("x", "s"), op("Eltwise", "add", ["s", "r"], ["e"], arg_i("operation", 1)),
          op("Activate", "relu", ["e"], ["a"], arg_i("type", 1)), op("Unary", "abs", ["e"], ["m"], arg_i("operation", 0))],
         ["a", "m"], ["s", "e", "a", "m"], []),
}


@pytest.mark.parametrize("why", sorted(BLOCKED))
def test_blocked(gpu, why):
    ops, out, written, groups = BLOCKED[why]
    net = make(ops, out, inputs=("x", "r"))
    weights, feed = data(SHAPE, ("x", "r"), seed=17, specials=False)
    run_all(net, weights, feed, written, fp64=("pool",), expect_fused=groups)


@pytest.mark.parametrize("operation", [0, 1, 2, 3])
@pytest.mark.parametrize("inputs", [2, 3, 9])
@pytest.mark.parametrize("in_place", [True, False])
def test_eltwise_relu(gpu, operation, inputs, in_place):
    """The add and the ReLU that close a residual block whose normalisation the converter
    folded into the convolution; any operation, any number of inputs (nine: two passes)."""
    names = ["x%d" % k for k in range(inputs)]
    top = "e" if in_place else "a"
    args = [arg_i("operation", operation)]
    if operation == 1 and inputs == 3:
        args.append(("coeff", "v_f", [F(1), F(-0.5), F(2)]))
    net = make([op("Eltwise", "add", names, ["e"], *args), op("Activate", "relu", ["e"], [top], arg_i("type", 1)),
                op("Unary", "abs", [top], ["out"], arg_i("operation", 0))], ["out"], inputs=names, params=())
    _, feed = data(SHAPE, names, seed=19 + operation, specials=True, nparams=0)
    run_all(net, [], feed, [top, "out"], expect_fused=["add(Eltwise) + relu(Activate) -> " + top])


def test_eltwise_whose_output_is_an_input_stays_an_operator(gpu):
    net = make([op("Eltwise", "add", ["x", "r"], ["x"], arg_i("operation", 1)),
                op("Activate", "relu", ["x"], ["x"], arg_i("type", 1))], ["x"], inputs=("x", "r"), params=())
    _, feed = data(SHAPE, ("x", "r"), seed=23, specials=False, nparams=0)
    # (the network oracle keeps blobs apart and does not model the cleared input: the two device runs only)
    run_all(net, [], feed, ["x"], expect_fused=[], against_oracle=False)


def test_scale_with_host_values_stays_an_operator(gpu):
    net = make([op("Scale", "sc", ["x"], ["s"], arg_i("axis", 1), ("scale_value", "v_f", [F(0.5)]),
                   ("bias_value", "v_f", [F(0.25)])), op("Activate", "relu", ["s"], ["s"], arg_i("type", 1))], ["s"], params=())
    _, feed = data(nparams=0)
    run_all(net, [], feed, ["s"], expect_fused=[])


def test_inputs_reshaped_between_forwards(gpu):
    net = make(tail_ops(keep_dims=False), ["e", "pool"], inputs=("x", "r"))
    text = onet.write_text(net)
    weights, _ = data(SHAPE, ("x", "r"))
    with shadow_amd.Network(text, weights) as nw:
        assert nw.fused == TAIL
        for shape in (SHAPE, (2, 6, 9, 4), (4, 6, 3, 3), SHAPE):
            _, feed = data(shape, ("x", "r"), seed=sum(shape), specials=False)
            want = onet.run(make(tail_ops(keep_dims=False), ["e", "pool"], shape=shape, inputs=("x", "r")), weights, feed)
            nw.forward(feed, reshape=True)
            assert_bit_exact(nw.blob("e"), want["e"], "e %s" % (shape,))
            assert nw.blob_shape("pool") == list(shape[:2])
            assert assert_rel_close(nw.blob("pool"), want["pool"], 1e-5, "pool") == 0


def test_full_size_bottleneck_tail_through_the_network(gpu):
    """BASELINE configs[4] as a converted model would hold it."""
    shape = (64, 1024, 14, 14)
    net = make(tail_ops(), ["e", "pool"], shape=shape, inputs=("x", "r"))
    weights = [uniform(502, 1024, 0.5, 1.5), uniform(503, 1024, -0.1, 0.1)]
    feed = {"x": normal(501, shape), "r": normal(504, shape)}
    text = onet.write_text(net)
    with shadow_amd.Network(text, weights, fuse=False) as plain:
        plain.forward(feed)
        e, pool = plain.blob("e"), plain.blob("pool")
    with shadow_amd.Network(text, weights) as nw:
        assert nw.fused == TAIL
        nw.forward(feed)
        assert_bit_exact(nw.blob("e"), e, "e")
        assert_bit_exact(nw.blob("pool"), pool, "pool")


# ---- BatchNorm -> Scale [-> ReLU] -------------------------------------------------------------------------------
def bn_net(ops, out, shape=SHAPE, factor=False, scale_param_shape=None, params=("gamma", "beta")):
    """mean, var [, factor], then the Scale parameters as declared blobs, in that order."""
    c = shape[1]
    blobs = [("mean", "float", [c]), ("var", "float", [c])] + ([("factor", "float", [1])] if factor else [])
    blobs += [(p, "float", list(scale_param_shape or [c])) for p in params]
    return {"name": "fusion", "arg": [("out_blob", "v_s", list(out))], "blob": blobs,
            "op": [op("Input", "in", [], ["x"], ("x", "v_i", list(shape)))] + list(ops)}


def bn_data(shape=SHAPE, factor=None, scale_param_shape=None, seed=40):
    c = shape[1]
    pshape = tuple(scale_param_shape or [c])
    weights = [normal(seed, c), uniform(seed + 1, c, 0.0, 30.0)] + ([np.array([factor], F)] if factor is not None else [])
    weights += [uniform(seed + 2, pshape, 0.5, 1.5), normal(seed + 3, pshape, 0.3)]
    return weights, {"x": with_specials(normal(seed + 4, shape, 2.0), seed).reshape(shape)}


def bn_op(bottom, top, factor=False):
    return op("BatchNorm", "bn", [bottom, "mean", "var"] + (["factor"] if factor else []), [top],
              ("eps", "s_f", 1e-3))


@pytest.mark.parametrize("in_place", [False, True])
@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("factor", [None, 999.982, 0.0])
def test_batch_norm_scale_relu(gpu, in_place, relu, factor):
    """How a Caffe-style model holds a normalisation, in place (one blob name throughout) and not."""
    n, s, y = ("x", "x", "x") if in_place else ("n", "s", "y")
    ops = [bn_op("x", n, factor is not None), scale_op(n, s, name="sc")]
    if relu:
        ops.append(op("Activate", "relu", [s], [y], arg_i("type", 1)))
    last = y if relu else s
    ops.append(op("Unary", "neg", [last], ["out"], arg_i("operation", 13)))
    net = bn_net(ops, ["out"], factor=factor is not None)
    weights, feed = bn_data(factor=factor)
    want = "bn(BatchNorm) + sc(Scale)" + (" + relu(Activate)" if relu else "") + " -> " + last
    run_all(net, weights, feed, [last, "out"], expect_fused=[want])


@pytest.mark.parametrize("has_scale,has_bias", [(True, False), (False, True)])
def test_batch_norm_scale_with_one_parameter_blob(gpu, has_scale, has_bias):
    net = bn_net([bn_op("x", "n"), scale_op("n", "s", has_scale, has_bias, name="sc"),
                  op("Activate", "relu", ["s"], ["s"], arg_i("type", 1))], ["s"],
                 params=["gamma"] if has_scale else ["beta"])
    weights, feed = bn_data()
    weights = weights[:2] + [w for w, keep in zip(weights[2:], (has_scale, has_bias)) if keep]
    run_all(net, weights, feed, ["s"], expect_fused=["bn(BatchNorm) + sc(Scale) + relu(Activate) -> s"])


def test_batch_norm_scale_on_long_rows_and_on_single_positions(gpu):
    for shape in ((2, 4, 6, 64), (5, 9, 1, 1), (3, 7, 1, 3)):
        net = bn_net([bn_op("x", "x"), scale_op("x", "x", name="sc"), op("Activate", "relu", ["x"], ["x"], arg_i("type", 1))],
                     ["x"], shape=shape)
        weights, feed = bn_data(shape)
        run_all(net, weights, feed, ["x"], expect_fused=["bn(BatchNorm) + sc(Scale) + relu(Activate) -> x"])


def test_batch_norm_scale_falls_back_where_the_parameters_are_not_one_per_channel(gpu):
    """Scale parameters over two axes: the group exists (shapes are not known when the network is
    built), declines at run time, and the operators run one by one."""
    shape = (2, 4, 6, 8)
    net = bn_net([bn_op("x", "n"), scale_op("n", "s", name="sc")], ["s"], shape=shape, scale_param_shape=[4, 6])
    weights, feed = bn_data(shape, scale_param_shape=[4, 6])
    run_all(net, weights, feed, ["s"], expect_fused=["bn(BatchNorm) + sc(Scale) -> s"])


def test_batch_norm_output_with_another_reader_is_not_fused(gpu):
    net = bn_net([bn_op("x", "n"), scale_op("n", "s", name="sc"), op("Activate", "relu", ["s"], ["y"], arg_i("type", 1)),
                  op("Unary", "neg", ["n"], ["out"], arg_i("operation", 13))], ["y", "out"])
    weights, feed = bn_data()
    # the normalised blob is read again: BatchNorm stays; Scale -> ReLU still goes together
    run_all(net, weights, feed, ["n", "y", "out"], expect_fused=["sc(Scale) + relu(Activate) -> y"])


@pytest.mark.parametrize("shape", [SHAPE, (2, 8, 4, 8), (5, 3, 1, 1)])
@pytest.mark.parametrize("residual_first", [False, True])
@pytest.mark.parametrize("factor", [None, 999.982])
def test_batch_norm_in_front_of_a_residual_tail_goes_with_it(gpu, shape, residual_first, factor):
    """The last normalisation of a Caffe-style bottleneck: BatchNorm -> Scale -> Eltwise -> ReLU -> mean."""
    ops = [bn_op("x", "n", factor is not None), scale_op("n", "s", name="sc"),
           op("Eltwise", "add", ["r", "s"] if residual_first else ["s", "r"], ["e"], arg_i("operation", 1)),
           op("Activate", "relu", ["e"], ["e"], arg_i("type", 1)),
           op("Reduce", "gap", ["e"], ["pool"], arg_i("operation", 4), ("axes", "v_i", [2, 3]))]
    net = bn_net(ops, ["e", "pool"], shape=shape, factor=factor is not None)
    net["op"][0] = op("Input", "in", [], ["x", "r"], ("x", "v_i", list(shape)), ("r", "v_i", list(shape)))
    weights, feed = bn_data(shape, factor=factor)
    feed = {"x": normal(51, shape, 2.0), "r": normal(52, shape)}
    run_all(net, weights, feed, ["e", "pool"], fp64=("pool",),
            expect_fused=["bn(BatchNorm) + sc(Scale) + add(Eltwise) + relu(Activate) + gap(Reduce) -> e, pool"])


def test_batch_norm_in_front_of_a_residual_tail_in_place_and_with_special_values(gpu):
    """One blob name from the BatchNorm to the Scale, as Caffe writes it; the residual is the block's input."""
    ops = [op("Unary", "branch", ["x"], ["t"], arg_i("operation", 13)),
           bn_op("t", "t"), scale_op("t", "t", name="sc"),
           op("Eltwise", "add", ["x", "t"], ["e"], arg_i("operation", 1)),
           op("Activate", "relu", ["e"], ["e"], arg_i("type", 1))]
    net = bn_net(ops, ["e"])
    weights, feed = bn_data()
    run_all(net, weights, feed, ["e"], expect_fused=["bn(BatchNorm) + sc(Scale) + add(Eltwise) + relu(Activate) -> e"])


def test_batch_norm_whose_output_is_read_again_stays_out_of_the_tail(gpu):
    ops = [bn_op("x", "n"), scale_op("n", "s", name="sc"),
           op("Eltwise", "add", ["s", "x"], ["e"], arg_i("operation", 1)),
           op("Activate", "relu", ["e"], ["e"], arg_i("type", 1)),
           op("Unary", "neg", ["n"], ["out"], arg_i("operation", 13))]
    net = bn_net(ops, ["e", "out"])
    weights, feed = bn_data()
    run_all(net, weights, feed, ["n", "e", "out"], expect_fused=["sc(Scale) + add(Eltwise) + relu(Activate) -> e"])


def test_tail_behind_a_batch_norm_falls_back_where_the_scale_is_not_per_channel(gpu):
    shape = (2, 4, 6, 8)
    ops = [bn_op("x", "n"), scale_op("n", "s", name="sc"),
           op("Eltwise", "add", ["s", "x"], ["e"], arg_i("operation", 1)),
           op("Activate", "relu", ["e"], ["e"], arg_i("type", 1))]
    net = bn_net(ops, ["e"], shape=shape, scale_param_shape=[4, 6])
    weights, feed = bn_data(shape, scale_param_shape=[4, 6])
    run_all(net, weights, feed, ["e"], expect_fused=["bn(BatchNorm) + sc(Scale) + add(Eltwise) + relu(Activate) -> e"])


def test_batch_norm_scale_in_front_of_a_sum_without_relu(gpu):
    """No tail to leave the Scale to: it goes with its BatchNorm."""
    ops = [bn_op("x", "n"), scale_op("n", "s", name="sc"),
           op("Eltwise", "add", ["s", "x"], ["e"], arg_i("operation", 1))]
    net = bn_net(ops, ["e"])
    weights, feed = bn_data()
    run_all(net, weights, feed, ["s", "e"], expect_fused=["bn(BatchNorm) + sc(Scale) -> s"])
