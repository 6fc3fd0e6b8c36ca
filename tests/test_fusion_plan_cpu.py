"""The fusion pass's matcher on the CPU: which operators of a text model go into one
launch is decided from the operators' parameters alone (`shdw_host_plan_fusion`,
the planner `Native::Initial` runs), so every pattern and every condition that
keeps an operator out of a group can be pinned without a device.  What the
groups compute is the GPU suite's business (tests/test_gpu_fusion.py runs these
same networks fused, unfused and through the oracle)."""
import numpy as np
import pytest

import shadow_amd
from oracle import net as onet
from tests.test_gpu_fusion import (ADD_RELU, BLOCKED, TAIL, arg_i, bn_net, bn_op, make, op, scale_op, tail_ops)

F = np.float32


def plan(net):
    return shadow_amd.plan_fusion(onet.write_text(net))


def relu(bottom, top, name="relu"):
    return op("Activate", name, [bottom], [top], arg_i("type", 1))


def neg(bottom, top, name="neg"):
    return op("Unary", name, [bottom], [top], arg_i("operation", 13))


# ---- Scale -> ReLU ----
@pytest.mark.parametrize("top", ["s", "y"])
@pytest.mark.parametrize("has_scale,has_bias", [(True, True), (True, False), (False, True)])
def test_scale_relu(top, has_scale, has_bias):
    params = (["gamma"] if has_scale else []) + (["beta"] if has_bias else [])
    net = make([scale_op("x", "s", has_scale, has_bias), relu("s", top), neg(top, "out")], ["out"], params=params)
    assert plan(net) == ["bn(Scale) + relu(Activate) -> " + top]


def test_scale_relu_needs_the_scale_output_to_itself():
    # not in place and the Scale output is read again, or handed out: the Scale has to write it
    assert plan(make([scale_op("x", "s"), relu("s", "y"), neg("s", "out")], ["y", "out"])) == []
    assert plan(make([scale_op("x", "s"), relu("s", "y")], ["s", "y"])) == []
    # in place, later readers see the activated values either way
    assert plan(make([scale_op("x", "s"), relu("s", "s"), neg("s", "out")], ["s", "out"])) == [
        "bn(Scale) + relu(Activate) -> s"]
    # parameters as host values: staged on every run, left alone
    host_values = op("Scale", "sc", ["x"], ["s"], arg_i("axis", 1), ("scale_value", "v_f", [F(0.5)]))
    assert plan(make([host_values, relu("s", "s")], ["s"], params=())) == []
    # leaky relu is another function
    assert plan(make([scale_op("x", "s"), op("Activate", "act", ["s"], ["s"], arg_i("type", 2))], ["s"])) == []


# ---- Scale -> Eltwise -> ReLU [-> Reduce] ----
@pytest.mark.parametrize("residual_first", [False, True])
@pytest.mark.parametrize("keep_dims", [True, False])
def test_residual_tail(residual_first, keep_dims):
    net = make(tail_ops(residual_first=residual_first, keep_dims=keep_dims), ["e", "pool"], inputs=("x", "r"))
    assert plan(net) == TAIL
    assert plan(make(tail_ops()[:3], ["e"], inputs=("x", "r"))) == ["bn(Scale) + add(Eltwise) + relu(Activate) -> e"]
    assert plan(make(tail_ops(relu_top="a", scale_top="x"), ["a", "pool"], inputs=("x", "r"))) == [
        "bn(Scale) + add(Eltwise) + relu(Activate) + gap(Reduce) -> a, pool"]


def test_residual_tail_takes_any_axes_and_leaves_the_shapes_to_the_run():
    for axes in ([3], [1, 2, 3], [0], []):
        assert plan(make(tail_ops(axes=axes), ["e", "pool"], inputs=("x", "r"))) == TAIL


def test_operators_between_the_members():
    ops = tail_ops()
    ops.insert(1, op("Unary", "abs", ["r"], ["m"], arg_i("operation", 0)))  # reads an input of the group
    assert plan(make(ops, ["m", "pool"], inputs=("x", "r"))) == TAIL
    ops = tail_ops()
    ops.insert(3, op("Unary", "abs", ["e"], ["m"], arg_i("operation", 0)))  # reads what the group writes
    assert plan(make(ops, ["m", "pool"], inputs=("x", "r"))) == ["bn(Scale) + add(Eltwise) + relu(Activate) -> e"]


@pytest.mark.parametrize("why", sorted(BLOCKED))
def test_blocked(why):
    ops, out, _, groups = BLOCKED[why]
    assert plan(make(ops, out, inputs=("x", "r"))) == groups


# ---- Eltwise -> ReLU ----
@pytest.mark.parametrize("operation", [0, 1, 2, 3])
@pytest.mark.parametrize("inputs", [2, 3, 9])
def test_eltwise_relu(operation, inputs):
    names = ["x%d" % k for k in range(inputs)]
    for top in ("e", "a"):
        net = make([op("Eltwise", "add", names, ["e"], arg_i("operation", operation)), relu("e", top)], [top],
                   inputs=names, params=())
        assert plan(net) == ["add(Eltwise) + relu(Activate) -> " + top]


def test_eltwise_relu_is_left_alone():
    # the output among the inputs: cleared before it is read
    in_place = [op("Eltwise", "add", ["x", "r"], ["x"], arg_i("operation", 1)), relu("x", "x")]
    assert plan(make(in_place, ["x"], inputs=("x", "r"), params=())) == []
    # the sum is wanted as it is
    kept = [op("Eltwise", "add", ["x", "r"], ["e"], arg_i("operation", 1)), relu("e", "a")]
    assert plan(make(kept, ["e", "a"], inputs=("x", "r"), params=())) == []
    assert plan(make(kept, ["a"], inputs=("x", "r"), params=())) == ["add(Eltwise) + relu(Activate) -> a"]
    # an operation the operator does not know
    bad = [op("Eltwise", "add", ["x", "r"], ["e"], arg_i("operation", 4)), relu("e", "e")]
    assert plan(make(bad, ["e"], inputs=("x", "r"), params=())) == []


# ---- BatchNorm -> Scale [-> ReLU] ----
@pytest.mark.parametrize("names", [("x", "x", "x"), ("n", "s", "y"), ("n", "n", "n"), ("x", "s", "s")])
@pytest.mark.parametrize("with_relu", [False, True])
@pytest.mark.parametrize("factor", [False, True])
def test_batch_norm_scale(names, with_relu, factor):
    n, s, y = names
    ops = [bn_op("x", n, factor), scale_op(n, s, name="sc")] + ([relu(s, y)] if with_relu else [])
    last = y if with_relu else s
    net = bn_net(ops + [neg(last, "out")], ["out"], factor=factor)
    assert plan(net) == ["bn(BatchNorm) + sc(Scale)" + (" + relu(Activate)" if with_relu else "") + " -> " + last]


def test_batch_norm_scale_is_left_alone():
    # the normalised values are read again: BatchNorm stays, Scale -> ReLU still goes together
    ops = [bn_op("x", "n"), scale_op("n", "s", name="sc"), relu("s", "y"), neg("n", "out")]
    assert plan(bn_net(ops, ["y", "out"])) == ["sc(Scale) + relu(Activate) -> y"]
    # ... or handed out
    assert plan(bn_net(ops[:3], ["n", "y"])) == ["sc(Scale) + relu(Activate) -> y"]
    # the normalised blob is the Scale's parameter, not its data
    as_parameter = op("Scale", "sc", ["x", "n"], ["s"], arg_i("axis", 1), arg_i("has_scale", 1), arg_i("has_bias", 0))
    assert plan(bn_net([bn_op("x", "n"), as_parameter], ["s"])) == []
    # BatchNorm with two inputs is not the stored-statistics form
    short = op("BatchNorm", "bn", ["x", "mean"], ["n"])
    assert plan(bn_net([short, scale_op("n", "s", name="sc")], ["s"])) == []
    # the activated values go elsewhere and the scaled ones are wanted too: the ReLU stays out
    ops = [bn_op("x", "n"), scale_op("n", "s", name="sc"), relu("s", "y")]
    assert plan(bn_net(ops, ["s", "y"])) == ["bn(BatchNorm) + sc(Scale) -> s"]
    # something between the two rewrites the statistics
    ops = [bn_op("x", "n"), neg("mean", "mean"), scale_op("n", "s", name="sc")]
    assert plan(bn_net(ops, ["s"])) == []


# ---- BatchNorm -> Scale -> Eltwise -> ReLU [-> Reduce] ----
def bn_tail(residual="x", mean=True, bn_top="n", scale_top="s"):
    ops = [bn_op("t", bn_top), scale_op(bn_top, scale_top, name="sc"),
           op("Eltwise", "add", [scale_top, residual], ["e"], arg_i("operation", 1)), relu("e", "e")]
    if mean:
        ops.append(op("Reduce", "gap", ["e"], ["pool"], arg_i("operation", 4), ("axes", "v_i", [2, 3])))
    return [neg("x", "t", "branch")] + ops


def test_batch_norm_joins_the_tail_behind_it():
    assert plan(bn_net(bn_tail(), ["e", "pool"])) == [
        "bn(BatchNorm) + sc(Scale) + add(Eltwise) + relu(Activate) + gap(Reduce) -> e, pool"]
    assert plan(bn_net(bn_tail(mean=False), ["e"])) == ["bn(BatchNorm) + sc(Scale) + add(Eltwise) + relu(Activate) -> e"]
    # one blob name from the branch to the sum, as Caffe writes it
    assert plan(bn_net(bn_tail(bn_top="t", scale_top="t", mean=False), ["e"])) == [
        "bn(BatchNorm) + sc(Scale) + add(Eltwise) + relu(Activate) -> e"]


def test_batch_norm_stays_out_of_the_tail():
    # its output is read again
    ops = bn_tail(mean=False) + [neg("n", "out")]
    assert plan(bn_net(ops, ["e", "out"])) == ["sc(Scale) + add(Eltwise) + relu(Activate) -> e"]
    # no ReLU behind the sum: no tail, the Scale goes with its BatchNorm
    ops = bn_tail(mean=False)[:-1]
    assert plan(bn_net(ops, ["e"])) == ["bn(BatchNorm) + sc(Scale) -> s"]
    # the Scale's input comes from another kind of operator
    ops = [neg("x", "n", "branch"), scale_op("n", "s", name="sc"),
           op("Eltwise", "add", ["s", "x"], ["e"], arg_i("operation", 1)), relu("e", "e")]
    assert plan(bn_net(ops, ["e"])) == ["sc(Scale) + add(Eltwise) + relu(Activate) -> e"]


# ---- several groups ----
def test_groups_come_in_the_order_of_their_last_members_and_share_no_operator():
    ops = [bn_op("x", "a"), scale_op("a", "a", name="sc1"), relu("a", "a", "relu1"),           # stem: bn + scale + relu
           bn_op("a", "b"), scale_op("b", "b", name="sc2"),                                      # branch
           op("Eltwise", "add", ["b", "a"], ["c"], arg_i("operation", 1)), relu("c", "c", "relu2"),  # ... closes a tail
           op("Eltwise", "mul", ["c", "a"], ["d"], arg_i("operation", 0)), relu("d", "d", "relu3")]
    ops[3]["name"] = "bn2"
    got = plan(bn_net(ops, ["d"]))
    assert got == ["bn(BatchNorm) + sc1(Scale) + relu1(Activate) -> a",
                   "bn2(BatchNorm) + sc2(Scale) + add(Eltwise) + relu2(Activate) -> c",
                   "mul(Eltwise) + relu3(Activate) -> d"]


def test_a_model_without_out_blob_is_refused():
    net = make([scale_op("x", "s"), relu("s", "s")], ["s"])
    net["arg"] = []
    with pytest.raises(shadow_amd.ShadowError, match="out_blob"):
        plan(net)
    assert plan(make([neg("x", "y")], ["y"], params=())) == []
