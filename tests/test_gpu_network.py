"""Whole graphs through Network / Native (text model in, host inputs in, blobs
out) against oracle.net.run, which applies the operator-level oracle functions
in file order.  Every operator of these graphs is bit-exact on its own, and
the graphs must be too, except downstream of the fp64-accumulating operators
(Reduce sum/avg, Group/LayerNorm), where the 1e-5 contract applies and the
observed difference is zero."""
import numpy as np
import pytest

import shadow_amd
from oracle import net as onet
from shadow_amd import ShadowError
from tests.helpers import assert_bit_exact, assert_rel_close, normal, uniform

pytestmark = pytest.mark.gpu
F = np.float32


def arg_i(name, v):
    return (name, "s_i", int(v))


def op(typ, name, bottom, top, *args):
    return {"type": typ, "name": name, "bottom": list(bottom), "top": list(top), "arg": list(args)}


def resnet_tail(n=4, c=16, hw=7):
    net = {"name": "tail", "arg": [("out_blob", "v_s", ["prob", "feat"])],
           "blob": [("bn_scale", "float", [c]), ("bn_bias", "float", [c]), ("gate", "float", [1, c, 1, 1])],
           "op": [
               op("Input", "data", [], ["data", "skip"], ("data", "v_i", [n, c, hw, hw]), ("skip", "v_i", [n, c, hw, hw])),
               op("Scale", "bn", ["data", "bn_scale", "bn_bias"], ["bn_out"], arg_i("axis", 1), arg_i("has_scale", 1),
                  arg_i("has_bias", 1)),
               op("Eltwise", "add", ["bn_out", "skip"], ["sum"], arg_i("operation", 1)),
               op("Activate", "relu", ["sum"], ["sum"], arg_i("type", 1)),
               op("Binary", "gate", ["sum", "gate"], ["feat"], arg_i("operation", 2)),
               op("Pooling", "gap", ["feat"], ["pooled"], arg_i("pool", 1), arg_i("global_pooling", 1)),
               op("Flatten", "flat", ["pooled"], ["flat"], arg_i("axis", 1)),
               op("Softmax", "prob", ["flat"], ["prob"], arg_i("axis", 1)),
           ]}
    weights = [uniform(1, c, 0.5, 1.5), normal(2, c, 0.2), uniform(3, (1, c, 1, 1), 0.0, 1.0)]
    inputs = {"data": normal(4, (n, c, hw, hw), 2.0), "skip": normal(5, (n, c, hw, hw))}
    return net, weights, inputs


def mixed_graph():
    n, c, h, w = 3, 8, 10, 12
    net = {"name": "mixed", "arg": [("out_blob", "v_s", ["out"]), ("note", "s_s", "x")],
           "blob": [("mean", "float", [c]), ("var", "float", [c]), ("factor", "float", [1]), ("ln_s", "float", [w]),
                    ("ln_b", "float", [w]), ("alpha", "float", [n, c])],
           "op": [
               op("Input", "in", [], ["x"], ("x", "v_i", [n, c, h, w])),
               op("BatchNorm", "bn", ["x", "mean", "var", "factor"], ["bn"], ("eps", "s_f", F(1e-3))),
               op("Pooling", "pool", ["bn"], ["p"], arg_i("pool", 0), ("kernel_size", "v_i", [3]), ("stride", "v_i", [2]),
                  ("pad", "v_i", [1]), arg_i("full_pooling", 0)),
               op("LRN", "lrn", ["p"], ["lr"], arg_i("local_size", 3), ("alpha", "s_f", F(1e-2)), ("beta", "s_f", F(0.75))),
               op("Unary", "abs", ["p"], ["pa"], arg_i("operation", 0)),
               op("Unary", "sqrt", ["pa"], ["ps"], arg_i("operation", 2)),
               op("Reshape", "rs", ["ps"], ["r"], ("shape", "v_i", [0, -1, 6])),
               op("Unsqueeze", "us", ["r"], ["u"], ("axes", "v_i", [1])),
               op("Squeeze", "sq", ["u"], ["s"], ("axes", "v_i", [1])),
               op("Normalize", "l2", ["s"], ["nz"], ("p", "s_f", F(2.0)), arg_i("axis", 1)),
               op("Reduce", "max", ["nz"], ["rmax"], arg_i("operation", 2), ("axes", "v_i", [2]), arg_i("keep_dims", 0)),
               op("LayerNorm", "ln", ["x", "ln_s", "ln_b"], ["ln"], ("normalized_shape", "v_i", [w])),
               op("Activate", "tanh", ["ln"], ["ln"], arg_i("type", 5)),
               op("Axpy", "axpy", ["alpha", "ln", "x"], ["ax"]),
               op("InstanceNorm", "inorm", ["ax"], ["inn"]),
               op("Reduce", "avg", ["inn"], ["ravg"], arg_i("operation", 4), ("axes", "v_i", [2, 3])),
               op("Flatten", "f1", ["ravg"], ["favg"]),
               op("Flatten", "f2", ["rmax"], ["fmax"]),
               op("Scale", "sc", ["fmax"], ["fms"], arg_i("axis", 1), ("scale_value", "v_f", [F(0.5)]),
                  ("bias_value", "v_f", [F(0.25)])),
               op("Softmax", "sm", ["fms"], ["out"], arg_i("axis", -1)),
           ]}
    weights = [normal(6, c), uniform(7, c, 0.2, 3.0), F([0.999]), uniform(8, w, 0.5, 1.5), normal(9, w, 0.1),
               uniform(10, (n, c), -1.0, 1.0)]
    inputs = {"x": normal(11, (n, c, h, w), 1.5)}
    return net, weights, inputs


FP64_SUM_DOWNSTREAM = {"ln", "ax", "inn", "ravg", "favg"}


def compare(nw, want, names):
    for name in names:
        got = nw.blob(name)
        assert list(got.shape) == list(want[name].shape), name
        if name in FP64_SUM_DOWNSTREAM:
            assert assert_rel_close(got, want[name], 1e-5, name) == 0
        else:
            assert_bit_exact(got, want[name], name)


def test_resnet_tail_graph(gpu):
    net, weights, inputs = resnet_tail()
    want = onet.run(net, weights, inputs)
    with shadow_amd.Network(onet.write_text(net), weights, fuse=False) as nw:
        assert nw.fused == []
        nw.forward(inputs)
        compare(nw, want, ["bn_out", "sum", "feat", "pooled", "flat", "prob"])
    with shadow_amd.Network(onet.write_text(net), weights) as nw:
        assert nw.in_blob == ["data", "skip"] and nw.out_blob == ["prob", "feat"]
        assert nw.blob_shape("data") == [4, 16, 7, 7]
        # Scale, Eltwise and the in-place relu run as one launch; bn_out, which only the Eltwise reads, is not written
        assert nw.fused == ["bn(Scale) + add(Eltwise) + relu(Activate) -> sum"]
        nw.forward(inputs)
        compare(nw, want, ["sum", "feat", "pooled", "flat", "prob"])
        # a second pass over the same network gives the same bits
        first = nw.blob("prob").copy()
        nw.forward(inputs)
        assert_bit_exact(nw.blob("prob"), first, "second pass")


def test_mixed_graph(gpu):
    net, weights, inputs = mixed_graph()
    want = onet.run(net, weights, inputs)
    with shadow_amd.Network(onet.write_text(net), weights, debug=True) as nw:
        nw.forward(inputs)
        compare(nw, want, ["bn", "p", "lr", "ps", "r", "u", "s", "nz", "rmax", "ln", "ax", "inn", "ravg", "favg", "fmax",
                           "fms", "out"])
        assert nw.blob_shape("r") == [3, 40, 6] and nw.blob_shape("u") == [3, 1, 40, 6]


def test_binary_models_with_embedded_weights(gpu):
    """The same graphs from serialized NetParam / MetaNetParam bytes whose blobs
    carry their contents (python-protobuf writes them, the C++ reader decodes
    them): every blob as from the text form with separate weights."""
    from tests import shadow_proto as sp
    net, weights, inputs = resnet_tail()
    want = onet.run(net, weights, inputs)
    wire = sp.from_oracle_net(net, weights).SerializeToString()
    with shadow_amd.Network.from_binary(wire, fuse=False) as nw:
        assert nw.in_blob == ["data", "skip"] and nw.out_blob == ["prob", "feat"]
        nw.forward(inputs)
        compare(nw, want, ["bn_out", "sum", "feat", "pooled", "flat", "prob"])
    with shadow_amd.Network.from_binary(wire) as nw:
        assert len(nw.fused) == 1
        nw.forward(inputs)
        compare(nw, want, ["sum", "feat", "pooled", "flat", "prob"])
    net2, weights2, inputs2 = mixed_graph()
    meta = sp.MetaNetParam()
    meta.name = "two networks"
    meta.network.add().CopyFrom(sp.from_oracle_net(net, weights))
    meta.network.add().CopyFrom(sp.from_oracle_net(net2, weights2))
    want2 = onet.run(net2, weights2, inputs2)
    with shadow_amd.Network.from_binary(meta.SerializeToString(), network_index=1) as nw:
        nw.forward(inputs2)
        compare(nw, want2, ["bn", "p", "nz", "rmax", "ln", "ax", "inn", "ravg", "fms", "out"])
    # a blob whose contents do not match its shape is refused (native.cpp:155)
    bad = sp.from_oracle_net(net, weights)
    bad.blob[0].data_f.append(1.0)
    with pytest.raises(ShadowError, match="Check Failed"):
        shadow_amd.Network.from_binary(bad.SerializeToString())
    with pytest.raises(ShadowError, match="Error when loading proto"):
        shadow_amd.Network.from_binary(wire[:-3])


def test_inputs_can_be_reshaped_per_call(gpu):
    net, weights, _ = resnet_tail()
    with shadow_amd.Network(onet.write_text(net), weights) as nw:
        for n in (2, 6, 1):
            inputs = {"data": normal(20 + n, (n, 16, 7, 7), 2.0), "skip": normal(30 + n, (n, 16, 7, 7))}
            nw.forward(inputs, reshape=True)
            want = onet.run(net, weights, inputs)
            compare(nw, want, ["feat", "pooled", "prob"])
            assert nw.blob_shape("prob") == [n, 16]


def test_global_pooling_keeps_the_first_plane_size(gpu):
    # The reference's PoolingOp records the plane extents on its first run
    # (shadow/operators/pooling_op.cpp:63-67); a later, larger input is pooled
    # with that stale window.  Kept as it is: same outputs as the reference.
    net = {"name": "gap", "arg": [("out_blob", "v_s", ["y"])], "blob": [],
           "op": [op("Input", "in", [], ["x"], ("x", "v_i", [1, 2, 4, 4])),
                  op("Pooling", "gap", ["x"], ["y"], arg_i("pool", 1), arg_i("global_pooling", 1))]}
    stale = {"name": "gap", "arg": net["arg"], "blob": [],
             "op": [net["op"][0], op("Pooling", "gap", ["x"], ["y"], arg_i("pool", 1), ("kernel_size", "v_i", [4]))]}
    with shadow_amd.Network(onet.write_text(net)) as nw:
        small, large = normal(50, (1, 2, 4, 4)), normal(51, (1, 2, 8, 8))
        nw.forward({"x": small}, reshape=True)
        assert_bit_exact(nw.blob("y"), onet.run(net, [], {"x": small})["y"], "first run")
        nw.forward({"x": large}, reshape=True)
        assert nw.blob_shape("y") == [1, 2, 5, 5]
        assert_bit_exact(nw.blob("y"), onet.run(stale, [], {"x": large})["y"], "stale window")


def test_loading_errors(gpu):
    net, weights, _ = resnet_tail()
    text = onet.write_text(net)
    with pytest.raises(ShadowError, match="out_blob"):
        shadow_amd.Network(onet.write_text(dict(net, arg=[])), weights)
    with pytest.raises(ShadowError, match="not registered"):
        shadow_amd.Network(text.replace("[Softmax]", "[Softmin]"), weights)
    with pytest.raises(ShadowError, match="not registered"):
        shadow_amd.Network(text, weights, backend_type="TensorRT")
    with pytest.raises(ShadowError):
        shadow_amd.Network(text, weights, backend_type="")
    two_inputs = dict(net, op=[net["op"][0]] + net["op"])
    with pytest.raises(ShadowError, match="Check Failed"):
        shadow_amd.Network(onet.write_text(two_inputs), weights)
    with pytest.raises(ShadowError):
        shadow_amd.Network("", weights)


def test_running_errors(gpu):
    net, weights, inputs = resnet_tail()
    dangling = dict(net, op=net["op"][:-1] + [op("Softmax", "prob", ["nowhere"], ["prob"])])
    with shadow_amd.Network(onet.write_text(dangling), weights) as nw:
        with pytest.raises(ShadowError, match="Can not find input blob nowhere"):
            nw.forward(inputs)
    with shadow_amd.Network(onet.write_text(net), weights) as nw:
        with pytest.raises(ShadowError, match="Can not find blob"):
            nw.forward({"other": inputs["data"]})
        with pytest.raises(ShadowError, match="Unknown blob"):
            nw.blob("missing")
