"""The model text form and the view-only shape rules, without a GPU: pins for the
Python restatement (oracle/net.py) and the C++ parser against it.

The reference ships no model in this form; the pins are a text written out by
hand from the converter's format strings
(shadow/python/converter/shadow/transformer.py:30-65), the write -> parse round
trip, and numpy.reshape for the shape rules."""
import numpy as np
import pytest

import oracle
import shadow_amd
from oracle import net as onet
from shadow_amd import ShadowError

F = np.float32

HAND_WRITTEN = (
    "[resnet_tail]\n"
    "[{out_blob, v_s, [prob # feat]}; {share_weight, s_i, [0]}; {scale, s_f, [0.017]}; {tag, s_s, [v1]}]\n"
    "[{bn_scale, float, [8]}; {bn_bias, float, [8]}; {idx, int, [2 # 2]}]\n"
    "[Input] | [data] | [0 1 1] | [] | [data] | [{data, v_i, [2 # 8 # 6 # 6]}]\n"
    "[Scale] | [bn] | [3 1 3] | [data; bn_scale; bn_bias] | [bn_out] | "
    "[{axis, s_i, [1]}; {has_scale, s_i, [1]}; {has_bias, s_i, [1]}]\n"
    "[Activate] | [relu] | [1 1 2] | [bn_out] | [bn_out] | [{type, s_i, [1]}; {slope, s_f, [0.1]}]\n"
    "[Eltwise] | [sum] | [2 1 2] | [bn_out; data] | [feat] | [{operation, s_i, [1]}; {coeff, v_f, [1.0 # -0.5]}]\n"
    "[Pooling] | [gap] | [1 1 2] | [feat] | [pooled] | [{pool, s_i, [1]}; {global_pooling, s_i, [1]}]\n"
    "[Flatten] | [flat] | [1 1 0] | [pooled] | [flat_out] | []\n"
    "[Softmax] | [prob] | [1 1 1] | [flat_out] | [prob] | [{axis, s_i, [1]}]\n")


def test_hand_written_text_parses_to_the_known_structure():
    net = onet.parse_text(HAND_WRITTEN)
    assert net["name"] == "resnet_tail"
    assert net["arg"] == [("out_blob", "v_s", ["prob", "feat"]), ("share_weight", "s_i", 0),
                          ("scale", "s_f", F(0.017)), ("tag", "s_s", "v1")]
    assert net["blob"] == [("bn_scale", "float", [8]), ("bn_bias", "float", [8]), ("idx", "int", [2, 2])]
    assert [o["type"] for o in net["op"]] == ["Input", "Scale", "Activate", "Eltwise", "Pooling", "Flatten", "Softmax"]
    assert net["op"][0] == {"type": "Input", "name": "data", "bottom": [], "top": ["data"],
                            "arg": [("data", "v_i", [2, 8, 6, 6])]}
    assert net["op"][1]["bottom"] == ["data", "bn_scale", "bn_bias"]
    assert net["op"][3]["arg"] == [("operation", "s_i", 1), ("coeff", "v_f", [F(1.0), F(-0.5)])]
    assert net["op"][5]["arg"] == [] and net["op"][5]["top"] == ["flat_out"]


def test_write_parse_round_trip():
    net = onet.parse_text(HAND_WRITTEN)
    assert onet.parse_text(onet.write_text(net)) == net
    # the writer reproduces the converter's spelling for this net exactly
    # (floats print through str(), as in the converter)
    respelt = onet.write_text(net)
    assert respelt.splitlines()[0] == "[resnet_tail]"
    assert respelt.splitlines()[3] == HAND_WRITTEN.splitlines()[3]
    assert respelt.splitlines()[8] == "[Flatten] | [flat] | [1 1 0] | [pooled] | [flat_out] | []"


def test_cpp_parser_agrees_with_the_restatement():
    for text in (HAND_WRITTEN, onet.write_text(onet.parse_text(HAND_WRITTEN))):
        canonical = shadow_amd.parse_net(text)
        assert onet.parse_text(canonical) == onet.parse_text(text)
        # canonical form is a fixed point of the C++ reader/writer
        assert shadow_amd.parse_net(canonical) == canonical


def test_cpp_parser_keeps_every_fp32_value():
    values = [0.1, 1e-5, 1e-12, 3.4028235e38, 1.17549435e-38, 1e-45, -0.0, 16777217.0, 0.017]
    net = {"name": "n", "arg": [("out_blob", "v_s", ["y"]), ("eps", "s_f", F(1e-5))], "blob": [],
           "op": [{"type": "Scale", "name": "s", "bottom": ["x"], "top": ["y"],
                   "arg": [("scale_value", "v_f", [F(v) for v in values])]}]}
    back = onet.parse_text(shadow_amd.parse_net(onet.write_text(net)))
    got = back["op"][0]["arg"][0][2]
    assert [np.float32(v).tobytes() for v in got] == [np.float32(v).tobytes() for v in values]
    assert back["arg"][1][2] == F(1e-5)


@pytest.mark.parametrize("bad", [
    "", "[n]\n[]\n", "[n]\n[]\n[]\n[Unary] | [u] | [1 1 1] | [x] | [y]\n",
    "[n]\n[]\n[]\n[Unary] | [u] | [1 1 1] | [x] | [y] | [{operation, s_q, [1]}]\n",
    "[n]\n[]\n[]\n[Unary] | [u] | [1 1 1] | [x] | [y] | [{operation, s_i, [one]}]\n",
    "[n]\n[]\n[{w, float}]\n", "[n]\n[{a, s_i, 1}]\n[]\n",
    "[n]\n[]\n[]\n[Unary] | [u] | [2 1 0] | [x] | [y] | []\n",
])
def test_cpp_parser_rejects_malformed_text(bad):
    with pytest.raises(ShadowError):
        shadow_amd.parse_net(bad)


# ------------------------------------------------------------ shape rules ---
@pytest.mark.parametrize("in_shape,shape,axis,num_axes,want", [
    ((2, 3, 4, 5), [0, -1], 0, -1, [2, 60]), ((2, 3, 4, 5), [6, 20], 0, -1, [6, 20]),
    ((2, 3, 4, 5), [0, 0, -1], 0, -1, [2, 3, 20]), ((2, 3, 4, 5), [12], 1, 2, [2, 12, 5]),
    ((2, 3, 4, 5), [2, 2], 2, 1, [2, 3, 2, 2, 5]), ((2, 3, 4, 5), [-1], -2, -1, [2, 3, 20]),
    ((6,), [2, 0], 0, 0, None), ((2, 3, 4), [5, -1], 0, -1, None), ((2, 3, 4), [-1, -1], 0, -1, None),
    ((2, 3, 4), [7], 0, -1, None),
])
def test_reshape_rule(in_shape, shape, axis, num_axes, want):
    if want is None:
        with pytest.raises(oracle.OracleCheckError):
            onet.reshape_shape(in_shape, shape, axis, num_axes)
        return
    got = onet.reshape_shape(in_shape, shape, axis, num_axes)
    assert got == want
    assert np.arange(np.prod(in_shape)).reshape(in_shape).reshape(got).shape == tuple(want)


def test_flatten_squeeze_unsqueeze_rules():
    assert onet.flatten_shape((2, 3, 4, 5)) == [2, 60]
    assert onet.flatten_shape((2, 3, 4, 5), 0, 1) == [6, 4, 5]
    assert onet.flatten_shape((2, 3, 4, 5), 2, 2) == [2, 3, 4, 5]
    assert onet.flatten_shape((7,), 0) == [7]
    assert onet.squeeze_shape((2, 1, 3, 1)) == [2, 3]
    assert onet.squeeze_shape((2, 1, 3, 1), [1]) == [2, 3, 1]
    assert onet.squeeze_shape((1, 1), []) == []
    assert onet.unsqueeze_shape((2, 3), [0, 3]) == [1, 2, 3, 1]
    assert onet.unsqueeze_shape((2, 3), [-1]) == [2, 3, 1]
    assert onet.unsqueeze_shape((2, 3), [1]) == [2, 1, 3]
    for bad in (lambda: onet.flatten_shape((2, 3), 2), lambda: onet.flatten_shape((2, 3), 1, 0),
                lambda: onet.squeeze_shape((2, 3), [0]), lambda: onet.unsqueeze_shape((2, 3), [5])):
        with pytest.raises(oracle.OracleCheckError):
            bad()


def test_native_backend_is_registered():
    lib = shadow_amd.host()
    import ctypes
    buf = ctypes.create_string_buffer(256)
    lib.shdw_host_backend_keys(buf, 256)
    assert buf.value.decode().split("\n") == ["Native"]
