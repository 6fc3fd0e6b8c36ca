"""Binary model files (serialized shadow.NetParam / MetaNetParam) without a GPU.

The C++ reader and writer decode the protobuf wire format by hand; the
independent implementation they are checked against is python-protobuf on a
descriptor of the same five messages (tests/shadow_proto.py).  Checked both
ways: bytes written by python-protobuf are read by the C++ reader, and bytes
written by the C++ writer are parsed by python-protobuf back to the same message."""
import struct

import numpy as np
import pytest

import shadow_amd
from oracle import net as onet
from shadow_amd import ShadowError
from tests import shadow_proto as sp
from tests.test_net_cpu import HAND_WRITTEN

F = np.float32


def rich_net():
    """Every field of every message, awkward values included."""
    n = sp.NetParam()
    n.name = "net é"
    b = n.blob.add()
    b.name, b.type = "w", "float"
    b.shape.extend([2, 3])
    b.data_f.extend([0.0, -0.0, 1.5, -3.25e-30, 3.4e38, float("inf")])
    b = n.blob.add()
    b.name, b.type = "idx", "int32"
    b.shape.extend([4])
    b.data_i.extend([0, -1, 2147483647, -2147483648])
    b.data_b.append(np.arange(4, dtype=np.int32).tobytes())
    b = n.blob.add()          # no type: has_type() stays false, the reader's default applies
    b.name = "plain"
    b.shape.extend([1])
    o = n.op.add()
    o.type, o.name = "Input", "in"
    o.top.append("data")
    sp.add_arg(o, ("data", "v_i", [1, 3, 224, 224]))
    o = n.op.add()
    o.type, o.name = "Scale", "s"
    o.bottom.extend(["data", "w"])
    o.top.append("out")
    sp.add_arg(o, ("axis", "s_i", -1))
    sp.add_arg(o, ("eps", "s_f", 1e-5))
    sp.add_arg(o, ("mode", "s_s", "a;b | c"))
    sp.add_arg(o, ("coeff", "v_f", [1.0, -0.5, 1e-20]))
    sp.add_arg(o, ("names", "v_s", ["x", "", "y z"]))
    sp.add_arg(o, ("neg", "v_i", [-7, 0, 300, 1 << 30]))
    sp.add_arg(n, ("out_blob", "v_s", ["out"]))
    return n


def test_reader_and_writer_against_python_protobuf():
    n = rich_net()
    wire = n.SerializeToString()
    again = sp.NetParam()
    again.ParseFromString(shadow_amd.reencode_proto(wire))
    assert again == n
    # the writer emits the canonical encoding: same bytes as python-protobuf
    assert shadow_amd.reencode_proto(wire) == wire
    meta = sp.MetaNetParam()
    meta.name = "model"
    meta.network.add().CopyFrom(n)
    second = meta.network.add()
    second.name = "second"
    sp.add_arg(meta, ("version", "s_s", "1.2"))
    wire = meta.SerializeToString()
    again = sp.MetaNetParam()
    again.ParseFromString(shadow_amd.reencode_proto(wire, meta=True))
    assert again == meta
    assert shadow_amd.reencode_proto(wire, meta=True) == wire


def test_unpacked_packed_and_unknown_fields():
    def tag(field, wt):
        return bytes([(field << 3) | wt])

    def ld(field, payload):
        return tag(field, 2) + bytes([len(payload)]) + payload

    # Blob written the other way round: shape packed, data_f and data_i unpacked,
    # an unknown varint, 64-bit and length-delimited field in between
    blob = (ld(1, b"w") + ld(3, bytes([2, 3])) + tag(9, 0) + bytes([0x96, 0x01]) +
            tag(4, 5) + struct.pack("<f", 1.5) + tag(10, 1) + bytes(8) + tag(4, 5) + struct.pack("<f", -2.0) +
            ld(13, b"junk") + tag(5, 0) + bytes([0xff] * 9 + [0x01]) + tag(5, 0) + bytes([5]))
    wire = ld(1, b"n") + ld(5, blob) + tag(2, 0) + bytes([1])
    want = sp.NetParam()
    want.name = "n"
    b = want.blob.add()
    b.name = "w"
    b.shape.extend([2, 3])
    b.data_f.extend([1.5, -2.0])
    b.data_i.extend([-1, 5])
    got = sp.NetParam()
    got.ParseFromString(shadow_amd.reencode_proto(wire))
    assert got == want
    # python-protobuf reads the same bytes the same way (unknown fields aside)
    ref = sp.NetParam()
    ref.ParseFromString(wire)
    assert ref.blob[0].data_i == [-1, 5] and list(ref.blob[0].shape) == [2, 3]
    # a later optional value replaces the earlier one
    wire = ld(1, b"first") + ld(1, b"second")
    got.ParseFromString(shadow_amd.reencode_proto(wire))
    assert got.name == "second"


@pytest.mark.parametrize("cut", [1, 2, 5, 17, 40, -1, -3])
def test_truncated_input_is_refused(cut):
    wire = rich_net().SerializeToString()
    broken = wire[:cut]
    ref = sp.NetParam()
    try:
        ref.ParseFromString(broken)
        parses = True
    except Exception:
        parses = False
    if parses:   # a cut that happens to fall on a field boundary is a valid shorter message
        assert shadow_amd.reencode_proto(broken) == ref.SerializeToString()
    else:
        with pytest.raises(ShadowError, match="Error when loading proto"):
            shadow_amd.reencode_proto(broken)


def test_malformed_input_is_refused():
    for wire in (bytes([0x0b]),                 # group start: not used by these messages
                 bytes([0x00, 0x00]),           # field number 0
                 bytes([0x0a, 0x05, 0x61]),     # string longer than the message
                 bytes([0x80] * 11),            # varint that never ends
                 bytes([0x18, 0x01])):          # field 3 as a varint: unknown to NetParam, skipped
        try:
            out = shadow_amd.reencode_proto(wire)
            ok = True
        except ShadowError:
            ok = False
        ref = sp.NetParam()
        try:
            ref.ParseFromString(wire)
            ref_ok = True
        except Exception:
            ref_ok = False
        assert ok == ref_ok, wire.hex()
    # a known field with the wrong wire type: refused (python-protobuf keeps it as unknown; the
    # reference's generated C++ parser does the same, so this reader is the stricter one)
    with pytest.raises(ShadowError):
        shadow_amd.reencode_proto(bytes([0x08, 0x01]))   # NetParam.name as a varint


def test_text_form_and_binary_form_describe_the_same_net():
    text_net = onet.parse_text(HAND_WRITTEN.replace("{idx, int, [2 # 2]}", "{idx, int32, [2 # 2]}"))
    wire = sp.from_oracle_net(text_net).SerializeToString()
    canonical = shadow_amd.parse_net_binary(wire)
    assert onet.parse_text(canonical) == text_net
    assert canonical == shadow_amd.parse_net(onet.write_text(text_net))
    # and through a MetaNetParam, by index
    meta = sp.MetaNetParam()
    meta.network.add().name = "other"
    meta.network.add().CopyFrom(sp.from_oracle_net(text_net))
    assert shadow_amd.parse_net_binary(meta.SerializeToString(), 1) == canonical
    with pytest.raises(ShadowError, match="Check Failed"):
        shadow_amd.parse_net_binary(meta.SerializeToString(), 2)
    # text -> C++ writer -> python-protobuf
    got = sp.NetParam()
    got.ParseFromString(shadow_amd.serialize_net(onet.write_text(text_net)))
    assert got == sp.from_oracle_net(text_net)


def test_model_files(tmp_path):
    lib = shadow_amd.host()
    meta = sp.MetaNetParam()
    meta.name = "file model"
    meta.network.add().CopyFrom(rich_net())
    src, dst = tmp_path / "in.shadowmodel", tmp_path / "out.shadowmodel"
    src.write_bytes(meta.SerializeToString())
    assert lib.shdw_host_proto_file_reencode(str(src).encode(), str(dst).encode(), 1) == 0
    again = sp.MetaNetParam()
    again.ParseFromString(dst.read_bytes())
    assert again == meta
    # an absent file is a CHECK failure like the reference's "File not found"
    assert lib.shdw_host_proto_file_reencode(str(tmp_path / "absent").encode(), str(dst).encode(), 1) != 0
    assert "File not found" in lib.shdw_host_last_error().decode()
    src.write_bytes(meta.SerializeToString()[:-2])
    assert lib.shdw_host_proto_file_reencode(str(src).encode(), str(dst).encode(), 1) != 0


def test_random_nets_round_trip():
    """Seeded random messages of every shape the schema allows, both directions."""
    rng = np.random.default_rng(7)
    words = ["", "a", "conv1/out", "x y", "\u00e9\u4e2d", "blob_%d"]

    def word():
        w = words[rng.integers(len(words))]
        return w % rng.integers(100) if "%d" in w else w

    def fill_arg(a):
        a.name = word()
        kind = rng.integers(7)
        if kind == 0:
            a.s_f = float(np.float32(rng.normal() * 10.0 ** int(rng.integers(-30, 30))))
        elif kind == 1:
            a.s_i = int(rng.integers(-2 ** 31, 2 ** 31))
        elif kind == 2:
            a.s_s = word()
        elif kind == 3:
            a.v_f.extend(float(np.float32(v)) for v in rng.normal(size=rng.integers(0, 6)))
        elif kind == 4:
            a.v_i.extend(int(v) for v in rng.integers(-2 ** 31, 2 ** 31, size=rng.integers(0, 6)))
        elif kind == 5:
            a.v_s.extend(word() for _ in range(rng.integers(0, 4)))

    for _ in range(60):
        n = sp.NetParam()
        if rng.integers(2):
            n.name = word()
        for _ in range(rng.integers(0, 4)):
            b = n.blob.add()
            if rng.integers(4):
                b.name = word() or "w"
            if rng.integers(2):
                b.type = ["float", "int32", "uint8"][rng.integers(3)]
            b.shape.extend(int(v) for v in rng.integers(0, 300, size=rng.integers(0, 5)))
            b.data_f.extend(float(np.float32(v)) for v in rng.normal(size=rng.integers(0, 9)))
            b.data_i.extend(int(v) for v in rng.integers(-2 ** 31, 2 ** 31, size=rng.integers(0, 9)))
            for _ in range(rng.integers(0, 3)):
                b.data_b.append(rng.integers(0, 256, size=rng.integers(0, 40), dtype=np.uint8).tobytes())
        for _ in range(rng.integers(0, 5)):
            o = n.op.add()
            o.type, o.name = word() or "T", word() or "n"
            o.bottom.extend(word() for _ in range(rng.integers(0, 3)))
            o.top.extend(word() for _ in range(rng.integers(0, 3)))
            for _ in range(rng.integers(0, 4)):
                fill_arg(o.arg.add())
        for _ in range(rng.integers(0, 3)):
            fill_arg(n.arg.add())
        wire = n.SerializeToString()
        assert shadow_amd.reencode_proto(wire) == wire
