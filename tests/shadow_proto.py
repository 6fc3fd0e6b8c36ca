"""The five messages of Shadow's model files (shadow/proto/shadow.proto:5-47)
as python-protobuf classes, built from a descriptor written out here (there is
no protoc in this environment).  Test infrastructure: python-protobuf is the
independent implementation the C++ wire reader and writer are checked against."""
from google.protobuf import descriptor_pb2, descriptor_pool, message_factory

_T = descriptor_pb2.FieldDescriptorProto
_SCALAR = {"string": _T.TYPE_STRING, "float": _T.TYPE_FLOAT, "int32": _T.TYPE_INT32, "bytes": _T.TYPE_BYTES}

# message -> [(field name, number, type, repeated, packed)]
_SCHEMA = {
    "Blob": [("name", 1, "string", False, False), ("type", 2, "string", False, False),
             ("shape", 3, "int32", True, False), ("data_f", 4, "float", True, True),
             ("data_i", 5, "int32", True, True), ("data_b", 6, "bytes", True, False)],
    "Argument": [("name", 1, "string", False, False), ("s_f", 2, "float", False, False),
                 ("s_i", 3, "int32", False, False), ("s_s", 4, "string", False, False),
                 ("v_f", 5, "float", True, False), ("v_i", 6, "int32", True, False),
                 ("v_s", 7, "string", True, False)],
    "OpParam": [("name", 1, "string", False, False), ("type", 2, "string", False, False),
                ("bottom", 3, "string", True, False), ("top", 4, "string", True, False),
                ("arg", 11, "Argument", True, False)],
    "NetParam": [("name", 1, "string", False, False), ("blob", 5, "Blob", True, False),
                 ("op", 11, "OpParam", True, False), ("arg", 12, "Argument", True, False)],
    "MetaNetParam": [("name", 1, "string", False, False), ("network", 11, "NetParam", True, False),
                     ("arg", 12, "Argument", True, False)],
}


def _build(package):
    fd = descriptor_pb2.FileDescriptorProto()
    fd.name, fd.package, fd.syntax = package + ".proto", package, "proto2"
    for msg_name, fields in _SCHEMA.items():
        msg = fd.message_type.add()
        msg.name = msg_name
        for name, number, kind, repeated, packed in fields:
            f = msg.field.add()
            f.name, f.number = name, number
            f.label = _T.LABEL_REPEATED if repeated else _T.LABEL_OPTIONAL
            if kind in _SCALAR:
                f.type = _SCALAR[kind]
            else:
                f.type, f.type_name = _T.TYPE_MESSAGE, ".%s.%s" % (package, kind)
            if packed:
                f.options.packed = True
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    return {n: message_factory.GetMessageClass(pool.FindMessageTypeByName("%s.%s" % (package, n))) for n in _SCHEMA}


_classes = _build("shadow")
Blob, Argument, OpParam, NetParam, MetaNetParam = (_classes[n] for n in
                                                   ("Blob", "Argument", "OpParam", "NetParam", "MetaNetParam"))


def add_arg(owner, arg):
    """Append an Argument from oracle.net's (name, type, value) triple."""
    name, typ, value = arg
    a = owner.arg.add()
    a.name = name
    if typ == "s_f":
        a.s_f = float(value)
    elif typ == "s_i":
        a.s_i = int(value)
    elif typ == "s_s":
        a.s_s = str(value)
    elif typ == "v_f":
        a.v_f.extend(float(v) for v in value)
    elif typ == "v_i":
        a.v_i.extend(int(v) for v in value)
    elif typ == "v_s":
        a.v_s.extend(str(v) for v in value)
    else:
        raise ValueError(typ)
    return a


def from_oracle_net(net, weights=None):
    """oracle.net's dict form -> NetParam message.  weights: arrays in declared
    blob order, stored as data_f (float blobs) or data_b (anything else)."""
    import numpy as np
    msg = NetParam()
    msg.name = net["name"]
    for arg in net.get("arg", []):
        add_arg(msg, arg)
    for i, (name, typ, shape) in enumerate(net.get("blob", [])):
        blob = msg.blob.add()
        blob.name, blob.type = name, typ
        blob.shape.extend(int(d) for d in shape)
        if weights is not None:
            w = np.ascontiguousarray(weights[i])
            if typ == "float":
                blob.data_f.extend(w.astype(np.float32).ravel().tolist())
            else:
                blob.data_b.append(w.tobytes())
    for o in net["op"]:
        op = msg.op.add()
        op.type, op.name = o["type"], o["name"]
        op.bottom.extend(o.get("bottom", []))
        op.top.extend(o.get("top", []))
        for arg in o.get("arg", []):
            add_arg(op, arg)
    return msg
