"""TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.

The two steps either side of the operators, restated in Python:

  * the line-oriented model text: `write_text` follows the converter's writer
    (shadow/python/converter/shadow/transformer.py:30-65), `parse_text` the
    reference's reader (shadow/core/parser.cpp:1045-1110 ParseArgument /
    ParseCommon, :1844-1913 ParseNet);
  * the Native backend: `run` follows Native::Initial / Run / CopyWeights
    (shadow/backends/native/native.cpp:139-190, 38-98, 251-274) with the
    operator-level oracle functions in place of the operators, and the
    view-only operators restated here (shadow/operators/{input,reshape,
    flatten,squeeze,unsqueeze}_op.cpp).

A net is a plain dict:
  {"name": str, "arg": [(name, type, value)...],
   "blob": [(name, type, shape)...],
   "op": [{"type", "name", "bottom": [...], "top": [...], "arg": [(name, type, value)...]}]}
with argument types s_i / s_f / s_s / v_i / v_f / v_s.

Pinned by tests/test_net_cpu.py: hand-written texts with known structure, the
write -> parse round trip, and the reshape rules against numpy.reshape.
"""
import numpy as np

import oracle

F = np.float32


# ------------------------------------------------------------------ text ----
def _arg_text(arg):
    name, typ, value = arg
    if typ in ("s_i", "s_f", "s_s"):
        body = str(value)
    else:
        body = " # ".join(str(v) for v in value)
    return "{%s, %s, [%s]}" % (name, typ, body)


def write_text(net):
    lines = ["[%s]" % net["name"], "[%s]" % "; ".join(_arg_text(a) for a in net.get("arg", []))]
    lines.append("[%s]" % "; ".join(
        "{%s, %s, [%s]}" % (n, t, " # ".join(str(d) for d in shape)) for n, t, shape in net.get("blob", [])))
    for op in net["op"]:
        args = op.get("arg", [])
        lines.append("[%s] | [%s] | [%d %d %d] | [%s] | [%s] | [%s]" % (
            op["type"], op["name"], len(op["bottom"]), len(op["top"]), len(args),
            "; ".join(op["bottom"]), "; ".join(op["top"]), "; ".join(_arg_text(a) for a in args)))
    return "\n".join(lines) + "\n"


def _tokens(text, sep):
    return [t for t in text.split(sep) if t != ""]


def _inner(text):
    text = text.strip()
    return text[1:-1]


def _parse_args(text):
    out = []
    for item in _tokens(text, ";"):
        if not item.strip():
            continue
        parts = [p.strip() for p in _tokens(_inner(item), ",")]
        assert len(parts) == 3, item
        name, typ, value = parts[0], parts[1], _inner(parts[2])
        if typ == "s_f":
            val = F(float(value))
        elif typ == "s_i":
            val = int(value)
        elif typ == "s_s":
            val = value
        elif typ == "v_f":
            val = [F(float(v)) for v in _tokens(value, "#")]
        elif typ == "v_i":
            val = [int(v) for v in _tokens(value, "#")]
        elif typ == "v_s":
            val = [v.strip() for v in _tokens(value, "#")]
        else:
            raise oracle.OracleCheckError("Unsupported argument type " + typ)
        out.append((name, typ, val))
    return out


def parse_text(text):
    marks = _tokens(text, "\n")
    net = {"name": _inner(marks[0]), "arg": _parse_args(_inner(marks[1])), "blob": [], "op": []}
    for item in _tokens(_inner(marks[2]), ";"):
        if not item.strip():
            continue
        parts = [p.strip() for p in _tokens(_inner(item), ",")]
        assert len(parts) == 3, item
        net["blob"].append((parts[0], parts[1], [int(d) for d in _tokens(_inner(parts[2]), "#")]))
    for line in marks[3:]:
        if not line.strip():
            continue
        params = [_inner(p) for p in _tokens(line, "|")]
        assert len(params) == 6, line
        nb, nt, na = [int(c) for c in _tokens(params[2], " ")]
        net["op"].append({
            "type": params[0], "name": params[1],
            "bottom": [b.strip() for b in _tokens(params[3], ";")] if nb > 0 else [],
            "top": [t.strip() for t in _tokens(params[4], ";")] if nt > 0 else [],
            "arg": _parse_args(params[5]) if na > 0 else []})
    return net


# ---------------------------------------------------------- view-only ops ----
def reshape_shape(in_shape, shape, axis=0, num_axes=-1):
    """shadow/operators/reshape_op.cpp:17-76"""
    in_shape, shape = list(in_shape), list(shape)
    rank = len(in_shape)
    oracle._check(-rank <= axis < rank, "axis in range")
    start = axis + rank if axis < 0 else axis
    oracle._check(num_axes >= -1, "num_axes >= -1")
    end = rank if num_axes == -1 else start + num_axes
    oracle._check(end <= rank, "end_axis <= num_axes")
    out = in_shape[:start] + shape + in_shape[end:]
    count = int(np.prod(in_shape, dtype=np.int64))
    explicit = int(np.prod(in_shape[:start], dtype=np.int64)) * int(np.prod(in_shape[end:], dtype=np.int64))
    inferred = -1
    for d, dim in enumerate(shape):
        if dim == 0:
            oracle._check(rank > start + d, "copied axis exists")
            out[start + d] = in_shape[start + d]
            explicit *= out[start + d]
        elif dim == -1:
            oracle._check(inferred == -1, "one inferred axis")
            inferred = d
        else:
            explicit *= dim
    if inferred >= 0:
        oracle._check(count % explicit == 0, "count divisible")
        out[start + inferred] = count // explicit
    oracle._check(int(np.prod(out, dtype=np.int64)) == count, "output->count() == input->count()")
    return out


def flatten_shape(in_shape, axis=1, end_axis=-1):
    """shadow/operators/flatten_op.cpp:15-38"""
    in_shape = list(in_shape)
    oracle._check(axis >= 0, "axis >= 0")
    if end_axis == -1:
        end_axis = len(in_shape) - 1
    oracle._check(end_axis < len(in_shape) and axis <= end_axis, "axis <= end_axis < num_axes")
    return in_shape[:axis] + [int(np.prod(in_shape[axis:end_axis + 1], dtype=np.int64))] + in_shape[end_axis + 1:]


def squeeze_shape(in_shape, axes=()):
    """shadow/operators/squeeze_op.cpp:13-50"""
    out = []
    for n, dim in enumerate(in_shape):
        drop = (dim <= 1) if not axes else (n in axes)
        if drop:
            oracle._check(dim == 1, "squeezed dim == 1")
        else:
            out.append(dim)
    return out


def unsqueeze_shape(in_shape, axes):
    """shadow/operators/unsqueeze_op.cpp:13-43"""
    rank = len(in_shape)
    out = [0] * (rank + len(axes))
    for a in axes:
        a = a + rank + 1 if a < 0 else a
        oracle._check(0 <= a < len(out), "axis in range")
        out[a] = 1
    it = iter(in_shape)
    try:
        out = [next(it) if d == 0 else d for d in out]
    except StopIteration:
        raise oracle.OracleCheckError("Check Failed: d == num_axes")
    oracle._check(sum(1 for _ in it) == 0, "d == num_axes")
    return out


# ---------------------------------------------------------------- running ----
def _args(op):
    return {name: (typ, value) for name, typ, value in op.get("arg", [])}


def _single(args, name, default):
    return args[name][1] if name in args else default


def _repeated(args, name, default=()):
    """get_repeated_argument, including the form that accepts a single value."""
    if name not in args:
        return list(default)
    typ, value = args[name]
    return list(value) if typ.startswith("v_") else [value]


def _run_op(op, blobs):
    a = _args(op)
    x = [blobs[b] for b in op["bottom"]]
    t = op["type"]
    if t == "Input":
        return None
    if t == "Unary":
        return oracle.unary_op(x[0], _single(a, "operation", -1))
    if t == "Binary":
        if "scalar" in a:
            return oracle.binary_op(x[0], None, operation=_single(a, "operation", -1), scalar=a["scalar"][1])
        return oracle.binary_op(x[0], x[1], operation=_single(a, "operation", -1))
    if t == "Eltwise":
        return oracle.eltwise_op(x, _single(a, "operation", 1), _repeated(a, "coeff"))
    if t == "Reduce":
        return oracle.reduce_op(x[0], _single(a, "operation", 0), _repeated(a, "axes"),
                                bool(_single(a, "keep_dims", True)))
    if t == "Activate":
        return oracle.activate_op(x[0], _single(a, "type", 1), _single(a, "slope", F(0.1)),
                                  x[1] if len(x) > 1 else None)
    if t == "Scale":
        has_scale, has_bias = bool(_single(a, "has_scale", False)), bool(_single(a, "has_bias", False))
        if has_scale or has_bias:
            return oracle.scale_op(x[0], _single(a, "axis", 1), x[1] if has_scale else None,
                                   x[2 if has_scale else 1] if has_bias else None)
        return oracle.scale_op(x[0], _single(a, "axis", 1), None, None, _repeated(a, "scale_value"),
                               _repeated(a, "bias_value"))
    if t == "Axpy":
        oracle._check(len(x) == 3, "three inputs")
        return oracle.axpy_op(x[0], x[1], x[2])
    if t == "BatchNorm":
        oracle._check(len(x) >= 3, "inputs.size() >= 3")
        return oracle.batch_norm_op(x[0], x[1], x[2], x[3] if len(x) == 4 else None,
                                    _single(a, "eps", F(1e-5)), bool(_single(a, "use_global_stats", True)))
    if t == "GridSample":
        oracle._check(len(x) == 2, "inputs.size() == 2")
        return oracle.grid_sample_op(x[0], x[1], _single(a, "mode", 1), _single(a, "padding_mode", 0))
    if t == "LRN":
        return oracle.lrn_op(x[0], _single(a, "local_size", 5), _single(a, "alpha", F(1)), _single(a, "beta", F(0.75)),
                             _single(a, "norm_region", 0), _single(a, "k", F(1)))
    if t == "Softmax":
        return oracle.softmax_op(x[0], _single(a, "axis", 1))
    if t == "Normalize":
        return oracle.normalize_op(x[0], _single(a, "p", F(2)), _single(a, "axis", 1), _single(a, "eps", F(1e-12)))
    if t == "SSDNormalize":
        oracle._check(len(x) in (1, 2), "inputs.size() == 2")
        return oracle.ssd_normalize_op(x[0], x[1] if len(x) == 2 else None,
                                       bool(_single(a, "across_spatial", True)),
                                       bool(_single(a, "channel_shared", True)), _single(a, "eps", F(1e-5)))
    if t == "Pooling":
        return oracle.pooling_op(x[0], _single(a, "pool", 0), _repeated(a, "kernel_size", [0]),
                                 _repeated(a, "stride", [1]), _repeated(a, "pad", [0]),
                                 bool(_single(a, "global_pooling", False)), bool(_single(a, "full_pooling", True)))
    if t in ("GroupNorm", "InstanceNorm"):
        oracle._check(len(x) in (1, 3), "inputs.size() == 3")
        sc, bi = (x[1], x[2]) if len(x) == 3 else (None, None)
        if t == "InstanceNorm":
            return oracle.instance_norm_op(x[0], _single(a, "eps", F(1e-5)), sc, bi)
        return oracle.group_norm_op(x[0], _single(a, "group", 1), _single(a, "eps", F(1e-5)), sc, bi)
    if t == "LayerNorm":
        oracle._check(len(x) in (1, 3), "inputs.size() == 3")
        sc, bi = (x[1], x[2]) if len(x) == 3 else (None, None)
        return oracle.layer_norm_op(x[0], _repeated(a, "normalized_shape"), _single(a, "eps", F(1e-5)), sc, bi)
    if t == "Concat":
        return oracle.concat_op(x, _single(a, "axis", 1))
    if t == "Slice":
        return oracle.slice_op(x[0], len(op["top"]), _single(a, "axis", 1), _repeated(a, "slice_point"))
    if t == "Stack":
        return oracle.stack_op(x, _single(a, "axis", 0))
    if t == "Gather":
        idx = _repeated(a, "indexes")
        if not idx:
            oracle._check(len(op["bottom"]) == 2, "inputs.size() == 2")
            idx = np.asarray(blobs[op["bottom"][1]]).astype(np.int32).ravel()
        return oracle.gather_op(x[0], _single(a, "axis", 0), idx)
    if t == "Pad":
        return oracle.pad_op(x[0], _repeated(a, "paddings"), _single(a, "value", F(0)))
    if t == "Permute":
        return oracle.permute_op(x[0], _repeated(a, "order"))
    if t == "Reorg":
        return oracle.reorg_op(x[0], _single(a, "type", 0), _single(a, "stride", 2))
    if t == "ShuffleChannel":
        return oracle.shuffle_channel_op(x[0], _single(a, "group", 0))
    if t == "Resize":
        return oracle.resize_op(x[0], _repeated(a, "size", [0]), _repeated(a, "scale", [F(1)]),
                                _single(a, "type", 1), bool(_single(a, "align_corners", False)))
    if t == "Reshape":
        return x[0].reshape(reshape_shape(x[0].shape, _repeated(a, "shape"), _single(a, "axis", 0),
                                          _single(a, "num_axes", -1)))
    if t == "Flatten":
        return x[0].reshape(flatten_shape(x[0].shape, _single(a, "axis", 1), _single(a, "end_axis", -1)))
    if t == "Squeeze":
        return x[0].reshape(squeeze_shape(x[0].shape, _repeated(a, "axes")))
    if t == "Unsqueeze":
        return x[0].reshape(unsqueeze_shape(x[0].shape, _repeated(a, "axes")))
    raise oracle.OracleCheckError("Check Failed: operator type %s is not registered" % t)


def run(net, weights, inputs):
    """weights: arrays in declared-blob order (None or [] when the net declares
    none); inputs: {input blob name: array}.  Returns every blob by name."""
    weights = list(weights or [])
    oracle._check(len(weights) == len(net.get("blob", [])), "net_param.blob_size() == weights.size()")
    blobs = {}
    for (name, typ, shape), w in zip(net.get("blob", []), weights):
        oracle._check(typ in ("float", "int32"), "float and int32 blobs only in this oracle")
        blobs[name] = np.asarray(w, F if typ == "float" else np.int32).reshape(shape)
    net_args = {name: value for name, _, value in net.get("arg", [])}
    oracle._check("out_blob" in net_args, "Network must have out_blob argument")
    seen_input = False
    for op in net["op"]:
        if op["type"] == "Input":
            oracle._check(not seen_input, "in_blob_.empty()")
            seen_input = True
            a = _args(op)
            for top in op["top"]:
                oracle._check(top in a, "input shape argument")
                oracle._check(top in inputs, top + " has data")
                blobs[top] = np.asarray(inputs[top], F).reshape(inputs[top].shape)
    for op in net["op"]:
        for b in op["bottom"]:
            oracle._check(b in blobs, op["name"] + ": Can not find input blob " + b)
        out = _run_op(op, blobs)
        if isinstance(out, list):  # Slice: one array per top
            for top, part in zip(op["top"], out):
                blobs[top] = np.asarray(part, F)
        elif out is not None:
            oracle._check(len(op["top"]) >= 1, "an output blob")
            blobs[op["top"][0]] = np.asarray(out, F)
    return blobs
