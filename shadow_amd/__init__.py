"""shadow_amd -- MI355X (gfx950) device layer for Shadow's tensor hot path.

The product is two shared libraries built in ``shadow_amd/lib``:

``libshadow_hip.so``
    hand-written HIP kernels behind the C ABI declared in ``include/shadow_hip.h``;
``libshadow_host.so``
    the C++ operator layer (Operator / Kernel registries, Blob, Workspace and the
    Unary, Binary, Eltwise, Reduce, Activate and Scale operators) that calls it.

This Python package is only a ctypes loader used by the tests, the benchmark and
the smoke check.  It never computes anything itself: if a library is missing it
raises, there is no fallback path.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_HERE, "lib")

c_void_pp = ctypes.POINTER(ctypes.c_void_p)
c_int_p = ctypes.POINTER(ctypes.c_int)
c_float_p = ctypes.POINTER(ctypes.c_float)

_hip = None


class HipError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("%s (code %d)" % (text, code))
        self.code = code


# name -> (restype, argtypes); pointers to device memory travel as c_void_p
_V, _I, _F, _Z = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t
SIGNATURES = {
    "shdw_hip_device_count": (_I, [c_int_p]),
    "shdw_hip_set_device": (_I, [_I]),
    "shdw_hip_device_info": (_I, [_I, ctypes.c_char_p, _Z]),
    "shdw_hip_stream_create": (_I, [c_void_pp]),
    "shdw_hip_stream_destroy": (_I, [_V]),
    "shdw_hip_stream_sync": (_I, [_V]),
    "shdw_hip_error_string": (ctypes.c_char_p, [_I]),
    "shdw_hip_last_error": (_I, []),
    "shdw_hip_malloc": (_I, [c_void_pp, _Z]),
    "shdw_hip_free": (_I, [_V]),
    "shdw_hip_memcpy_h2d": (_I, [_V, _V, _Z, _V]),
    "shdw_hip_memcpy_d2h": (_I, [_V, _V, _Z, _V]),
    "shdw_hip_memcpy_d2d": (_I, [_V, _V, _Z, _V]),
    "shdw_hip_host_malloc": (_I, [c_void_pp, _Z]),
    "shdw_hip_host_free": (_I, [_V]),
    "shdw_hip_event_create": (_I, [c_void_pp]),
    "shdw_hip_event_destroy": (_I, [_V]),
    "shdw_hip_event_record": (_I, [_V, _V]),
    "shdw_hip_event_sync": (_I, [_V]),
    "shdw_hip_event_elapsed_ms": (_I, [_V, _V, c_float_p]),
    "shdw_hip_set": (_I, [_I, _F, _V, _V]),
    "shdw_hip_unary": (_I, [_I, _I, _V, _V, _V]),
    "shdw_hip_binary": (_I, [_I, _I, _V, _V, _V, _V]),
    "shdw_hip_binary_scalar": (_I, [_I, _I, _V, _F, _V, _V]),
    "shdw_hip_scal": (_I, [_I, _F, _V, _V]),
    "shdw_hip_copy": (_I, [_I, _V, _V, _V]),
    "shdw_hip_axpy": (_I, [_I, _F, _V, _V, _V]),
    "shdw_hip_asum": (_I, [_I, _V, c_float_p, _V, _Z, _V]),
    "shdw_hip_broadcast_binary": (_I, [_I, _I, c_int_p, c_int_p, c_int_p, _V, _V, _V, _V]),
    "shdw_hip_activate": (_I, [_I, _F, _I, _V, _V, _V]),
    "shdw_hip_prelu": (_I, [_I, _I, _I, _I, _V, _V, _V, _V]),
    "shdw_hip_scale_bias": (_I, [_I, _I, _I, _V, _V, _V, _I, _V, _V]),
    "shdw_hip_eltwise": (_I, [_I, _I, c_void_pp, c_float_p, _I, _V, _V]),
    "shdw_hip_eltwise_relu": (_I, [_I, _I, c_void_pp, c_float_p, _I, _V, _V]),
    "shdw_hip_probe_read": (_I, [_I, _V, _F, _V, _V]),
    "shdw_hip_reduce_workspace_bytes": (_Z, [_I, c_int_p, _I, c_int_p]),
    "shdw_hip_reduce": (_I, [_I, _I, c_int_p, _I, c_int_p, _V, _V, _V, _Z, _V]),
    "shdw_hip_reduce_static": (_I, [_I, _I, c_int_p, _I, c_int_p, _V, _V, _V]),
    "shdw_hip_reduce_static_max_workspace_bytes": (_Z, []),
    "shdw_hip_scale_residual_relu_rowmean": (_I, [_I, _I, _I, _V, _V, _V, _V, _V, _V, _V]),
    "shdw_hip_mem_info": (_I, [ctypes.POINTER(_Z), ctypes.POINTER(_Z)]),
    "shdw_hip_softmax_plan": (_I, [_I, _I, _I, c_int_p, c_int_p, ctypes.POINTER(ctypes.c_uint)]),
    "shdw_hip_normalize_plan": (_I, [_I, _I, _I, _F, c_int_p, c_int_p, ctypes.POINTER(ctypes.c_uint)]),
    "shdw_hip_pooling2d_plan": (_I, [c_int_p, _I, _I, _I, _I, _I, _I, _I, c_int_p, c_int_p, c_int_p,
                                     ctypes.POINTER(ctypes.c_uint)]),
    "shdw_hip_scale_residual_relu": (_I, [_I, _I, _I, _V, _V, _V, _V, _I, _V, _V, _V]),
    "shdw_hip_batch_norm_scale_residual_relu": (_I, [_I, _I, _I, _V, _V, _V, _F, _F, _V, _V, _V, _I, _V, _V, _V]),
    "shdw_hip_grid_sample": (_I, [c_int_p, c_int_p, _I, _I, _V, _V, _V, _V]),
    "shdw_hip_lrn": (_I, [c_int_p, _I, _F, _F, _F, _V, _V, _V]),
    "shdw_hip_axpy_rows": (_I, [_I, _I, _V, _V, _V, _V, _V]),
    "shdw_hip_batch_norm": (_I, [_I, _I, _I, _V, _V, _V, _F, _F, _V, _V]),
    "shdw_hip_batch_norm_scale": (_I, [_I, _I, _I, _V, _V, _V, _F, _F, _V, _V, _I, _V, _V]),
    "shdw_hip_group_norm": (_I, [_I, _I, _F, _V, _V, _V, _I, _I, _V, _V]),
    "shdw_hip_group_norm_workspace_bytes": (_Z, [_I, _I]),
    "shdw_hip_group_norm_ws": (_I, [_I, _I, _F, _V, _V, _V, _I, _I, _V, _V, _Z, _V]),
    "shdw_hip_softmax": (_I, [_I, _I, _I, _V, _V, _V]),
    "shdw_hip_normalize": (_I, [_I, _I, _I, _F, _F, _V, _V, _V]),
    "shdw_hip_ssd_normalize_workspace_bytes": (_Z, [_I, _I, _I, _I]),
    "shdw_hip_ssd_normalize": (_I, [_I, _I, _I, _I, _F, _V, _V, _I, _V, _V, _V]),
    "shdw_hip_pooling2d": (_I, [c_int_p, _I, _I, _I, _I, _I, _I, _I, c_int_p, _V, _V, _V]),
    "shdw_hip_pooling3d": (_I, [c_int_p, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, c_int_p, _V, _V, _V]),
    "shdw_hip_copy_chunks": (_I, [_I, _I, _V, _I, _I, _V, _I, _I, _V]),
    "shdw_hip_gather": (_I, [_I, _I, _I, _I, _V, _V, _V, _V]),
    "shdw_hip_shuffle_channel": (_I, [_I, _I, _I, _I, _V, _V, _V]),
    "shdw_hip_pad": (_I, [c_int_p, c_int_p, _F, _V, _V, _V]),
    "shdw_hip_permute": (_I, [_I, c_int_p, c_int_p, _V, _V, _V]),
    "shdw_hip_reorg": (_I, [c_int_p, _I, _I, _V, _V, _V]),
    "shdw_hip_resize": (_I, [c_int_p, c_int_p, _I, _I, _V, _V, _V]),
    "shdw_hip_plan_broadcast": (_I, [_I, c_int_p, c_int_p, c_int_p, c_int_p, c_int_p, c_int_p]),
    "shdw_hip_plan_reduce": (_I, [_I, c_int_p, _I, c_int_p, c_int_p, c_int_p, c_int_p, c_int_p, c_int_p]),
}


def hip_library_path():
    return os.path.join(LIB_DIR, "libshadow_hip.so")


def hip():
    """The C-ABI library; raises if it has not been built."""
    global _hip
    if _hip is None:
        path = hip_library_path()
        if not os.path.exists(path):
            raise RuntimeError("%s is missing: build it with `python -m shadow_amd.build hip`" % path)
        lib = ctypes.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _hip = lib
    return _hip


def check(rc):
    if rc != 0:
        raise HipError(rc, hip().shdw_hip_error_string(rc).decode())


def ints(values):
    values = [int(v) for v in values]
    return (ctypes.c_int * max(1, len(values)))(*values)


def device_count():
    n = ctypes.c_int(0)
    rc = hip().shdw_hip_device_count(ctypes.byref(n))
    return n.value if rc == 0 else 0


class Buffer:
    """A device allocation made through the C ABI."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = ctypes.c_void_p()
        check(hip().shdw_hip_malloc(ctypes.byref(p), max(self.nbytes, 16)))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, arr):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        buf.upload(arr)
        return buf

    def upload(self, arr, offset_bytes=0):
        arr = np.ascontiguousarray(arr)
        check(hip().shdw_hip_memcpy_h2d(self.ptr + offset_bytes, arr.ctypes.data, arr.nbytes, None))

    def download(self, dtype=np.float32, count=None, offset_bytes=0):
        dtype = np.dtype(dtype)
        if count is None:
            count = (self.nbytes - offset_bytes) // dtype.itemsize
        out = np.empty(count, dtype)
        check(hip().shdw_hip_memcpy_d2h(out.ctypes.data, self.ptr + offset_bytes, out.nbytes, None))
        return out

    def free(self):
        if self.ptr:
            check(hip().shdw_hip_free(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


# --------------------------------------------------------------------------
# libshadow_host.so: the C++ operator layer behind its C facade (host/src/capi.cpp)
# --------------------------------------------------------------------------
_host = None

HOST_SIGNATURES = {
    "shdw_host_last_error": (ctypes.c_char_p, []),
    "shdw_host_kernel_keys": (_I, [ctypes.c_char_p, _Z]),
    "shdw_host_operator_keys": (_I, [ctypes.c_char_p, _Z]),
    "shdw_host_workspace_create": (_V, [ctypes.c_char_p, _I]),
    "shdw_host_workspace_destroy": (None, [_V]),
    "shdw_host_sync": (_I, [_V]),
    "shdw_host_blob_create": (_I, [_V, ctypes.c_char_p, ctypes.c_char_p]),
    "shdw_host_blob_set": (_I, [_V, ctypes.c_char_p, c_int_p, _I, _V]),
    "shdw_host_blob_shape": (_I, [_V, ctypes.c_char_p, c_int_p, _I]),
    "shdw_host_blob_get": (_I, [_V, ctypes.c_char_p, _V, _I]),
    "shdw_host_opparam_create": (_V, [ctypes.c_char_p, ctypes.c_char_p]),
    "shdw_host_opparam_destroy": (None, [_V]),
    "shdw_host_opparam_add_bottom": (None, [_V, ctypes.c_char_p]),
    "shdw_host_opparam_add_top": (None, [_V, ctypes.c_char_p]),
    "shdw_host_opparam_arg_i": (None, [_V, ctypes.c_char_p, _I]),
    "shdw_host_opparam_arg_f": (None, [_V, ctypes.c_char_p, _F]),
    "shdw_host_opparam_arg_s": (None, [_V, ctypes.c_char_p, ctypes.c_char_p]),
    "shdw_host_opparam_arg_vi": (None, [_V, ctypes.c_char_p, c_int_p, _I]),
    "shdw_host_opparam_arg_vf": (None, [_V, ctypes.c_char_p, c_float_p, _I]),
    "shdw_host_op_create": (_V, [_V, _V]),
    "shdw_host_op_destroy": (None, [_V]),
    "shdw_host_op_run": (_I, [_V, _V]),
    "shdw_host_op_debug_log": (_I, [_V, _V, ctypes.c_char_p, _Z]),
    "shdw_host_parse_net": (_I, [ctypes.c_char_p, ctypes.c_char_p, _Z]),
    "shdw_host_backend_keys": (_I, [ctypes.c_char_p, _Z]),
    "shdw_host_network_create": (_V, [ctypes.c_char_p, _I, _I, _I, _I, ctypes.c_char_p, _V]),
    "shdw_host_network_create_from_binary": (_V, [ctypes.c_char_p, _I, _I, _I, _I, _V, _I, _I]),
    "shdw_host_parse_net_binary": (_I, [_V, _I, _I, ctypes.c_char_p, _Z]),
    "shdw_host_plan_fusion": (_I, [ctypes.c_char_p, ctypes.c_char_p, _Z]),
    "shdw_host_proto_reencode": (_I, [_V, _I, _I, _V, _Z]),
    "shdw_host_serialize_net": (_I, [ctypes.c_char_p, _V, _Z]),
    "shdw_host_proto_file_reencode": (_I, [ctypes.c_char_p, ctypes.c_char_p, _I]),
    "shdw_host_network_destroy": (None, [_V]),
    "shdw_host_network_io": (_I, [_V, _I, ctypes.c_char_p, _Z]),
    "shdw_host_network_forward": (_I, [_V, _I, ctypes.POINTER(ctypes.c_char_p), c_void_pp, c_int_p, c_int_p]),
    "shdw_host_network_run": (_I, [_V]),
    "shdw_host_network_stream": (_V, [_V]),
    "shdw_host_network_blob_shape": (_I, [_V, ctypes.c_char_p, c_int_p, _I]),
    "shdw_host_network_blob_get": (_I, [_V, ctypes.c_char_p, c_float_p, _I]),
    "shdw_host_face_blas": (_I, [_V, ctypes.c_char_p, _I, c_float_p, _I, _I, c_float_p, _I, _I, _F, c_float_p, _I, _I]),
    "shdw_host_face_conv_epilogue": (_I, [_V, c_float_p, _I, c_float_p, _I, _I, _I, _I]),
    "shdw_host_face_eltwise_sum": (_I, [_V, _I, ctypes.POINTER(c_float_p), c_float_p, _I, c_float_p]),
    "shdw_host_face_ssd_normalize": (_I, [_V, c_float_p, _I, _I, _I, _I, _I, _F, c_float_p, c_float_p]),
    "shdw_host_probe_create_kernel": (_I, [ctypes.c_char_p, _I]),
    "shdw_host_probe_argument": (_I, [ctypes.c_char_p, ctypes.c_char_p]),
}


class ShadowError(RuntimeError):
    """A CHECK / LOG(FATAL) of the C++ layer fired (std::runtime_error there)."""


def host():
    global _host
    if _host is None:
        hip()  # resolves libshadow_hip.so first
        path = os.path.join(LIB_DIR, "libshadow_host.so")
        if not os.path.exists(path):
            raise RuntimeError("%s is missing: build it with `python -m shadow_amd.build host`" % path)
        lib = ctypes.CDLL(path)
        for name, (res, args) in HOST_SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _host = lib
    return _host


def host_check(ok):
    if not ok:
        raise ShadowError(host().shdw_host_last_error().decode())


class Workspace:
    """A Shadow::Workspace with a GPU context, plus blob and operator helpers."""

    def __init__(self, backend_type="Native", device_id=0):
        self.lib = host()
        self.ptr = self.lib.shdw_host_workspace_create(backend_type.encode(), device_id)
        host_check(self.ptr)
        self._ops = []

    def close(self):
        for op in self._ops:
            op.close()
        self._ops = []
        if self.ptr:
            self.lib.shdw_host_workspace_destroy(self.ptr)
            self.ptr = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def set_blob(self, name, array, dtype="float"):
        array = np.ascontiguousarray(array, dtype=np.float32 if dtype == "float" else np.int32)
        host_check(self.lib.shdw_host_blob_create(self.ptr, name.encode(), dtype.encode()) == 0)
        shape = ints(array.shape) if array.ndim else ints([1])
        rank = array.ndim if array.ndim else 1
        host_check(self.lib.shdw_host_blob_set(self.ptr, name.encode(), shape, rank,
                                               array.ctypes.data) == 0)

    def run(self):
        """The operators once more on what the input blobs hold; enqueued, not waited for."""
        host_check(self.lib.shdw_host_network_run(self.ptr) == 0)

    @property
    def stream(self):
        return ctypes.c_void_p(self.lib.shdw_host_network_stream(self.ptr))

    def blob_shape(self, name):
        shape = (ctypes.c_int * 16)()
        rank = self.lib.shdw_host_blob_shape(self.ptr, name.encode(), shape, 16)
        host_check(rank >= 0)
        return [shape[i] for i in range(rank)]

    def get_blob(self, name, dtype=np.float32):
        shape = self.blob_shape(name)
        count = int(np.prod(shape, dtype=np.int64)) if shape else 1
        out = np.empty(count, dtype)
        host_check(self.lib.shdw_host_blob_get(self.ptr, name.encode(), out.ctypes.data, count) == 0)
        return out.reshape(shape)

    def sync(self):
        host_check(self.lib.shdw_host_sync(self.ptr) == 0)

    def create_op(self, op_type, bottoms, tops, args=None, name=None):
        op = Op(self, op_type, bottoms, tops, args or {}, name or op_type.lower())
        self._ops.append(op)
        return op


class Op:
    """One Shadow operator.  `args` values: int/bool -> s_i, float -> s_f,
    str -> s_s, list of int -> v_i, list of float -> v_f."""

    def __init__(self, ws, op_type, bottoms, tops, args, name):
        lib = ws.lib
        self.ws = ws
        param = lib.shdw_host_opparam_create(op_type.encode(), name.encode())
        try:
            for b in bottoms:
                lib.shdw_host_opparam_add_bottom(param, b.encode())
            for t in tops:
                lib.shdw_host_opparam_add_top(param, t.encode())
            for key, val in args.items():
                k = key.encode()
                if isinstance(val, (bool, int, np.integer)):
                    lib.shdw_host_opparam_arg_i(param, k, int(val))
                elif isinstance(val, (float, np.floating)):
                    lib.shdw_host_opparam_arg_f(param, k, float(val))
                elif isinstance(val, str):
                    lib.shdw_host_opparam_arg_s(param, k, val.encode())
                elif len(val) and isinstance(val[0], (float, np.floating)):
                    arr = (ctypes.c_float * len(val))(*[float(v) for v in val])
                    lib.shdw_host_opparam_arg_vf(param, k, arr, len(val))
                else:
                    lib.shdw_host_opparam_arg_vi(param, k, ints(val), len(val))
            self.ptr = lib.shdw_host_op_create(ws.ptr, param)
        finally:
            lib.shdw_host_opparam_destroy(param)
        host_check(self.ptr)

    def run(self):
        host_check(self.ws.lib.shdw_host_op_run(self.ws.ptr, self.ptr) == 0)

    def debug_log(self):
        buf = ctypes.create_string_buffer(4096)
        host_check(self.ws.lib.shdw_host_op_debug_log(self.ws.ptr, self.ptr, buf, 4096) >= 0)
        return buf.value.decode()

    def close(self):
        if self.ptr:
            self.ws.lib.shdw_host_op_destroy(self.ptr)
            self.ptr = None


def parse_net(proto_text):
    """Canonical spelling of a text model as the C++ parser understood it (host only)."""
    lib = host()
    buf = ctypes.create_string_buffer(max(4096, 4 * len(proto_text) + 1024))
    n = lib.shdw_host_parse_net(proto_text.encode(), buf, len(buf))
    host_check(n >= 0)
    return buf.value.decode()


def plan_fusion(proto_text):
    """The groups the Native backend's fusion pass forms for a text model, as Network.fused
    lists them once the model is loaded (host only)."""
    lib = host()
    buf = ctypes.create_string_buffer(max(4096, 4 * len(proto_text) + 1024))
    n = lib.shdw_host_plan_fusion(proto_text.encode(), buf, len(buf))
    host_check(n >= 0)
    text = buf.value.decode()
    return text.split("\n") if text else []


def parse_net_binary(data, network_index=-1):
    """Canonical text form of a binary model: a serialized NetParam, or network
    `network_index` of a serialized MetaNetParam (host only)."""
    lib = host()
    data = bytes(data)
    buf = ctypes.create_string_buffer(max(4096, 8 * len(data) + 1024))
    n = lib.shdw_host_parse_net_binary(data, len(data), network_index, buf, len(buf))
    host_check(n >= 0)
    return buf.value.decode()


def reencode_proto(data, meta=False):
    """Decode and re-encode a serialized NetParam / MetaNetParam (host only)."""
    lib = host()
    data = bytes(data)
    buf = ctypes.create_string_buffer(2 * len(data) + 1024)
    n = lib.shdw_host_proto_reencode(data, len(data), int(meta), buf, len(buf))
    host_check(0 <= n <= len(buf))
    return buf.raw[:n]


def serialize_net(proto_text):
    """A text model as a serialized NetParam (host only)."""
    lib = host()
    buf = ctypes.create_string_buffer(4 * len(proto_text) + 1024)
    n = lib.shdw_host_serialize_net(proto_text.encode(), buf, len(buf))
    host_check(0 <= n <= len(buf))
    return buf.raw[:n]


class Network:
    """Shadow::Network over the Native backend: a text model plus packed float32
    weights (declared-blob order), run with host inputs.  from_binary() takes a
    serialized model whose blobs carry their contents instead."""

    @classmethod
    def from_binary(cls, data, network_index=-1, backend_type="Native", device_id=0, debug=False,
                    device_input=False, fuse=True):
        self = cls.__new__(cls)
        self.lib = host()
        self.device_input = device_input
        data = bytes(data)
        self.ptr = self.lib.shdw_host_network_create_from_binary(
            backend_type.encode(), device_id, int(debug), int(device_input), int(fuse), data, len(data),
            network_index)
        host_check(self.ptr)
        return self

    def __init__(self, proto_text, weights=None, backend_type="Native", device_id=0, debug=False,
                 device_input=False, fuse=True):
        self.lib = host()
        self.device_input = device_input
        packed = None
        if weights is not None and len(weights):
            packed = np.concatenate([np.ascontiguousarray(w, np.float32).ravel() for w in weights])
        self.ptr = self.lib.shdw_host_network_create(
            backend_type.encode(), device_id, int(debug), int(device_input), int(fuse), proto_text.encode(),
            packed.ctypes.data if packed is not None else None)
        host_check(self.ptr)

    def _names(self, which):
        buf = ctypes.create_string_buffer(8192)
        host_check(self.lib.shdw_host_network_io(self.ptr, which, buf, len(buf)) >= 0)
        text = buf.value.decode()
        return text.split("\n") if text else []

    @property
    def in_blob(self):
        return self._names(0)

    @property
    def out_blob(self):
        return self._names(1)

    @property
    def fused(self):
        """One line per group of operators that the backend runs as one launch."""
        return self._names(2)

    def forward(self, inputs, reshape=False):
        """inputs: {blob name: float32 array}.  reshape=True passes each array's
        shape along, so the input blob is reshaped before the copy."""
        names = list(inputs)
        c_names = (ctypes.c_char_p * len(names))(*[k.encode() for k in names])
        if self.device_input:  # {name: Buffer}; shapes stay as declared
            c_data = (ctypes.c_void_p * len(names))(*[inputs[k].ptr for k in names])
            host_check(self.lib.shdw_host_network_forward(self.ptr, len(names), c_names, c_data, None, None) == 0)
            return
        arrays = [np.ascontiguousarray(inputs[k], np.float32) for k in names]
        c_data = (ctypes.c_void_p * len(names))(*[a.ctypes.data for a in arrays])
        ranks = ints([a.ndim if reshape else 0 for a in arrays])
        dims = ints([d for a in arrays for d in (a.shape if reshape else ())])
        host_check(self.lib.shdw_host_network_forward(self.ptr, len(names), c_names, c_data, ranks, dims) == 0)

    def run(self):
        """The operators once more on what the input blobs hold; enqueued, not waited for."""
        host_check(self.lib.shdw_host_network_run(self.ptr) == 0)

    @property
    def stream(self):
        return ctypes.c_void_p(self.lib.shdw_host_network_stream(self.ptr))

    def blob_shape(self, name):
        shape = (ctypes.c_int * 16)()
        rank = self.lib.shdw_host_network_blob_shape(self.ptr, name.encode(), shape, 16)
        host_check(rank >= 0)
        return [shape[i] for i in range(rank)]

    def blob(self, name):
        shape = self.blob_shape(name)
        out = np.empty(int(np.prod(shape, dtype=np.int64)) if shape else 1, np.float32)
        host_check(self.lib.shdw_host_network_blob_get(
            self.ptr, name.encode(), out.ctypes.data_as(c_float_p), out.size) == 0)
        return out.reshape(shape)

    def close(self):
        if self.ptr:
            self.lib.shdw_host_network_destroy(self.ptr)
            self.ptr = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
