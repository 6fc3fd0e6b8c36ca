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
    "shdw_hip_reduce_workspace_bytes": (_Z, [_I, c_int_p, _I, c_int_p]),
    "shdw_hip_reduce": (_I, [_I, _I, c_int_p, _I, c_int_p, _V, _V, _V, _Z, _V]),
    "shdw_hip_scale_residual_relu_rowmean": (_I, [_I, _I, _I, _V, _V, _V, _V, _V, _V, _V]),
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
