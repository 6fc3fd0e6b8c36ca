"""shdw_hip_reduce_static: the reduce entry point that allocates nothing.

Sliced shapes keep their partial results in the library's own device memory
instead of a caller's workspace.  Every case is compared with shdw_hip_reduce on
the same device input, bit for bit (same kernels, same fold order), on two calls
in a row, the second with a smaller input, so that what the first call left in
the shared buffer is seen not to matter."""
import numpy as np
import pytest

import shadow_amd
from shadow_amd import Buffer, check, ints
from tests.helpers import normal

pytestmark = pytest.mark.gpu


def _both(op, shape, axes, seed):
    lib = shadow_amd.hip()
    x = normal(seed, shape)
    d = Buffer.from_numpy(x.ravel())
    out_shape = list(shape)
    for ax in axes:
        out_shape[ax] = 1
    n_out = int(np.prod(out_shape, dtype=np.int64))
    need = lib.shdw_hip_reduce_workspace_bytes(len(shape), ints(shape), len(axes), ints(axes))
    ws = Buffer(need) if need else None
    y_ref, y_new = Buffer(4 * n_out), Buffer(4 * n_out)
    check(lib.shdw_hip_reduce(op, len(shape), ints(shape), len(axes), ints(axes), d.ptr, y_ref.ptr,
                              ws.ptr if ws else None, need, None))
    check(lib.shdw_hip_reduce_static(op, len(shape), ints(shape), len(axes), ints(axes), d.ptr, y_new.ptr, None))
    check(lib.shdw_hip_stream_sync(None))
    return y_ref.download(count=n_out), y_new.download(count=n_out), need


# (larger shape, smaller shape): both sliced, so both use the shared buffer
PAIRS = [
    (([3, 1 << 20], [1]), ([2, 40000], [1])),               # long rows: slices folded by the last workgroup
    (([1 << 22], [0]), ([100003], [0])),                    # full sum
    (([2, 30000, 8], [1]), ([2, 4097, 127], [1])),          # few columns, flat walk
    (([2, 6000, 512], [1]), ([1, 3000, 256], [1])),         # column tiles, sliced
    (([1, 65536, 128], [1]), ([1, 20000, 132], [1])),       # more partials than one workgroup folds: second launch
    (([2, 5000, 201], [1]), ([1, 3000, 129], [1])),         # one column per lane, sliced
    (([64, 96, 28, 28], [0, 2, 3]), ([6, 5, 7, 7], [0, 2, 3])),   # a reduced dim in front: partials per leading index
    (([300, 64, 7, 9], [0, 2]), ([40, 6, 7, 5], [0, 2])),         # the leading dim first, nested second stage
]


@pytest.mark.parametrize("big,small", PAIRS)
@pytest.mark.parametrize("op", [1, 2, 4, 6])
def test_static_scratch_matches_the_workspace_form(gpu, big, small, op):
    for k, (shape, axes) in enumerate((big, small)):
        ref, new, need = _both(op, shape, axes, 900 + k)
        assert need > 0, "the case is meant to be sliced"
        assert need <= shadow_amd.hip().shdw_hip_reduce_static_max_workspace_bytes()
        assert (ref.view(np.uint32) == new.view(np.uint32)).all(), (shape, axes, op)


def test_unsliced_shapes_and_errors(gpu):
    lib = shadow_amd.hip()
    ref, new, need = _both(1, [32, 64, 28, 28], [2, 3], 910)
    assert need == 0 and (ref.view(np.uint32) == new.view(np.uint32)).all()
    limit = lib.shdw_hip_reduce_static_max_workspace_bytes()
    assert limit == 1 << 20
    # a shape whose partials do not fit is refused before anything is launched
    shape, axes = [1000, 200, 127], [1]
    need = lib.shdw_hip_reduce_workspace_bytes(3, ints(shape), 1, ints(axes))
    assert need > limit
    d, y = Buffer(16), Buffer(16)  # never touched
    rc = lib.shdw_hip_reduce_static(1, 3, ints(shape), 1, ints(axes), d.ptr, y.ptr, None)
    assert rc == -4 and b"static" in lib.shdw_hip_error_string(rc)
    assert lib.shdw_hip_reduce_static(1, 1, ints([8]), 1, ints([0]), None, y.ptr, None) == -1


def test_a_warmed_up_call_leaves_the_free_device_memory_as_it_was(gpu):
    """Sliced shapes, whose partials go to the library's own buffer: nothing is allocated for them."""
    import ctypes
    lib = shadow_amd.hip()

    def free_bytes():
        f, t = ctypes.c_size_t(), ctypes.c_size_t()
        check(lib.shdw_hip_mem_info(ctypes.byref(f), ctypes.byref(t)))
        assert 0 < f.value <= t.value
        return f.value

    shape, axes = [2, 6000, 512], [1]
    assert lib.shdw_hip_reduce_workspace_bytes(3, ints(shape), 1, ints(axes)) > 0
    d, y = Buffer.from_numpy(normal(920, shape).ravel()), Buffer(4 * 2 * 512)
    check(lib.shdw_hip_reduce_static(1, 3, ints(shape), 1, ints(axes), d.ptr, y.ptr, None))  # warm-up: module, symbol
    check(lib.shdw_hip_stream_sync(None))
    before = free_bytes()
    for op in (1, 2, 4):
        check(lib.shdw_hip_reduce_static(op, 3, ints(shape), 1, ints(axes), d.ptr, y.ptr, None))
    check(lib.shdw_hip_reduce_static(1, 1, ints([1 << 22]), 1, ints([0]), d.ptr, y.ptr, None))
    check(lib.shdw_hip_stream_sync(None))
    assert free_bytes() == before
    # the workspace form of the same call, by contrast, has its caller allocate: the probe sees that
    ws = Buffer(64 << 20)
    assert free_bytes() < before
    ws.free()
