"""CPU-only checks: the C-ABI library loads and exports every symbol the header
declares, the launch planners produce the expected collapsed forms, and the host
layer's registries / argument handling behave like the reference's.  No kernel is
launched here."""
import ctypes
import os
import re

import pytest

import shadow_amd
from shadow_amd import ints

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "shadow_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(shdw_hip_\w+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    lib = shadow_amd.hip()
    names = declared_symbols()
    assert len(names) >= 35
    for name in names:
        assert hasattr(lib, name), name + " is declared in include/shadow_hip.h but not exported"
        assert name in shadow_amd.SIGNATURES, name + " has no ctypes signature"
    assert sorted(shadow_amd.SIGNATURES) == names


def test_error_strings():
    lib = shadow_amd.hip()
    assert lib.shdw_hip_error_string(0) == b"success"
    assert b"invalid argument" in lib.shdw_hip_error_string(-1)
    assert b"unsupported" in lib.shdw_hip_error_string(-2)
    assert b"workspace" in lib.shdw_hip_error_string(-3)


def plan_broadcast(a, b):
    rank = max(len(a), len(b))
    a = [1] * (rank - len(a)) + list(a)
    b = [1] * (rank - len(b)) + list(b)
    out = [max(x, y) for x, y in zip(a, b)]
    dims, sa, sb = (ctypes.c_int * 8)(), (ctypes.c_int * 8)(), (ctypes.c_int * 8)()
    n = shadow_amd.hip().shdw_hip_plan_broadcast(rank, ints(a), ints(b), ints(out), dims, sa, sb)
    return n, list(dims[:max(n, 0)]), list(sa[:max(n, 0)]), list(sb[:max(n, 0)])


def test_broadcast_plans_of_the_benchmark_shapes():
    # channel broadcast: [8,64,112,112] + [1,64,1,1] -> [8, 64, 12544]
    assert plan_broadcast([8, 64, 112, 112], [1, 64, 1, 1]) == (3, [8, 64, 12544], [802816, 12544, 1], [0, 1, 0])
    # stays 4-d
    assert plan_broadcast([16, 1, 128, 256], [1, 32, 128, 1]) == (
        4, [16, 32, 128, 256], [32768, 0, 256, 1], [0, 128, 1, 0])
    assert plan_broadcast([4, 64, 1, 512], [64, 512]) == (3, [256, 64, 512], [512, 0, 1], [0, 512, 1])
    assert plan_broadcast([128, 1024], [1]) == (1, [131072], [1], [0])
    assert plan_broadcast([5, 3], [5, 3]) == (1, [15], [1], [1])
    assert plan_broadcast([1, 1], [1]) == (0, [], [], [])
    assert plan_broadcast([2, 1], [3]) == (2, [2, 3], [1, 0], [0, 1])


def test_broadcast_plan_rejects_bad_shapes():
    lib = shadow_amd.hip()
    d = (ctypes.c_int * 8)()
    assert lib.shdw_hip_plan_broadcast(2, ints([2, 3]), ints([2, 2]), ints([2, 3]), d, d, d) == -1
    assert lib.shdw_hip_plan_broadcast(1, ints([3]), ints([1]), ints([4]), d, d, d) == -1
    assert lib.shdw_hip_plan_broadcast(1, ints([0]), ints([1]), ints([1]), d, d, d) == -1
    nine_a, nine_b = [2, 1] * 4 + [2], [1, 2] * 4 + [1]
    assert lib.shdw_hip_plan_broadcast(9, ints(nine_a), ints(nine_b), ints([2] * 9), d, d, d) == -2


def plan_reduce(shape, axes):
    out = [ctypes.c_int() for _ in range(5)]
    rc = shadow_amd.hip().shdw_hip_plan_reduce(len(shape), ints(shape), len(axes), ints(axes),
                                               *[ctypes.byref(o) for o in out])
    return rc, [o.value for o in out]


def test_reduce_plans_of_the_benchmark_shapes():
    ROWS, STRIDED, GENERIC = 0, 1, 2
    rc, (kind, outer, red, inner, splits) = plan_reduce([32, 512, 28, 28], [2, 3])
    assert (rc, kind, outer, red, inner, splits) == (0, ROWS, 16384, 784, 1, 1)
    rc, (kind, outer, red, inner, splits) = plan_reduce([32, 512, 28, 28], [1])
    assert (rc, kind, outer, red, inner, splits) == (0, STRIDED, 32, 512, 784, 1)  # single stage
    rc, (kind, outer, red, inner, splits) = plan_reduce([2, 100000, 8], [1])
    assert (rc, kind, outer, red, inner) == (0, STRIDED, 2, 100000, 8) and splits > 1
    rc, (kind, outer, red, inner, splits) = plan_reduce([32, 512, 28, 28], [0, 1, 2, 3])
    assert (rc, kind, outer, red, inner) == (0, ROWS, 1, 12845056, 1) and splits > 64
    rc, (kind, outer, red, inner, splits) = plan_reduce([64, 1024, 14, 14], [2, 3])
    assert (rc, kind, outer, red, inner, splits) == (0, ROWS, 65536, 196, 1, 1)
    # one reduced dim in front of a rows or strided view is folded by the second stage: the view
    # counts it among the outer indices, and the workspace holds a partial per leading index
    assert plan_reduce([2, 3, 4, 5], [0, 2])[1][:4] == [STRIDED, 6, 4, 5]
    assert plan_reduce([64, 256, 28, 28], [0, 2, 3])[1] == [ROWS, 64 * 256, 784, 1, 1]
    assert plan_reduce([8, 16, 4, 28], [1, 3])[1][:4] == [ROWS, 8 * 16 * 4, 28, 1]
    # a short reduced dim behind a long leading one: the leading dim first, over all that follows as columns
    assert plan_reduce([8, 256, 4, 28], [1, 3])[1][:4] == [STRIDED, 8, 256, 4 * 28]
    assert plan_reduce([256, 1024, 7, 7], [0, 2])[1][:4] == [STRIDED, 1, 256, 1024 * 49]
    assert plan_reduce([2, 3, 4, 5, 6], [0, 2, 4])[1][0] == GENERIC
    assert plan_reduce([2, 3, 4, 5], [3, 2])[1][0] == GENERIC  # list order is not memory order
    assert plan_reduce([6, 1, 5], [1])[1][:4] == [STRIDED, 1, 1, 30]
    assert plan_reduce([2, 3], [-1])[0] == -1
    assert plan_reduce([2, 3], [1, 1])[0] == -1
    assert plan_reduce([2, 3], [2])[0] == -1
    lib = shadow_amd.hip()
    assert lib.shdw_hip_reduce_workspace_bytes(4, ints([32, 512, 28, 28]), 2, ints([2, 3])) == 0
    assert lib.shdw_hip_reduce_workspace_bytes(1, ints([1 << 24]), 1, ints([0])) % 8 == 0
    assert lib.shdw_hip_reduce_workspace_bytes(4, ints([64, 256, 28, 28]), 3, ints([0, 2, 3])) == 8 * 256 * 64


def keys(fn):
    buf = ctypes.create_string_buffer(8192)
    fn(buf, 8192)
    return buf.value.decode().split("\n")


def test_registries_hold_exactly_the_gpu_default_kernels():
    h = shadow_amd.host()
    kernels = ["Activate", "Axpy", "BatchNorm", "Binary", "Concat", "Eltwise", "Gather", "GridSample", "GroupNorm", "LRN",
               "LayerNorm",
               "Normalize", "Pad", "Permute", "Pooling", "Reduce", "Reorg", "Resize", "SSDNormalize", "Scale",
               "ShuffleChannel", "Slice", "Softmax", "Stack", "Unary"]
    # InstanceNorm runs on the GroupNorm kernel (shadow/operators/instance_norm_op.cpp:14)
    # and the view-only operators need no kernel
    assert keys(h.shdw_host_operator_keys) == sorted(
        kernels + ["InstanceNorm", "Input", "Reshape", "Flatten", "Squeeze", "Unsqueeze"])
    kk = keys(h.shdw_host_kernel_keys)
    assert kk == ["%sGPU(Default)" % t for t in kernels]
    # a CUDNN flavour would outrank Default; a CPU kernel would be a compute fallback
    assert not any("CUDNN" in k or "CPU" in k for k in kk)


def test_kernel_lookup_and_argument_errors_throw():
    h = shadow_amd.host()
    for op in ("Unary", "Binary", "Eltwise", "Reduce", "Activate", "Scale"):
        assert h.shdw_host_probe_create_kernel(op.encode(), 1) == 0
        assert h.shdw_host_probe_create_kernel(op.encode(), 0) == -1  # no CPU kernels in this build
    assert h.shdw_host_probe_create_kernel(b"Conv", 1) == -1
    assert b"ConvGPU(None) is not registered" in h.shdw_host_last_error()
    assert h.shdw_host_probe_argument(b"int", b"int") == 0
    assert h.shdw_host_probe_argument(b"int", b"float") == -1   # present, wrong kind
    assert h.shdw_host_probe_argument(b"float", b"string") == -1
    assert h.shdw_host_probe_argument(b"none", b"int") == 0     # absent -> default
    assert h.shdw_host_probe_argument(b"int", b"dup") == -1
    assert b"Duplicated argument name" in h.shdw_host_last_error()


def test_entry_points_validate_before_touching_the_device():
    """Bad arguments are refused on the host: these calls return without a GPU."""
    lib = shadow_amd.hip()
    ints = shadow_amd.ints
    p = ctypes.c_void_p(4096)  # never dereferenced: validation fails first
    E, U = -1, -2
    assert lib.shdw_hip_softmax(-1, 2, 2, p, p, None) == E
    assert lib.shdw_hip_softmax(2, 2, 2, None, p, None) == E
    assert lib.shdw_hip_softmax(0, 5, 5, None, None, None) == 0
    assert lib.shdw_hip_normalize(65536, 65536, 2, 2.0, 0.0, p, p, None) == E
    assert lib.shdw_hip_batch_norm(8, 0, 1, p, p, p, 1.0, 0.0, p, None) == E
    assert lib.shdw_hip_ssd_normalize(2, -1, 4, 0, 1e-5, p, None, 1, p, None, None) == E
    assert lib.shdw_hip_ssd_normalize(2, 65536, 65536, 0, 1e-5, p, None, 1, p, None, None) == E
    assert lib.shdw_hip_ssd_normalize(2, 8, 4, 1, 1e-5, p, None, 1, p, None, None) == E   # no workspace
    assert lib.shdw_hip_ssd_normalize(2, 8, 4, 1, 1e-5, p, None, 1, p, ctypes.c_void_p(4100), None) == E
    assert lib.shdw_hip_ssd_normalize(2, 8, 4, 0, 1e-5, None, None, 1, p, None, None) == E
    assert lib.shdw_hip_ssd_normalize(0, 8, 4, 1, 1e-5, None, None, 1, None, None, None) == 0
    assert lib.shdw_hip_ssd_normalize_workspace_bytes(8, 512, 1444, 0) == 0
    assert 8 * 8 < lib.shdw_hip_ssd_normalize_workspace_bytes(8, 512, 1444, 1) <= 8 * 64 * 8  # several parts per item
    assert lib.shdw_hip_ssd_normalize_workspace_bytes(4096, 2, 8, 1) == 4096 * 8
    assert lib.shdw_hip_batch_norm(0, 4, 1, None, None, None, 1.0, 0.0, None, None) == 0
    assert lib.shdw_hip_batch_norm_scale(8, 2, 4, p, p, p, 1.0, 0.0, None, None, 1, p, None) == E  # neither scale nor bias
    assert lib.shdw_hip_batch_norm_scale(8, 0, 4, p, p, p, 1.0, 0.0, p, p, 1, p, None) == E
    assert lib.shdw_hip_batch_norm_scale(8, 2, 4, p, None, p, 1.0, 0.0, p, p, 0, p, None) == E
    assert lib.shdw_hip_batch_norm_scale(0, 2, 4, None, None, None, 1.0, 0.0, p, None, 0, None, None) == 0
    assert lib.shdw_hip_batch_norm_scale_residual_relu(16, 2, 8, p, p, None, 1.0, 0.0, p, p, p, 0, p, p, None) == E
    assert lib.shdw_hip_batch_norm_scale_residual_relu(16, 2, 8, p, p, p, 1.0, 0.0, p, p, None, 0, p, p, None) == E
    assert lib.shdw_hip_batch_norm_scale_residual_relu(15, 2, 8, p, p, p, 1.0, 0.0, p, p, p, 0, p, p, None) == E
    assert lib.shdw_hip_batch_norm_scale_residual_relu(0, 2, 8, p, p, p, 1.0, 0.0, p, p, p, 0, p, p, None) == 0
    gs = ints([1, 2, 2, 2])
    assert lib.shdw_hip_grid_sample(gs, gs, 2, 0, p, p, ctypes.c_void_p(8192), None) == E
    assert lib.shdw_hip_grid_sample(gs, gs, 1, 2, p, p, ctypes.c_void_p(8192), None) == E
    assert lib.shdw_hip_grid_sample(gs, ints([1, 3, 2, 2]), 1, 0, p, p, ctypes.c_void_p(8192), None) == E   # channels differ
    assert lib.shdw_hip_grid_sample(gs, gs, 1, 0, p, p, p, None) == E                                        # output is the input
    assert lib.shdw_hip_grid_sample(ints([1, 2, 0, 2]), gs, 1, 0, p, p, ctypes.c_void_p(8192), None) == E    # nothing to sample
    assert lib.shdw_hip_grid_sample(gs, ints([1, 2, 0, 2]), 1, 0, None, None, None, None) == 0
    lrn = ints([2, 3, 4, 4])
    assert lib.shdw_hip_lrn(lrn, 4, 1.0, 0.75, 1.0, p, p, None) == E            # even window
    assert lib.shdw_hip_lrn(lrn, 9, 1.0, 0.75, 1.0, p, p, None) == E            # four channels behind the centre, three there
    assert lib.shdw_hip_lrn(lrn, 5, 1.0, 0.75, 1.0, None, p, None) == E
    assert lib.shdw_hip_lrn(None, 5, 1.0, 0.75, 1.0, p, p, None) == E
    assert lib.shdw_hip_lrn(ints([2, 80, 1, 1]), 65, 1.0, 0.75, 1.0, p, p, None) == U   # windows over 63 channels
    assert lib.shdw_hip_lrn(ints([65536, 65536, 1, 1]), 5, 1.0, 0.75, 1.0, p, p, None) == U
    assert lib.shdw_hip_lrn(ints([2, 0, 4, 4]), 1, 1.0, 0.75, 1.0, None, None, None) == 0
    assert lib.shdw_hip_axpy_rows(65536, 65536, p, p, p, p, None) == E
    assert lib.shdw_hip_axpy_rows(4, 4, None, p, p, p, None) == E
    assert lib.shdw_hip_group_norm(2, 8, 1e-5, p, p, None, 1, 1, p, None) == E
    assert lib.shdw_hip_group_norm(2, 8, 1e-5, p, p, p, 0, 1, p, None) == E
    assert lib.shdw_hip_group_norm(0, 8, 1e-5, None, None, None, 1, 1, None, None) == 0
    sh = ints([1, 1, 4, 4])
    assert lib.shdw_hip_pooling2d(sh, 2, 2, 2, 1, 1, 0, 0, sh, p, p, None) == E
    assert lib.shdw_hip_pooling2d(sh, 0, 0, 2, 1, 1, 0, 0, sh, p, p, None) == E
    assert lib.shdw_hip_pooling2d(sh, 0, 2, 2, 0, 1, 0, 0, sh, p, p, None) == E
    assert lib.shdw_hip_pooling2d(sh, 0, 2, 2, 1, 1, -1, 0, sh, p, p, None) == E
    assert lib.shdw_hip_pooling2d(sh, 0, 2, 2, 1, 1, 0, 0, ints([2, 1, 3, 3]), p, p, None) == E
    assert lib.shdw_hip_pooling2d(None, 0, 2, 2, 1, 1, 0, 0, sh, p, p, None) == E
    assert lib.shdw_hip_pooling3d(ints([1, 1, 2, 2, 2]), 0, 2, 2, 2, 1, 1, 1, 0, 0, 0, ints([1, 1, 0, 1, 1]), p, p, None) == 0
    assert lib.shdw_hip_copy_chunks(2, 8, p, 4, 0, p, 8, 0, None) == E       # chunk wider than its source row
    assert lib.shdw_hip_copy_chunks(2, 4, p, 8, 0, p, 8, 6, None) == E       # chunk leaves its destination row
    assert lib.shdw_hip_copy_chunks(-1, 4, p, 8, 0, p, 8, 0, None) == E
    assert lib.shdw_hip_copy_chunks(0, 4, None, 8, 0, None, 8, 0, None) == 0
    assert lib.shdw_hip_gather(2, 0, 4, 3, p, p, p, None) == E
    assert lib.shdw_hip_gather(2, 5, 4, 0, p, p, p, None) == E
    assert lib.shdw_hip_shuffle_channel(2, 6, 4, 4, p, p, None) == E          # 6 channels, 4 groups
    assert lib.shdw_hip_pad(ints([1, 1, 4, 4]), ints([-3, -3, 0, 0]), 0.0, p, p, None) == E
    assert lib.shdw_hip_pad(None, ints([0, 0, 0, 0]), 0.0, p, p, None) == E
    assert lib.shdw_hip_permute(3, ints([2, 3, 4]), ints([0, 1, 1]), p, p, None) == E
    assert lib.shdw_hip_permute(3, ints([2, 3, 4]), ints([0, 1, 3]), p, p, None) == E
    assert lib.shdw_hip_permute(9, ints([1] * 9), ints(list(range(9))), p, p, None) == E
    assert lib.shdw_hip_permute(0, ints([1]), ints([0]), p, p, None) == E
    assert lib.shdw_hip_reorg(ints([1, 6, 4, 4]), 0, 2, p, p, None) == E       # 6 % 4 != 0
    assert lib.shdw_hip_reorg(ints([1, 4, 5, 4]), 1, 2, p, p, None) == E
    assert lib.shdw_hip_reorg(ints([1, 4, 4, 4]), 2, 2, p, p, None) == E
    assert lib.shdw_hip_reorg(ints([1, 4, 4, 4]), 1, 0, p, p, None) == E
    assert lib.shdw_hip_resize(ints([1, 1, 4, 4]), ints([1, 2, 8, 8]), 1, 0, p, p, None) == E
    assert lib.shdw_hip_resize(ints([1, 1, 4, 4]), ints([1, 1, 8, 8]), 3, 0, p, p, None) == E
    assert lib.shdw_hip_resize(ints([1, 1, 4, 4]), ints([1, 1, 1, 8]), 1, 1, p, p, None) == U
    assert lib.shdw_hip_resize(ints([1, 1, 4, 4]), ints([1, 1, 0, 8]), 1, 0, p, p, None) == 0
