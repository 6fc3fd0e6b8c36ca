"""TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.

Python face of the CPU oracle: ctypes bindings to ``liboracle.so`` (the C
restatement in ``shadow_cpu.c``) plus the operator-level shape rules of the
reference's ``*_op.cpp`` files.  Only ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py`` may import this package.

Errors that the reference raises through ``CHECK`` (a thrown
``std::runtime_error``) are raised here as :class:`OracleCheckError`.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

_f32p = ctypes.POINTER(ctypes.c_float)
_i32p = ctypes.POINTER(ctypes.c_int)


class OracleCheckError(RuntimeError):
    """A condition the reference guards with CHECK/LOG(FATAL) failed."""


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            raise RuntimeError("oracle/liboracle.so is not built; run `python -m oracle.build`")
        _LIB = ctypes.CDLL(path)
        _LIB.orc_asum.restype = ctypes.c_float
    return _LIB


def _f(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return a.ctypes.data_as(_f32p)


def _ints(v):
    arr = (ctypes.c_int * max(1, len(v)))(*[int(x) for x in v])
    return arr


def _check(cond, msg):
    if not cond:
        raise OracleCheckError("Check Failed: " + msg)


# --------------------------------------------------------------------------
# kernel level (flat arrays)
# --------------------------------------------------------------------------
def blas_set(n, val):
    y = np.empty(n, np.float32)
    lib().orc_set(n, ctypes.c_float(val), _p(y))
    return y


def unary(op, a):
    a = _f(a)
    y = np.empty_like(a)
    _check(lib().orc_unary(int(op), a.size, _p(a), _p(y)) == 0, "unary operation")
    return y


def binary(op, a, b):
    a, b = _f(a), _f(b)
    assert a.size == b.size
    y = np.empty_like(a)
    _check(lib().orc_binary(int(op), a.size, _p(a), _p(b), _p(y)) == 0, "binary operation")
    return y


def binary_scalar(op, a, alpha):
    a = _f(a)
    y = np.empty_like(a)
    _check(lib().orc_binary_scalar(int(op), a.size, _p(a), ctypes.c_float(alpha), _p(y)) == 0,
           "binary operation")
    return y


def scal(alpha, x):
    x = _f(x).copy()
    lib().orc_scal(x.size, ctypes.c_float(alpha), _p(x))
    return x


def copy(x):
    x = _f(x)
    y = np.empty_like(x)
    lib().orc_copy(x.size, _p(x), _p(y))
    return y


def axpy(alpha, x, y):
    x, y = _f(x), _f(y).copy()
    lib().orc_axpy(x.size, ctypes.c_float(alpha), _p(x), _p(y))
    return y


def asum(x):
    x = _f(x)
    return np.float32(lib().orc_asum(x.size, _p(x)))


def broadcast_binary(op, a, a_shape, b, b_shape, out_shape):
    """a_shape / b_shape / out_shape are rank-aligned lists."""
    a, b = _f(a), _f(b)
    count = int(np.prod(out_shape, dtype=np.int64))
    out = np.empty(count, np.float32)
    rc = lib().orc_broadcast_binary(_p(a), _ints(a_shape), _p(b), _ints(b_shape), int(op),
                                    len(out_shape), count, _ints(out_shape), _p(out))
    _check(rc == 0, "broadcast binary arguments")
    return out


def activate(x, act_type, slope=0.1):
    x = _f(x)
    y = np.empty_like(x)
    lib().orc_activate(_p(x), _p(y), x.size, int(act_type), ctypes.c_float(slope))
    return y


def prelu(x, shape, channel_shared, slope):
    x, slope = _f(x), _f(slope)
    y = np.empty_like(x)
    lib().orc_prelu(_p(x), _p(y), _ints(shape), len(shape), int(bool(channel_shared)), _p(slope))
    return y


def scale_bias(x, scale, bias, scale_num, inner_num):
    x = _f(x)
    y = np.empty_like(x)
    if scale is not None and bias is not None:
        scale, bias = _f(scale), _f(bias)
        lib().orc_scale_bias(_p(x), x.size, _p(scale), _p(bias), scale_num, inner_num, _p(y))
    elif scale is not None:
        scale = _f(scale)
        lib().orc_scale(_p(x), x.size, _p(scale), scale_num, inner_num, _p(y))
    else:
        bias = _f(bias)
        lib().orc_bias(_p(x), x.size, _p(bias), scale_num, inner_num, _p(y))
    return y


def eltwise(op, inputs, coeff=None, out=None):
    """`out` may be one of the input arrays to model aliasing."""
    inputs = [x if x.dtype == np.float32 and x.flags.c_contiguous else _f(x) for x in inputs]
    k = len(inputs)
    n = inputs[0].size
    if out is None:
        out = np.empty(n, np.float32)
    ptrs = (_f32p * k)(*[_p(x) for x in inputs])
    co = _f(coeff if coeff is not None else np.ones(k))
    _check(lib().orc_eltwise(int(op), k, ptrs, _p(co), n, _p(out)) == 0, "eltwise arguments")
    return out


def reduce(op, x, shape, axes):
    x = _f(x)
    out_shape = list(shape)
    for ax in axes:
        out_shape[ax] = 1
    out = np.empty(int(np.prod(out_shape, dtype=np.int64)), np.float32)
    rc = lib().orc_reduce(int(op), _p(x), _ints(shape), len(shape), _ints(axes), len(axes), _p(out))
    _check(rc == 0, "reduce arguments")
    return out, out_shape


def axpy_rows(alpha, x, y, inner_num):
    alpha, x, y = _f(alpha).ravel(), _f(x).ravel(), _f(y).ravel()
    out = np.empty_like(x)
    lib().orc_axpy_rows(_p(alpha), _p(x), _p(y), alpha.size, int(inner_num), _p(out))
    return out


def batch_norm(x, mean, variance, channel, inner_num, scale_factor, eps):
    x, mean, variance = _f(x).ravel(), _f(mean).ravel(), _f(variance).ravel()
    out = np.empty_like(x)
    lib().orc_batch_norm(_p(x), x.size, _p(mean), _p(variance), int(channel), int(inner_num),
                         ctypes.c_float(scale_factor), ctypes.c_float(eps), _p(out))
    return out


def lrn(x, in_shape, size, alpha, beta, k):
    """(out, scale): Vision::LRN and the scale blob it leaves (k + alpha / size * windowed sum of squares)."""
    x = _f(x).ravel()
    out, scale = np.empty_like(x), np.empty_like(x)
    lib().orc_lrn(_p(x), _ints(in_shape), int(size), ctypes.c_float(alpha), ctypes.c_float(beta), ctypes.c_float(k),
                  _p(scale), _p(out))
    return out, scale


def grid_sample(x, in_shape, grid, mode, padding_mode, out_shape):
    x, grid = _f(x).ravel(), _f(grid).ravel()
    out = np.empty(int(np.prod(out_shape, dtype=np.int64)), np.float32)
    lib().orc_grid_sample(_p(x), _ints(in_shape), _p(grid), int(mode), int(padding_mode), _ints(out_shape), _p(out))
    return out


def softmax(x, outer, dim, inner):
    x = _f(x).ravel()
    out = np.empty_like(x)
    val = np.empty(max(1, outer * inner), np.float32)
    lib().orc_softmax(_p(x), int(outer), int(dim), int(inner), _p(val), _p(out))
    return out


def normalize(x, outer, dim, inner, p, eps):
    x = _f(x).ravel()
    out = np.empty_like(x)
    val = np.empty(max(1, outer * inner), np.float32)
    lib().orc_normalize(_p(x), int(outer), int(dim), int(inner), _p(val), ctypes.c_float(p),
                        ctypes.c_float(eps), _p(out))
    return out


def ssd_normalize(x, batch, channel, spatial_dim, across_spatial, channel_shared, eps, scale=None):
    """SSDNormalizeKernelDefault::Run on flat data."""
    x = _f(x).ravel()
    out = np.empty_like(x)
    val = np.empty(max(1, batch * spatial_dim), np.float32)
    sc = None if scale is None else _f(scale).ravel()
    lib().orc_ssd_normalize_run(_p(x), int(batch), int(channel), int(spatial_dim), int(bool(across_spatial)),
                                int(bool(channel_shared)), ctypes.c_float(eps),
                                _p(sc) if sc is not None else None, _p(val), _p(out))
    return out


def pooling(x, in_shape, pool_type, kernel, stride, pad, out_shape):
    """2-D or 3-D by len(kernel)."""
    x = _f(x).ravel()
    out = np.empty(int(np.prod(out_shape, dtype=np.int64)), np.float32)
    fn = lib().orc_pooling2d if len(kernel) == 2 else lib().orc_pooling3d
    fn(_p(x), _ints(in_shape), int(pool_type), *[int(v) for v in kernel], *[int(v) for v in stride],
       *[int(v) for v in pad], _ints(out_shape), _p(out))
    return out


def pooling_out_size(dim, kernel_size, stride, pad, full_pooling):
    return int(lib().orc_pooling_out_size(int(dim), int(kernel_size), int(stride), int(pad),
                                          int(bool(full_pooling))))


def normalize_rows(x, outer, inner, eps):
    """Mean / variance normalisation of rows, as the GroupNorm and LayerNorm kernel
    classes run it (before their ScaleBias)."""
    x = _f(x).ravel()
    out = np.empty_like(x)
    mean, var = np.zeros(max(1, outer), np.float32), np.zeros(max(1, outer), np.float32)
    temp = np.zeros(max(1, x.size), np.float32)
    lib().orc_normalize_rows(_p(x), int(outer), int(inner), ctypes.c_float(eps), _p(mean), _p(var),
                             _p(temp), _p(out))
    return out


# --------------------------------------------------------------------------
# operator level: argument checks and shape rules of shadow/operators/*_op.cpp
# --------------------------------------------------------------------------
def unary_op(x, operation):
    """shadow/operators/unary_op.cpp:9-28"""
    _check(0 <= operation <= 14, "operation_ in [0, 14]")
    x = _f(x)
    return unary(operation, x.ravel()).reshape(x.shape)


def binary_op(a, b=None, operation=-1, scalar=None):
    """shadow/operators/binary_op.cpp:9-65; `scalar` given selects the one-input form."""
    _check(0 <= operation <= 6, "operation_ in [0, 6]")
    a = _f(a)
    if scalar is not None:
        _check(b is None, "inputs.size() == 1")
        return binary_scalar(operation, a.ravel(), scalar).reshape(a.shape)
    _check(b is not None, "inputs.size() == 2")
    b = _f(b)
    if a.shape == b.shape:
        return binary(operation, a.ravel(), b.ravel()).reshape(a.shape)
    sa, sb = list(a.shape), list(b.shape)
    diff = len(sa) - len(sb)
    if diff > 0:
        sb = [1] * diff + sb
    elif diff < 0:
        sa = [1] * (-diff) + sa
    out_shape = []
    for da, db in zip(sa, sb):
        _check(da == db or da == 1 or db == 1, "in_dim == scalar_dim || in_dim == 1 || scalar_dim == 1")
        out_shape.append(max(da, db))
    out = broadcast_binary(operation, a.ravel(), sa, b.ravel(), sb, out_shape)
    return out.reshape(out_shape)


def eltwise_op(inputs, operation, coeff=()):
    """shadow/operators/eltwise_op.cpp:9-47"""
    _check(0 <= operation <= 3, "operation_ in [0, 3]")
    _check(len(inputs) >= 2, "inputs.size() >= 2")
    inputs = [_f(x) for x in inputs]
    for x in inputs[1:]:
        _check(x.shape == inputs[0].shape, "inputs[n]->shape() == input_0->shape()")
    coeff = list(coeff)
    _check(len(coeff) == 0 or len(coeff) == len(inputs), "one coefficient per input blob")
    _check(not (operation != 1 and len(coeff)), "coefficients only for summation")
    full = [1.0] * len(inputs)
    full[:len(coeff)] = coeff
    return eltwise(operation, [x.ravel() for x in inputs], full).reshape(inputs[0].shape)


def reduce_op(x, operation=0, axes=(), keep_dims=True):
    """shadow/operators/reduce_op.cpp:9-65 (non-negative, distinct axes only: the
    reference indexes its stride table with the raw axis value)."""
    _check(0 <= operation <= 6, "operation_ in [0, 6]")
    x = _f(x)
    axes = list(axes)
    if not axes:
        axes = list(range(x.ndim))
    for ax in axes:
        _check(0 <= ax < x.ndim, "axis in range")
    out, out_shape = reduce(operation, x.ravel(), list(x.shape), axes)
    if not keep_dims:
        out_shape = [d for n, d in enumerate(out_shape) if n not in axes]
    return out.reshape(out_shape)


def activate_op(x, act_type=1, slope=0.1, slope_blob=None):
    """shadow/operators/activate_op.cpp:9-34 and kernels/activate.hpp:44-74"""
    _check(0 <= act_type <= 8, "activate_type_ in [0, 8]")
    x = _f(x)
    if act_type == 0:
        _check(slope_blob is not None, "inputs.size() == 2")
        _check(x.ndim >= 2, "input->num_axes() >= 2")
        slope_blob = _f(slope_blob)
        shared = slope_blob.size == 1
        if not shared:
            _check(slope_blob.size == x.shape[1], "slope->count() == input->shape(1)")
        return prelu(x.ravel(), list(x.shape), shared, slope_blob.ravel()).reshape(x.shape)
    _check(slope_blob is None, "inputs.size() == 1")
    return activate(x.ravel(), act_type, slope).reshape(x.shape)


def scale_op(x, axis=1, scale=None, bias=None, scale_value=(), bias_value=()):
    """shadow/operators/scale_op.cpp:9-52 and kernels/scale.hpp:44-110.
    Blob form when `scale`/`bias` arrays are given, value form otherwise."""
    x = _f(x)
    count = lambda start: int(np.prod(x.shape[start:], dtype=np.int64))
    if scale is not None or bias is not None:
        ref = _f(scale if scale is not None else bias)
        if scale is not None and bias is not None:
            _check(np.shape(scale) == np.shape(bias), "scale->shape() == bias->shape()")
        inner = count(axis + ref.ndim)
        out = scale_bias(x.ravel(), None if scale is None else _f(scale).ravel(),
                         None if bias is None else _f(bias).ravel(), ref.size, inner)
        return out.reshape(x.shape)
    dim = x.shape[axis]
    sv, bv = list(scale_value), list(bias_value)
    if len(sv) > 1:
        _check(len(sv) == dim, "scale_value_.size() == dim")
    elif len(sv) == 1:
        sv = sv * dim
    if len(bv) > 1:
        _check(len(bv) == dim, "bias_value_.size() == dim")
    elif len(bv) == 1:
        bv = bv * dim
    _check(sv or bv, "!scale_value.empty() || !bias_value.empty()")
    out = scale_bias(x.ravel(), np.float32(sv) if sv else None, np.float32(bv) if bv else None,
                     dim, count(axis + 1))
    return out.reshape(x.shape)


def axpy_op(alpha, x, y):
    """shadow/operators/axpy_op.cpp:25-46"""
    alpha, x, y = _f(alpha), _f(x), _f(y)
    _check(alpha.shape[0] == x.shape[0], "alpha->shape(0) == x->shape(0)")
    _check(alpha.shape[1] == x.shape[1], "alpha->shape(1) == x->shape(1)")
    if alpha.ndim == 4:
        _check(alpha.shape[2] == 1 and alpha.shape[3] == 1, "alpha->shape(2/3) == 1")
    _check(x.shape == y.shape, "x->shape() == y->shape()")
    inner = int(np.prod(x.shape[2:], dtype=np.int64))
    return axpy_rows(alpha, x, y, inner).reshape(x.shape)


def batch_norm_op(x, mean, variance, scale=None, eps=1e-5, use_global_stats=True):
    """shadow/operators/batch_norm_op.cpp:9-40 and kernels/batch_norm.hpp:36-48"""
    _check(use_global_stats, "use_global_stats")
    x = _f(x)
    scale_factor = np.float32(1)
    if scale is not None:
        sc = _f(scale)
        _check(sc.size == 1, "inputs[3]->count() == 1")
        scale_factor = np.float32(0) if sc.ravel()[0] == 0 else np.float32(1) / sc.ravel()[0]
    channel = x.shape[1]
    _check(channel == np.size(mean), "channel == mean->count()")
    _check(channel == np.size(variance), "channel == variance->count()")
    inner = int(np.prod(x.shape[2:], dtype=np.int64))
    return batch_norm(x, mean, variance, channel, inner, scale_factor, np.float32(eps)).reshape(x.shape)


def lrn_op(x, local_size=5, alpha=1.0, beta=0.75, norm_region=0, k=1.0):
    """shadow/operators/lrn_op.cpp:9-33 and kernels/lrn.hpp:36-46; the input must be 4-D (the kernel
    reads in_shape[0..3]) with at least (local_size - 1) / 2 channels (fewer make the kernel's last
    loop write in front of its scale blob)."""
    _check(local_size % 2 == 1, "LRN only supports odd values for local_size")
    _check(norm_region == 0, "Currently only support norm region method: Across Channels!")
    x = _f(x)
    _check(x.ndim == 4, "4-D input")
    _check(x.shape[1] >= (local_size - 1) // 2, "in_c >= post_pad")
    out, _ = lrn(x, x.shape, local_size, alpha, beta, k)
    return out.reshape(x.shape)


def grid_sample_op(x, grid, mode=1, padding_mode=0):
    """shadow/operators/grid_sample_op.cpp:9-47: x [b, c, h, w], grid [b, out_h, out_w, 2] -> [b, c, out_h, out_w]"""
    _check(mode in (0, 1), "mode_ == 0 || mode_ == 1")
    _check(padding_mode in (0, 1), "padding_mode_ == 0 || padding_mode_ == 1")
    x, grid = _f(x), _f(grid)
    _check(x.ndim == 4 and grid.ndim == 4, "4-D input and grid")
    _check(x.shape[0] == grid.shape[0], "input->shape(0) == grid->shape(0)")
    _check(grid.shape[3] == 2, "grid->shape(3) == 2")
    out_shape = [x.shape[0], x.shape[1], grid.shape[1], grid.shape[2]]
    return grid_sample(x, x.shape, grid, mode, padding_mode, out_shape).reshape(out_shape)


def _canonical(axis, ndim):
    _check(-ndim <= axis < ndim, "axis in range")
    return axis + ndim if axis < 0 else axis


def softmax_op(x, axis=1):
    """shadow/operators/softmax_op.cpp:18-29 and kernels/softmax.hpp:29-41"""
    x = _f(x)
    axis = _canonical(axis, x.ndim)
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    return softmax(x, outer, x.shape[axis], inner).reshape(x.shape)


def normalize_op(x, p=2.0, axis=1, eps=1e-12):
    """shadow/operators/normalize_op.cpp:9-29 and kernels/normalize.hpp:29-38"""
    x = _f(x)
    axis = _canonical(axis, x.ndim)
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    return normalize(x, outer, x.shape[axis], inner, np.float32(p), np.float32(eps)).reshape(x.shape)


def ssd_normalize_op(x, scale=None, across_spatial=True, channel_shared=True, eps=1e-5):
    """shadow/operators/ssd_normalize_op.cpp:9-38 and kernels/ssd_normalize.hpp:36-83"""
    x = _f(x)
    _check(x.ndim >= 2, "SSDNormalize needs [batch, channel, ...]")
    spatial = int(np.prod(x.shape[2:], dtype=np.int64))
    if scale is not None:
        scale = _f(scale).ravel()
        if channel_shared:
            _check(scale.size == 1, "scale->count() == 1")
        else:
            _check(scale.size >= x.shape[1], "one scale value per channel")
    return ssd_normalize(x, x.shape[0], x.shape[1], spatial, across_spatial, channel_shared, np.float32(eps),
                         scale).reshape(x.shape)


def pooling_op(x, pool=0, kernel_size=(), stride=(1,), pad=(0,), global_pooling=False,
               full_pooling=True):
    """shadow/operators/pooling_op.cpp:28-95"""
    x = _f(x)
    _check(0 <= pool <= 1, "pool_type in [0, 1]")
    nsp = x.ndim - 2
    _check(nsp in (2, 3), "Only support 2D or 3D Pooling")
    kernel_size, stride, pad = list(kernel_size), list(stride), list(pad)
    if global_pooling:
        stride, pad = [1], [0]
        kernel_size = list(x.shape[2:])

    def expand(v):
        if len(v) == 1:
            return v * nsp
        _check(len(v) == nsp, "param.size() == num")
        return v

    kernel_size, stride, pad = expand(kernel_size), expand(stride), expand(pad)
    out_shape = list(x.shape)
    for n in range(nsp):
        out_shape[n + 2] = pooling_out_size(x.shape[n + 2], kernel_size[n], stride[n], pad[n],
                                            full_pooling)
    return pooling(x, x.shape, pool, kernel_size, stride, pad, out_shape).reshape(out_shape)


def group_norm_op(x, group=1, eps=1e-5, scale=None, bias=None):
    """shadow/operators/group_norm_op.cpp:9-43 and kernels/group_norm.hpp:41-86"""
    x = _f(x)
    _check(x.shape[1] % group == 0, "input->shape(1) % group == 0")
    _check((scale is None) == (bias is None), "inputs.size() == 3")
    outer = x.shape[0] * group
    out = normalize_rows(x, outer, x.size // outer, np.float32(eps))
    if scale is not None:
        channel, spatial = x.shape[1], int(np.prod(x.shape[2:], dtype=np.int64))
        _check(np.size(scale) == channel, "scale->count() == channel")
        _check(np.size(bias) == channel, "bias->count() == channel")
        out = scale_bias(out, _f(scale).ravel(), _f(bias).ravel(), channel, spatial)
    return out.reshape(x.shape)


def instance_norm_op(x, eps=1e-5, scale=None, bias=None):
    """shadow/operators/instance_norm_op.cpp:9-36: GroupNorm with one group per channel"""
    return group_norm_op(x, _f(x).shape[1], eps, scale, bias)


def layer_norm_op(x, normalized_shape, eps=1e-5, scale=None, bias=None):
    """shadow/operators/layer_norm_op.cpp:9-45 and kernels/layer_norm.hpp:22-69"""
    x = _f(x)
    ns = list(normalized_shape)
    _check(len(ns) > 0, "!normalized_shape.empty()")
    _check(len(ns) <= x.ndim and list(x.shape[x.ndim - len(ns):]) == ns,
           "input->shape(n - size) == normalized_shape[n]")
    _check((scale is None) == (bias is None), "inputs.size() == 3")
    inner = int(np.prod(ns, dtype=np.int64))
    out = normalize_rows(x, x.size // inner, inner, np.float32(eps))
    if scale is not None:
        _check(list(np.shape(scale)) == ns, "scale->shape() == normalized_shape")
        _check(list(np.shape(bias)) == ns, "bias->shape() == normalized_shape")
        out = scale_bias(out, _f(scale).ravel(), _f(bias).ravel(), inner, 1)
    return out.reshape(x.shape)


# --------------------------------------------------------------------------
# data movers (operator level; the kernel classes' loops over inputs / outputs
# are folded in)
# --------------------------------------------------------------------------
def _count(shape, start=0, end=None):
    return int(np.prod(list(shape)[start:end], dtype=np.int64))


def concat_op(inputs, axis=1):
    """shadow/operators/concat_op.cpp:18-40 and kernels/concat.hpp:24-40"""
    inputs = [_f(x) for x in inputs]
    _check(len(inputs) >= 2, "inputs.size() >= 2")
    first = inputs[0]
    axis = _canonical(axis, first.ndim)
    out_shape = list(first.shape)
    for x in inputs[1:]:
        _check(x.ndim == first.ndim, "Inputs must have the same axes!")
        for d in range(first.ndim):
            if d != axis:
                _check(x.shape[d] == first.shape[d], "Inputs must have the same shape, except at concat_axis!")
        out_shape[axis] += x.shape[axis]
    out = np.empty(_count(out_shape), np.float32)
    num_concats, concat_size, offset = _count(out_shape, 0, axis), _count(out_shape, axis + 1), 0
    for x in inputs:
        lib().orc_concat(_p(x), num_concats, concat_size, out_shape[axis], x.shape[axis], offset, _p(out))
        offset += x.shape[axis]
    return out.reshape(out_shape)


def slice_op(x, num_outputs, axis=1, slice_point=()):
    """shadow/operators/slice_op.cpp:20-55 and kernels/slice.hpp:24-40"""
    x = _f(x)
    _check(num_outputs >= 2, "outputs.size() >= 2")
    axis = _canonical(axis, x.ndim)
    extent = x.shape[axis]
    if not slice_point:
        _check(extent % num_outputs == 0, "in_slice_axis % num_outputs == 0")
        slices = [extent // num_outputs] * num_outputs
    else:
        _check(len(slice_point) == num_outputs - 1, "slice_point_.size() == num_outputs - 1")
        slices, prev = [], 0
        for point in slice_point:
            _check(point > prev, "point > prev")
            slices.append(point - prev)
            prev = point
        _check(extent > prev, "in_slice_axis > prev")
        slices.append(extent - prev)
    outs, offset = [], 0
    num_slices, slice_size = _count(x.shape, 0, axis), _count(x.shape, axis + 1)
    for width in slices:
        shape = list(x.shape)
        shape[axis] = width
        out = np.empty(_count(shape), np.float32)
        lib().orc_slice(_p(x), num_slices, slice_size, extent, width, offset, _p(out))
        outs.append(out.reshape(shape))
        offset += width
    return outs


def stack_op(inputs, axis=0):
    """shadow/operators/stack_op.cpp:18-37 and kernels/stack.hpp:23-36"""
    inputs = [_f(x) for x in inputs]
    _check(len(inputs) >= 2, "inputs.size() >= 2")
    rank = inputs[0].ndim
    _check(-(rank + 1) <= axis < rank + 1, "axis out of bound.")
    if axis < 0:
        axis += rank + 1
    out_shape = list(inputs[0].shape)
    out_shape.insert(axis, len(inputs))
    out = np.empty(_count(out_shape), np.float32)
    num_stacks, stack_size = _count(out_shape, 0, axis), _count(out_shape, axis + 1)
    for n, x in enumerate(inputs):
        lib().orc_stack(_p(x), num_stacks, stack_size, len(inputs), n, _p(out))
    return out.reshape(out_shape)


def gather_op(x, axis=0, indexes=()):
    """shadow/operators/gather_op.cpp:20-48 and kernels/gather.hpp:25-34"""
    x = _f(x)
    axis = _canonical(axis, x.ndim)
    idx = np.ascontiguousarray(indexes, np.int32).ravel()
    _check(idx.size > 0, "num_indexes > 0")
    out_shape = list(x.shape)
    out_shape[axis] = idx.size
    out = np.empty(_count(out_shape), np.float32)
    lib().orc_gather(_p(x), idx.ctypes.data_as(_i32p), idx.size, x.shape[axis], _count(x.shape, axis + 1),
                     out.size, _p(out))
    return out.reshape(out_shape)


def pad_op(x, paddings, value=0.0):
    """shadow/operators/pad_op.cpp:11-37 and kernels/pad.hpp:24-40"""
    x = _f(x)
    paddings = [int(p) for p in paddings]
    _check(len(paddings) == 4, "paddings_.size() == 4")
    out_shape = list(x.shape)
    out_shape[2] += paddings[0] + paddings[1]
    out_shape[3] += paddings[2] + paddings[3]
    _check(min(out_shape) > 0, "output extents > 0")
    if not any(paddings):
        return copy(x.ravel()).reshape(x.shape)
    out = np.empty(_count(out_shape), np.float32)
    lib().orc_pad(_p(x), _ints(x.shape), _ints(paddings), _ints(out_shape), ctypes.c_float(value), _p(out))
    return out.reshape(out_shape)


def permute_op(x, order):
    """shadow/operators/permute_op.cpp:17-33 and kernels/permute.hpp:26-52"""
    x = _f(x)
    order = [int(o) for o in order]
    _check(len(order) == x.ndim, "input->num_axes() == order_value_.size()")
    out_shape = [x.shape[a] for a in order]
    old_steps = [_count(x.shape, d + 1) for d in range(x.ndim)]
    new_steps = [_count(out_shape, d + 1) for d in range(x.ndim)]
    out = np.empty(x.size, np.float32)
    lib().orc_permute(_p(x), x.size, x.ndim, _ints(order), _ints(old_steps), _ints(new_steps), _p(out))
    return out.reshape(out_shape)


def reorg_op(x, type=0, stride=2):
    """shadow/operators/reorg_op.cpp:19-41"""
    x = _f(x)
    c, h, w = x.shape[1:4]
    if type == 0:
        _check(c % (stride * stride) == 0, "in_c % (stride * stride) == 0")
    _check(h % stride == 0 and w % stride == 0, "in_h, in_w % stride == 0")
    out_shape = [x.shape[0], c * stride * stride, h // stride, w // stride]
    out = np.empty(x.size, np.float32)
    _check(lib().orc_reorg(_p(x), _ints(x.shape), int(type), int(stride), _p(out)) == 0, "Unsupported reorg type")
    return out.reshape(out_shape)


def shuffle_channel_op(x, group):
    """shadow/operators/shuffle_channel_op.cpp:9-32"""
    x = _f(x)
    _check(group > 0, "group must be larger than 0")
    _check(x.shape[1] % group == 0, "input->shape(1) % group == 0")
    out = np.empty(x.size, np.float32)
    lib().orc_shuffle_channel(_p(x), x.shape[0], x.shape[1], _count(x.shape, 2), int(group), _p(out))
    return out.reshape(x.shape)


def resize_op(x, size=(0,), scale=(1.0,), type=1, align_corners=False):
    """shadow/operators/resize_op.cpp:21-62 and kernels/resize.hpp:28-50"""
    x = _f(x)
    _check(0 <= type <= 1, "type in [0, 1]")
    _check(x.ndim == 4, "Only support 2D Resize")

    def expand(v):
        v = list(v)
        if len(v) == 1:
            return v * 2
        _check(len(v) == 2, "param.size() == num")
        return v

    size, scale = expand(size), expand(scale)
    out_shape = list(x.shape)
    for n in range(2):
        out_shape[n + 2] = size[n] if size[n] > 0 else int(np.float32(x.shape[n + 2]) * np.float32(scale[n]))
        _check(out_shape[n + 2] > 0, "out_shape > 0")
    if out_shape[2:] == list(x.shape[2:]):
        return copy(x.ravel()).reshape(x.shape)
    out = np.empty(_count(out_shape), np.float32)
    if type == 0:
        lib().orc_resize_nearest(_p(x), _ints(x.shape), _ints(out_shape), _p(out))
    else:
        lib().orc_resize_bilinear(_p(x), _ints(x.shape), int(bool(align_corners)), _ints(out_shape), _p(out))
    return out.reshape(out_shape)
