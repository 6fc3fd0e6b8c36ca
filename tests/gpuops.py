"""Thin numpy-in / numpy-out wrappers over the C ABI for the GPU tests.

Every helper uploads its operands, calls exactly one ``shdw_hip_*`` entry point
on the null stream, synchronises and downloads the result."""
import ctypes

import numpy as np

import shadow_amd
from shadow_amd import Buffer, check, ints


def _lib():
    return shadow_amd.hip()


def _sync():
    check(_lib().shdw_hip_stream_sync(None))


def _f(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def set_(n, val):
    y = Buffer(4 * n)
    check(_lib().shdw_hip_set(n, val, y.ptr, None))
    _sync()
    return y.download(count=n)


def unary(op, x, inplace=False, offset=0):
    """offset (in floats) shifts both pointers off 16-byte alignment."""
    x = _f(x).ravel()
    n = x.size
    a = Buffer(4 * (n + offset))
    a.upload(x, 4 * offset)
    y = a if inplace else Buffer(4 * (n + offset))
    check(_lib().shdw_hip_unary(op, n, a.ptr + 4 * offset, y.ptr + 4 * offset, None))
    _sync()
    return y.download(count=n, offset_bytes=4 * offset)


def binary(op, a, b, inplace=False):
    a, b = _f(a).ravel(), _f(b).ravel()
    da, db = Buffer.from_numpy(a), Buffer.from_numpy(b)
    y = da if inplace else Buffer(a.nbytes)
    check(_lib().shdw_hip_binary(op, a.size, da.ptr, db.ptr, y.ptr, None))
    _sync()
    return y.download(count=a.size)


def binary_scalar(op, a, alpha):
    a = _f(a).ravel()
    da = Buffer.from_numpy(a)
    y = Buffer(a.nbytes)
    check(_lib().shdw_hip_binary_scalar(op, a.size, da.ptr, alpha, y.ptr, None))
    _sync()
    return y.download(count=a.size)


def scal(alpha, x):
    x = _f(x).ravel()
    d = Buffer.from_numpy(x)
    check(_lib().shdw_hip_scal(x.size, alpha, d.ptr, None))
    _sync()
    return d.download(count=x.size)


def copy(x):
    x = _f(x).ravel()
    d = Buffer.from_numpy(x)
    y = Buffer(x.nbytes)
    check(_lib().shdw_hip_copy(x.size, d.ptr, y.ptr, None))
    _sync()
    return y.download(count=x.size)


def axpy(alpha, x, y):
    x, y = _f(x).ravel(), _f(y).ravel()
    dx, dy = Buffer.from_numpy(x), Buffer.from_numpy(y)
    check(_lib().shdw_hip_axpy(x.size, alpha, dx.ptr, dy.ptr, None))
    _sync()
    return dy.download(count=x.size)


def reduce_workspace(shape, axes):
    return _lib().shdw_hip_reduce_workspace_bytes(len(shape), ints(shape), len(axes), ints(axes))


def asum(x):
    x = _f(x).ravel()
    d = Buffer.from_numpy(x)
    need = reduce_workspace([x.size], [0]) + 16
    ws = Buffer(need)
    out = ctypes.c_float(0)
    check(_lib().shdw_hip_asum(x.size, d.ptr, ctypes.byref(out), ws.ptr, need, None))
    return np.float32(out.value)


def broadcast_binary(op, a, a_shape, b, b_shape, out_shape):
    a, b = _f(a).ravel(), _f(b).ravel()
    da, db = Buffer.from_numpy(a), Buffer.from_numpy(b)
    n = int(np.prod(out_shape, dtype=np.int64))
    y = Buffer(4 * n)
    check(_lib().shdw_hip_broadcast_binary(op, len(out_shape), ints(a_shape), ints(b_shape),
                                           ints(out_shape), da.ptr, db.ptr, y.ptr, None))
    _sync()
    return y.download(count=n)


def activate(x, act_type, slope=0.1, inplace=False):
    x = _f(x).ravel()
    d = Buffer.from_numpy(x)
    y = d if inplace else Buffer(x.nbytes)
    check(_lib().shdw_hip_activate(act_type, slope, x.size, d.ptr, y.ptr, None))
    _sync()
    return y.download(count=x.size)


def prelu(x, shape, channel_shared, slope):
    x, slope = _f(x).ravel(), _f(slope).ravel()
    channels = shape[1]
    dim = int(np.prod(shape[2:], dtype=np.int64))
    d, ds = Buffer.from_numpy(x), Buffer.from_numpy(slope)
    y = Buffer(x.nbytes)
    check(_lib().shdw_hip_prelu(x.size, channels, dim, int(bool(channel_shared)), d.ptr, ds.ptr,
                                y.ptr, None))
    _sync()
    return y.download(count=x.size)


def scale_bias(x, scale, bias, scale_num, inner_num, relu=False, inplace=False, offset=0):
    x = _f(x).ravel()
    n = x.size
    d = Buffer(4 * (n + offset))
    d.upload(x, 4 * offset)
    ds = Buffer.from_numpy(_f(scale)) if scale is not None else None
    db = Buffer.from_numpy(_f(bias)) if bias is not None else None
    y = d if inplace else Buffer(4 * (n + offset))
    check(_lib().shdw_hip_scale_bias(n, scale_num, inner_num, d.ptr + 4 * offset,
                                     ds.ptr if ds else None, db.ptr if db else None,
                                     int(relu), y.ptr + 4 * offset, None))
    _sync()
    return y.download(count=n, offset_bytes=4 * offset)


def eltwise(op, inputs, coeff=None, alias=None, relu=False):
    """alias = index of the input whose buffer is also the output; relu: the fused Eltwise + Activate entry."""
    inputs = [_f(x).ravel() for x in inputs]
    n = inputs[0].size
    bufs = [Buffer.from_numpy(x) for x in inputs]
    y = bufs[alias] if alias is not None else Buffer(4 * n)
    ptrs = (ctypes.c_void_p * len(bufs))(*[b.ptr for b in bufs])
    co = None
    if coeff is not None:
        co = (ctypes.c_float * len(coeff))(*[float(c) for c in coeff])
    fn = _lib().shdw_hip_eltwise_relu if relu else _lib().shdw_hip_eltwise
    check(fn(op, len(bufs), ptrs, co, n, y.ptr, None))
    _sync()
    return y.download(count=n)


def reduce(op, x, shape, axes):
    x = _f(x).ravel()
    d = Buffer.from_numpy(x)
    out_shape = list(shape)
    for ax in axes:
        out_shape[ax] = 1
    n_out = int(np.prod(out_shape, dtype=np.int64))
    y = Buffer(4 * n_out)
    need = reduce_workspace(shape, axes)
    ws = Buffer(need) if need else None
    check(_lib().shdw_hip_reduce(op, len(shape), ints(shape), len(axes), ints(axes), d.ptr, y.ptr,
                                 ws.ptr if ws else None, need, None))
    _sync()
    return y.download(count=n_out), out_shape


def scale_residual_relu_rowmean(x, scale, bias, res, scale_num, inner_num, want_y=True):
    x, res = _f(x).ravel(), _f(res).ravel()
    n = x.size
    dx, dr = Buffer.from_numpy(x), Buffer.from_numpy(res)
    ds, db = Buffer.from_numpy(_f(scale)), Buffer.from_numpy(_f(bias))
    y = Buffer(4 * n) if want_y else None
    rows = n // inner_num
    mean = Buffer(4 * rows)
    check(_lib().shdw_hip_scale_residual_relu_rowmean(n, scale_num, inner_num, dx.ptr, ds.ptr,
                                                      db.ptr, dr.ptr, y.ptr if y else None,
                                                      mean.ptr, None))
    _sync()
    return (y.download(count=n) if y else None), mean.download(count=rows)


def scale_residual_relu(x, scale, bias, res, scale_num, inner_num, residual_first=False, want_y=True, want_mean=True):
    """shdw_hip_scale_residual_relu: scale or bias may be None, either output may be left out."""
    x, res = _f(x).ravel(), _f(res).ravel()
    n = x.size
    dx, dr = Buffer.from_numpy(x), Buffer.from_numpy(res)
    ds = Buffer.from_numpy(_f(scale)) if scale is not None else None
    db = Buffer.from_numpy(_f(bias)) if bias is not None else None
    y = Buffer(4 * n) if want_y else None
    rows = n // inner_num
    mean = Buffer(4 * rows) if want_mean else None
    check(_lib().shdw_hip_scale_residual_relu(n, scale_num, inner_num, dx.ptr, ds.ptr if ds else None,
                                              db.ptr if db else None, dr.ptr, int(residual_first),
                                              y.ptr if y else None, mean.ptr if mean else None, None))
    _sync()
    return (y.download(count=n) if y else None), (mean.download(count=rows) if mean else None)


def batch_norm_scale_residual_relu(x, stat_mean, stat_variance, scale_factor, eps, scale, bias, res, channel, inner_num,
                                   residual_first=False, want_y=True, want_mean=True):
    """shdw_hip_batch_norm_scale_residual_relu: scale or bias may be None, either output may be left out."""
    x, res = _f(x).ravel(), _f(res).ravel()
    n = x.size
    dx, dr = Buffer.from_numpy(x), Buffer.from_numpy(res)
    dm, dv = Buffer.from_numpy(_f(stat_mean)), Buffer.from_numpy(_f(stat_variance))
    ds = Buffer.from_numpy(_f(scale)) if scale is not None else None
    db = Buffer.from_numpy(_f(bias)) if bias is not None else None
    y = Buffer(4 * n) if want_y else None
    rows = n // inner_num
    mean = Buffer(4 * rows) if want_mean else None
    check(_lib().shdw_hip_batch_norm_scale_residual_relu(
        n, channel, inner_num, dx.ptr, dm.ptr, dv.ptr, float(scale_factor), float(eps), ds.ptr if ds else None,
        db.ptr if db else None, dr.ptr, int(residual_first), y.ptr if y else None, mean.ptr if mean else None, None))
    _sync()
    return (y.download(count=n) if y else None), (mean.download(count=rows) if mean else None)


def grid_sample(x, in_shape, grid, mode, padding_mode, out_shape):
    x, grid = _f(x).ravel(), _f(grid).ravel()
    n_out = int(np.prod(out_shape, dtype=np.int64))
    assert x.size == int(np.prod(in_shape, dtype=np.int64)) and grid.size == 2 * out_shape[0] * out_shape[2] * out_shape[3]
    dx, dg = Buffer.from_numpy(x), Buffer.from_numpy(grid)
    y = Buffer(max(4, 4 * n_out))
    check(_lib().shdw_hip_grid_sample(ints(in_shape), ints(out_shape), int(mode), int(padding_mode), dx.ptr, dg.ptr,
                                      y.ptr, None))
    _sync()
    return y.download(count=n_out)


def lrn(x, in_shape, size, alpha, beta, k, inplace=False):
    x = _f(x).ravel()
    dx = Buffer.from_numpy(x)
    y = dx if inplace else Buffer(max(4, x.nbytes))
    check(_lib().shdw_hip_lrn(ints(in_shape), int(size), float(alpha), float(beta), float(k), dx.ptr, y.ptr, None))
    _sync()
    return y.download(count=x.size)


def axpy_rows(alpha, x, y, inner_num, inplace=False):
    alpha, x, y = _f(alpha).ravel(), _f(x).ravel(), _f(y).ravel()
    da, dx, dy = Buffer.from_numpy(alpha), Buffer.from_numpy(x), Buffer.from_numpy(y)
    out = dy if inplace else Buffer(max(4, x.nbytes))
    check(_lib().shdw_hip_axpy_rows(alpha.size, inner_num, da.ptr, dx.ptr, dy.ptr, out.ptr, None))
    _sync()
    return out.download(count=x.size)


def batch_norm(x, mean, variance, channel, inner_num, scale_factor, eps, inplace=False):
    x = _f(x).ravel()
    dx, dm, dv = Buffer.from_numpy(x), Buffer.from_numpy(_f(mean)), Buffer.from_numpy(_f(variance))
    y = dx if inplace else Buffer(max(4, x.nbytes))
    check(_lib().shdw_hip_batch_norm(x.size, channel, inner_num, dx.ptr, dm.ptr, dv.ptr,
                                     scale_factor, eps, y.ptr, None))
    _sync()
    return y.download(count=x.size)


def batch_norm_scale(x, mean, variance, channel, inner_num, scale_factor, eps, scale, bias, relu, inplace=False):
    """BatchNorm -> Scale [-> ReLU] in one launch; scale or bias may be None."""
    x = _f(x).ravel()
    dx, dm, dv = Buffer.from_numpy(x), Buffer.from_numpy(_f(mean)), Buffer.from_numpy(_f(variance))
    ds = Buffer.from_numpy(_f(scale)) if scale is not None else None
    db = Buffer.from_numpy(_f(bias)) if bias is not None else None
    y = dx if inplace else Buffer(max(4, x.nbytes))
    check(_lib().shdw_hip_batch_norm_scale(x.size, channel, inner_num, dx.ptr, dm.ptr, dv.ptr, scale_factor, eps,
                                           ds.ptr if ds else None, db.ptr if db else None, 1 if relu else 0,
                                           y.ptr, None))
    _sync()
    return y.download(count=x.size)


def _shifted(x, offset, inplace, n_out=None):
    """x on the device `offset` floats into its buffer, and the output buffer likewise."""
    dx = Buffer(max(4, x.nbytes) + 4 * offset)
    dx.upload(x, 4 * offset)
    n_out = x.size if n_out is None else n_out
    y = dx if inplace else Buffer(max(4, 4 * n_out) + 4 * offset)
    return dx, y


def softmax(x, outer, dim, inner, inplace=False, offset=0):
    """offset (in floats) shifts both pointers off 16-byte alignment."""
    x = _f(x).ravel()
    dx, y = _shifted(x, offset, inplace)
    check(_lib().shdw_hip_softmax(outer, dim, inner, dx.ptr + 4 * offset, y.ptr + 4 * offset, None))
    _sync()
    return y.download(count=x.size, offset_bytes=4 * offset)


def normalize(x, outer, dim, inner, p, eps, inplace=False, offset=0):
    x = _f(x).ravel()
    dx, y = _shifted(x, offset, inplace)
    check(_lib().shdw_hip_normalize(outer, dim, inner, p, eps, dx.ptr + 4 * offset, y.ptr + 4 * offset, None))
    _sync()
    return y.download(count=x.size, offset_bytes=4 * offset)


def ssd_normalize(x, batch, channel, spatial, across_spatial, channel_shared, eps, scale=None, inplace=False,
                  offset=0):
    x = _f(x).ravel()
    dx, y = _shifted(x, offset, inplace)
    ds = None if scale is None else Buffer.from_numpy(_f(scale).ravel())
    nbytes = _lib().shdw_hip_ssd_normalize_workspace_bytes(batch, channel, spatial, int(across_spatial))
    ws = Buffer(nbytes) if nbytes else None
    check(_lib().shdw_hip_ssd_normalize(batch, channel, spatial, int(across_spatial), eps, dx.ptr + 4 * offset,
                                        ds.ptr if ds else None, int(channel_shared), y.ptr + 4 * offset,
                                        ws.ptr if ws else None, None))
    _sync()
    return y.download(count=x.size, offset_bytes=4 * offset)


def pooling(x, in_shape, pool_type, kernel, stride, pad, out_shape, offset=0):
    """2-D or 3-D by len(kernel)."""
    x = _f(x).ravel()
    n_out = int(np.prod(out_shape, dtype=np.int64))
    dx, y = _shifted(x, offset, False, n_out)
    fn = _lib().shdw_hip_pooling2d if len(kernel) == 2 else _lib().shdw_hip_pooling3d
    check(fn(ints(in_shape), pool_type, *kernel, *stride, *pad, ints(out_shape), dx.ptr + 4 * offset,
             y.ptr + 4 * offset, None))
    _sync()
    return y.download(count=n_out, offset_bytes=4 * offset)


def group_norm(x, outer, inner, eps, scale=None, bias=None, scale_num=1, scale_inner=1, inplace=False,
               offset=0, scratch=False):
    """offset (in floats) shifts x and y off 16-byte alignment; scratch: through the entry
    point that takes the caller's scratch memory (sliced rows where they are long and few)."""
    x = _f(x).ravel()
    dx = Buffer(4 * (x.size + offset) + 16)
    dx.upload(x, 4 * offset)
    y = dx if inplace else Buffer(4 * (x.size + offset) + 16)
    ds = Buffer.from_numpy(_f(scale)) if scale is not None else None
    db = Buffer.from_numpy(_f(bias)) if bias is not None else None
    if scratch:
        need = _lib().shdw_hip_group_norm_workspace_bytes(outer, inner)
        ws = Buffer(need) if need else None
        check(_lib().shdw_hip_group_norm_ws(outer, inner, eps, dx.ptr + 4 * offset, ds.ptr if ds else None,
                                            db.ptr if db else None, scale_num, scale_inner,
                                            y.ptr + 4 * offset, ws.ptr if ws else None, need, None))
    else:
        check(_lib().shdw_hip_group_norm(outer, inner, eps, dx.ptr + 4 * offset, ds.ptr if ds else None,
                                         db.ptr if db else None, scale_num, scale_inner,
                                         y.ptr + 4 * offset, None))
    _sync()
    return y.download(count=x.size, offset_bytes=4 * offset)
