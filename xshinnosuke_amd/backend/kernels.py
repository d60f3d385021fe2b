"""Array-level wrappers of the conv / max-pool entry points.

Each function takes and returns :class:`DeviceArray` values, checks shapes on
the host before anything is launched, and raises ``ValueError`` for geometry
the reference would also reject.
"""
import ctypes

import numpy as np

from .capi import lib, CONV_RELU, CONV_BF16
from .array import DeviceArray, Workspace, empty

_ws = Workspace()


def conv_out_hw(h, w, r, s, stride, pad):
    if stride[0] < 1 or stride[1] < 1 or pad < 0:
        raise ValueError("stride must be positive and padding non-negative (got %s, %s)" % (stride, pad))
    return (h + 2 * pad - r) // stride[0] + 1, (w + 2 * pad - s) // stride[1] + 1


def _dims(x_shape, w_shape, stride, pad):
    n, c, h, w = x_shape
    k, c2, r, s = w_shape
    if c2 != c:
        raise ValueError("conv2d: input has %d channels, weight expects %d" % (c, c2))
    return [int(v) for v in (n, c, h, w, k, r, s, stride[0], stride[1], pad)]


def _workspace(dims):
    need = lib.raw("xsmi_conv2d_workspace_bytes")(*dims)
    return _ws.get(need)


def _f32(a, what):
    if not isinstance(a, DeviceArray) or a.dtype != np.float32:
        raise TypeError("%s must be a float32 DeviceArray" % what)
    return a


def conv2d_fwd(x, w, bias=None, stride=(1, 1), pad=0, relu=False, out=None, neg_mask=None, bf16=False):
    _f32(x, "x"); _f32(w, "w")
    dims = _dims(x.shape, w.shape, stride, pad)
    n, c, h, wd, k, r, s = dims[:7]
    oh, ow = conv_out_hw(h, wd, r, s, stride, pad)
    if oh <= 0 or ow <= 0:
        raise ValueError("conv2d: filter %dx%d does not fit the padded input %dx%d" % (r, s, h + 2 * pad, wd + 2 * pad))
    if bias is not None:
        _f32(bias, "bias")
        if bias.size != k:
            raise ValueError("conv2d: bias has %d elements for %d filters" % (bias.size, k))
    if out is None:
        out = empty((n, k, oh, ow))
    elif out.shape != (n, k, oh, ow):
        raise ValueError("conv2d: out has shape %s, expected %s" % (out.shape, (n, k, oh, ow)))
    if neg_mask is not None and (neg_mask.dtype != np.uint8 or neg_mask.size != out.size):
        raise ValueError("conv2d: neg_mask must be uint8 with one byte per output element")
    flags = (CONV_RELU if relu else 0) | (CONV_BF16 if bf16 else 0)
    ws, ws_bytes = _workspace(dims)
    lib.call("xsmi_conv2d_fwd", x.cptr, w.cptr, bias.cptr if bias is not None else None, out.cptr,
             neg_mask.cptr if neg_mask is not None else None, *dims, flags, ws, ws_bytes)
    return out


def conv2d_bwd_data(dy, w, x_shape, stride=(1, 1), pad=0, dx=None, accumulate=False, bf16=False):
    _f32(dy, "dy"); _f32(w, "w")
    dims = _dims(x_shape, w.shape, stride, pad)
    n, c, h, wd, k, r, s = dims[:7]
    oh, ow = conv_out_hw(h, wd, r, s, stride, pad)
    if dy.shape != (n, k, oh, ow):
        raise ValueError("conv2d backward: dy has shape %s, expected %s" % (dy.shape, (n, k, oh, ow)))
    if dx is None:
        dx = empty(x_shape)
        accumulate = False
    elif dx.shape != tuple(x_shape):
        raise ValueError("conv2d backward: dx has shape %s, expected %s" % (dx.shape, tuple(x_shape)))
    ws, ws_bytes = _workspace(dims)
    lib.call("xsmi_conv2d_bwd_data", dy.cptr, w.cptr, dx.cptr, *dims, 1.0 if accumulate else 0.0,
             CONV_BF16 if bf16 else 0, ws, ws_bytes)
    return dx


def conv2d_bwd_weight(dy, x, w_shape, stride=(1, 1), pad=0, dw=None, db=None, accumulate=False, want_db=False,
                      bf16=False):
    _f32(dy, "dy"); _f32(x, "x")
    dims = _dims(x.shape, w_shape, stride, pad)
    n, c, h, wd, k, r, s = dims[:7]
    oh, ow = conv_out_hw(h, wd, r, s, stride, pad)
    if dy.shape != (n, k, oh, ow):
        raise ValueError("conv2d backward: dy has shape %s, expected %s" % (dy.shape, (n, k, oh, ow)))
    if dw is None:
        dw = empty(w_shape)
        if db is None and want_db:
            db = empty((k,))
        accumulate = False
    elif dw.shape != tuple(w_shape):
        raise ValueError("conv2d backward: dw has shape %s, expected %s" % (dw.shape, tuple(w_shape)))
    if db is not None and db.size != k:
        raise ValueError("conv2d backward: db has %d elements for %d filters" % (db.size, k))
    ws, ws_bytes = _workspace(dims)
    lib.call("xsmi_conv2d_bwd_weight", dy.cptr, x.cptr, dw.cptr, db.cptr if db is not None else None, *dims,
             1.0 if accumulate else 0.0, CONV_BF16 if bf16 else 0, ws, ws_bytes)
    return dw, db


def pool_out_hw(h, w, k, stride, pad):
    if stride[0] < 1 or stride[1] < 1 or pad < 0:
        raise ValueError("stride must be positive and padding non-negative (got %s, %s)" % (stride, pad))
    return (h + 2 * pad - k) // stride[0] + 1, (w + 2 * pad - k) // stride[1] + 1


def maxpool2d_fwd(x, k, stride, pad=0, out=None, idx=None, want_idx=True):
    _f32(x, "x")
    n, c, h, w = x.shape
    oh, ow = pool_out_hw(h, w, k, stride, pad)
    if oh <= 0 or ow <= 0:
        raise ValueError("max_pool2d: window %d does not fit the padded input %dx%d" % (k, h + 2 * pad, w + 2 * pad))
    if out is None:
        out = empty((n, c, oh, ow))
    elif out.shape != (n, c, oh, ow):
        raise ValueError("max_pool2d: out has shape %s, expected %s" % (out.shape, (n, c, oh, ow)))
    if idx is None and want_idx:
        idx = empty((n, c, oh, ow), np.uint8)
    lib.call("xsmi_maxpool2d_fwd", x.cptr, out.cptr, idx.cptr if idx is not None else None,
             n, c, h, w, int(k), int(stride[0]), int(stride[1]), int(pad))
    return out, idx


def maxpool2d_bwd(dy, idx, x_shape, k, stride, pad=0, dx=None, accumulate=False):
    _f32(dy, "dy")
    n, c, h, w = x_shape
    oh, ow = pool_out_hw(h, w, k, stride, pad)
    if dy.shape != (n, c, oh, ow) or idx.size != dy.size or idx.dtype != np.uint8:
        raise ValueError("max_pool2d backward: dy/idx do not match the pooled shape %s" % ((n, c, oh, ow),))
    if dx is None:
        dx = empty(x_shape)
        accumulate = False
    elif dx.shape != tuple(x_shape):
        raise ValueError("max_pool2d backward: dx has shape %s, expected %s" % (dx.shape, tuple(x_shape)))
    lib.call("xsmi_maxpool2d_bwd", dy.cptr, idx.cptr, dx.cptr, n, c, h, w, int(k), int(stride[0]), int(stride[1]),
             int(pad), 1.0 if accumulate else 0.0)
    return dx


def relu_mask_bwd(dy, neg_mask, dx=None, accumulate=False):
    _f32(dy, "dy")
    if dx is None:
        dx = empty(dy.shape)
        accumulate = False
    lib.call("xsmi_relu_mask_bwd", dy.cptr, neg_mask.cptr, dx.cptr, dy.size, 1.0 if accumulate else 0.0)
    return dx


def copy_kernel(dst, src):
    lib.call("xsmi_copy_kernel", dst.cptr, src.cptr, src.nbytes)
