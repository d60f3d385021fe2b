"""Array-level helpers for the ops that surround conv / max-pool in a network.

Each function accepts either host arrays (``numpy.ndarray``, computed with NumPy
like the reference's xs/nn/td_functional.py) or device arrays (computed by the
element-wise / reduction kernels of libxsmi355.so).  Conv and max-pool themselves
are not here: they always run on the device (``nn/functional.py``).
"""
import numpy as np

from ..backend import DeviceArray, kernels as K, to_device
from ..backend import array as dev


def is_device(a):
    return isinstance(a, DeviceArray)


def same_place(ref, a):
    """Bring ``a`` to where ``ref`` lives."""
    if is_device(ref):
        return a if is_device(a) else to_device(np.asarray(a), np.float32 if np.asarray(a).dtype.kind == 'f' else None)
    return a.numpy() if is_device(a) else a


def empty_like(a, shape=None):
    shape = a.shape if shape is None else shape
    return dev.empty(shape, a.dtype) if is_device(a) else np.empty(shape, dtype=a.dtype)


def zeros_like(a, shape=None):
    shape = a.shape if shape is None else shape
    return dev.zeros(shape, a.dtype) if is_device(a) else np.zeros(shape, dtype=a.dtype)


def iadd(dst, src):
    """dst += src (src broadcast over leading axes is summed by the caller)."""
    if is_device(dst):
        K.axpy(dst, same_place(dst, src), 1.0)
    else:
        np.add(dst, np.asarray(same_place(dst, src)).reshape(dst.shape), out=dst)


def add(a, b, out=None, defer=False):
    """``defer`` (device arrays, new result): see kernels.add."""
    if is_device(a):
        b = same_place(a, b)
        if b.size == a.size:
            return K.add(a, b, out, defer=defer)
        if b.size == 1:
            return K.add_scalar(a, float(b.numpy().reshape(-1)[0]), out)
        raise NotImplementedError('broadcast add of %s and %s on the device' % (a.shape, b.shape))
    r = np.add(a, same_place(a, b))
    if out is not None:
        out[...] = r
        return out
    return r


def relu(x, out=None):
    if is_device(x):
        return K.relu_fwd(x, out)
    r = np.maximum(0., x)
    if out is not None:
        out[...] = r
        return out
    return r.astype(x.dtype, copy=False)


def relu_grad(dy, pre):
    """dy where pre >= 0, else 0 -- the reference's strict mask (xs/nn/grad_fn.py:155-157)."""
    if is_device(dy):
        return K.relu_bwd(dy, pre)
    g = dy.copy()
    g[pre < 0] = 0
    return g


def activation(x, kind, out=None):
    """sigmoid / tanh as the reference computes them (xs/nn/td_functional.py:63-70)."""
    if is_device(x):
        return K.act_fwd(x, kind, out)
    r = 1. / (1. + np.exp(-x)) if kind == 'sigmoid' else np.tanh(x)
    if out is not None:
        out[...] = r
        return out
    return r.astype(x.dtype, copy=False)


def activation_grad(dy, y, kind):
    """dy * y * (1 - y) for sigmoid, dy * (1 - y^2) for tanh (xs/nn/grad_fn.py:161-170)."""
    if is_device(dy):
        return K.act_bwd(dy, same_place(dy, y), kind)
    y = np.asarray(same_place(dy, y))
    return dy * y * (1 - y) if kind == 'sigmoid' else dy * (1 - np.square(y))


def reshape(a, shape):
    return a.reshape(shape)


def addmm(x, w, b, out=None):
    """x @ w + b."""
    if is_device(x):
        return K.dense_fwd(x, same_place(x, w), None if b is None else same_place(x, b), out)
    r = np.dot(x, w)
    if b is not None:
        r = r + b
    if out is not None:
        out[...] = r
        return out
    return r


def mm_nt(a, b):
    """a @ b.T"""
    if is_device(a):
        return K.gemm(a, same_place(a, b), trans_b=True)
    return np.dot(a, b.T)


def mm_tn(a, b):
    """a.T @ b"""
    if is_device(a):
        return K.gemm(a, same_place(a, b), trans_a=True)
    return np.dot(a.T, b)


def sum_leading(a):
    """Sum over every axis but the last."""
    if is_device(a):
        return K.colsum(a.reshape(-1, a.shape[-1]))
    return a.reshape(-1, a.shape[-1]).sum(axis=0)


def total(a):
    if is_device(a):
        return K.sum_all(a)
    return np.asarray(a.sum()).reshape(1)


def scale(a, s):
    if is_device(a):
        return K.scale(a, float(s))
    return a * a.dtype.type(s)


def fill_like(a, value):
    if is_device(a):
        return to_device(np.full(a.shape, value, dtype=a.dtype), a.dtype)
    return np.full(a.shape, value, dtype=a.dtype)


def batch_norm_train(x, gamma, beta, eps, out=None, moving=None, momentum=0.0, neg_mask=None, want_xhat=True, defer=False):
    """Per-channel batch statistics over (N, H, W) or (N,).  Returns y, xhat, sqrtvar, mean, var.  A device
    ``out`` of the right size receives y directly; device ``moving`` statistics are updated by the same call
    (host ones are left to the caller).  On the device ``want_xhat=False`` returns None for xhat: the backward
    then takes x and the mean; ``defer``: see kernels.bn_fwd."""
    if is_device(x):
        y = out if (out is not None and is_device(out) and out.size == x.size) else None
        return K.bn_fwd(x, same_place(x, gamma), same_place(x, beta), eps, y=y, moving=moving, momentum=momentum,
                        neg_mask=neg_mask, want_xhat=want_xhat, defer=defer)
    axes = tuple(i for i in range(x.ndim) if i != 1)
    mean = x.mean(axis=axes, keepdims=True)
    var = x.var(axis=axes, keepdims=True)
    sqrtvar = np.sqrt(var + eps)
    xhat = (x - mean) / sqrtvar
    bshape = [1] * x.ndim
    bshape[1] = -1
    y = gamma.reshape(bshape) * xhat + beta.reshape(bshape)
    return y.astype(x.dtype, copy=False), xhat, sqrtvar, mean.ravel(), var.ravel()


def batch_norm_infer(x, gamma, beta, mean, var, eps, out=None, relu=False):
    if is_device(x):
        y = out if (out is not None and is_device(out) and out.size == x.size) else None
        return K.bn_infer(x, same_place(x, gamma), same_place(x, beta), same_place(x, mean), same_place(x, var), eps, y=y,
                          relu=relu)
    bshape = [1] * x.ndim
    bshape[1] = -1
    y = (x - mean.reshape(bshape)) / np.sqrt(var.reshape(bshape) + eps)
    return (gamma.reshape(bshape) * y + beta.reshape(bshape)).astype(x.dtype, copy=False)


def batch_norm_backward(dy, xhat, sqrtvar, gamma):
    """Returns dx, dgamma, dbeta (formula of the reference, xs/nn/grad_fn.py:379-411)."""
    if is_device(dy):
        return K.bn_bwd(dy, xhat, sqrtvar, same_place(dy, gamma))
    axes = tuple(i for i in range(dy.ndim) if i != 1)
    m = int(np.prod([dy.shape[a] for a in axes]))
    bshape = [1] * dy.ndim
    bshape[1] = -1
    dgamma = (dy * xhat).sum(axis=axes)
    dbeta = dy.sum(axis=axes)
    dxh = dy * gamma.reshape(bshape)
    dx = (dxh * m - dxh.sum(axis=axes, keepdims=True) - xhat * (dxh * xhat).sum(axis=axes, keepdims=True)) / (m * sqrtvar)
    return dx, dgamma, dbeta


def avg_pool_blocks(x, k, stride=None):
    """Mean over k x k windows at the given stride (default k: non-overlapping blocks), no padding: the im2col
    mode of the reference's avg_pool2d, float64 sum and one rounding."""
    sh, sw = (k, k) if stride is None else stride
    if is_device(x):
        return K.avgpool_fwd(x, k, (sh, sw))
    n, c, h, w = x.shape
    oh, ow = (h - k) // sh + 1, (w - k) // sw + 1
    acc = np.zeros((n, c, oh, ow), dtype=np.float64)
    for ky in range(k):
        for kx in range(k):
            acc += x[:, :, ky:ky + sh * oh:sh, kx:kx + sw * ow:sw]
    return (acc / (k * k)).astype(x.dtype, copy=False)


def avg_pool_blocks_grad(dy, x_shape, k, stride=None):
    """Every window hands dy / k^2 (rounded to dy's dtype, as the reference forms it) to its cells; overlapping
    windows add up in float64 in (ky, kx) order (the reference's col2im), rounded once."""
    sh, sw = (k, k) if stride is None else stride
    if is_device(dy):
        return K.avgpool_bwd(dy, x_shape, k, (sh, sw))
    n, c, h, w = x_shape
    oh, ow = dy.shape[2], dy.shape[3]
    share = (dy / dy.dtype.type(k * k)).astype(np.float64)
    g = np.zeros(x_shape, dtype=np.float64)
    for ky in range(k):
        for kx in range(k):
            g[:, :, ky:ky + sh * oh:sh, kx:kx + sw * ow:sw] += share
    return g.astype(dy.dtype, copy=False)


def softmax_cross_entropy(logits, labels, reduction):
    """Returns (loss array of shape (1,), softmax)."""
    if is_device(logits):
        return K.softmax_ce_fwd(logits, same_place(logits, labels), reduction)
    z = logits - logits.max(axis=-1, keepdims=True)
    e = np.exp(z)
    sm = e / e.sum(axis=-1, keepdims=True)
    lab = np.asarray(labels).astype(np.int64).reshape(-1)
    nll = -np.log(sm.reshape(-1, sm.shape[-1])[np.arange(lab.size), lab])
    loss = nll.mean() if reduction == 'mean' else nll.sum()
    return np.asarray(loss, dtype=logits.dtype).reshape(1), sm.astype(logits.dtype, copy=False)


def softmax_cross_entropy_grad(sm, labels, reduction, upstream):
    """(softmax - onehot) * upstream [/ N for 'mean']."""
    if is_device(sm):
        return K.softmax_ce_bwd(sm, same_place(sm, labels), reduction, upstream)
    g = sm.reshape(-1, sm.shape[-1]).copy()
    lab = np.asarray(labels).astype(np.int64).reshape(-1)
    g[np.arange(lab.size), lab] -= 1
    if reduction == 'mean':
        g /= sm.shape[0]
    g *= np.asarray(upstream).reshape(-1)[0]
    return g.reshape(sm.shape)


def sgd_step_all(pairs, lr):
    """param -= lr * grad for every (param, grad) pair; the device-resident pairs share one launch."""
    dev_p, dev_g = [], []
    for param, grad in pairs:
        if is_device(param) and is_device(grad) and param.dtype == np.float32 and grad.dtype == np.float32:
            dev_p.append(param); dev_g.append(grad)
        else:
            sgd_step(param, grad, lr)
    K.axpy_multi(dev_p, dev_g, -float(lr))
    K.refresh_layouts(dev_p)                      # filters among them: their kernels' layouts, made beside what follows


def sgd_step(param, grad, lr):
    """param -= lr * grad (reference xs/optim/sgd.py:4-9)."""
    if is_device(param):
        K.axpy(param, same_place(param, grad), -float(lr))
    else:
        param -= lr * np.asarray(same_place(param, grad)).reshape(param.shape)
