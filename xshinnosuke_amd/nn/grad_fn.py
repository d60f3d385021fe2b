"""Backward functions.  Each is a plain ``fn(outputs: Tensor) -> None`` stored in
``out.grad_fn`` that ACCUMULATES into the gradients of ``outputs.in_bounds``
(the convention of the reference's xs/nn/grad_fn.py).

``Conv2DBackward`` and ``Maxpool2DBackward`` are the hot-path pair: they always
run the HIP kernels of libxsmi355.so (there is no NumPy route for them); host
tensors are staged through device memory.
"""
import numpy as np

from ..core.base import Tensor, Parameter, is_device  # noqa: F401
from ..core import state as GLOBAL
from ..backend import kernels as K, to_device
from ..backend import array as dev
from . import array_ops as A


def initialize_ops_grad(*ops):
    """Give every input that needs a gradient a zero buffer (reference xs/utils/common.py:29-32)."""
    for op in ops:
        if op is not None and op.grad is None and op.requires_grad:
            op.zero_grad()


def _accumulate(t, g):
    """t.grad += g for host or device gradients."""
    dst = t.grad.eval
    if is_device(dst):
        g = A.same_place(dst, g)
        K.axpy(dst, g.reshape(dst.shape), 1.0)
    else:
        g = g.numpy() if is_device(g) else np.asarray(g)
        np.add(dst, g.reshape(dst.shape), out=dst)


def _product_into_fresh_grad(t, a, b, trans_a=False, trans_b=False):
    """t.grad = op(a) @ op(b) written straight into a device gradient whose clear is still pending (nothing to add
    to, so no temporary and no copy); False when that is not the situation."""
    dst = t.grad.eval
    if not (is_device(dst) and is_device(a) and is_device(b) and dst.is_fresh()):
        return False
    if any(v.dtype != np.float32 for v in (dst, a, b)) or len(a.shape) != 2 or len(b.shape) != 2:
        return False
    m = a.shape[1] if trans_a else a.shape[0]
    n = b.shape[0] if trans_b else b.shape[1]
    if dst.size != m * n:
        return False
    dst.take_fresh()
    K.gemm(a, b, trans_a=trans_a, trans_b=trans_b, out=dst)
    return True


def _f32_device(a):
    """Device float32 copy of a host array (or the device array itself)."""
    if is_device(a):
        return a
    return to_device(np.ascontiguousarray(a), np.float32)


# --------------------------------------------------------------------------- hot path
def Conv2DBackward(outputs):
    """dW, db, dX of conv2d (replaces reference xs/nn/grad_fn.py:186-203).

    Reads ``outputs.grad``, ``outputs.in_bounds == [inputs, weight, bias-or-None]`` and
    ``outputs.cache['stride'|'padding'|'x']``; adds into the inputs' gradients.
    """
    inputs, weight, bias = outputs.in_bounds
    stride, pad = outputs.cache['stride'], outputs.cache['padding']
    bf16 = bool(outputs.cache.get('bf16', False))
    x_dev = outputs.cache['x']                      # device copy of the forward input (stands in for 'col')
    dy = _f32_device(outputs.grad.eval)
    neg_mask = outputs.cache.get('neg_mask')
    if neg_mask is not None:                        # fused ReLU epilogue: strict mask, gradient passes at exactly 0
        dy = K.relu_mask_bwd(dy, neg_mask)
    w_dev = _f32_device(weight.eval)
    want_dw = weight.requires_grad
    want_db = bias is not None and bias.requires_grad
    if want_dw and inputs.requires_grad:
        dw_buf, dx_buf = weight.grad.eval, inputs.grad.eval
        db_buf = bias.grad.eval if want_db else None
        if is_device(dw_buf) and is_device(dx_buf) and (not want_db or is_device(db_buf)):
            # all gradients live on the device: one call; the weight gradient keeps running on the second
            # stream beside the rest of the sweep (the backend joins it before anything else can touch it)
            K.conv2d_bwd(dy, x_dev, w_dev, dx_buf, dw_buf, db_buf.reshape(-1) if want_db else None, stride, pad,
                         accumulate=True, bf16=bf16, async_dw=True, keep_layout=w_dev is weight.eval)
            return
    if want_dw or want_db:
        dw_buf = weight.grad.eval if want_dw else None
        db_buf = bias.grad.eval if want_db else None
        if want_dw and is_device(dw_buf) and (not want_db or is_device(db_buf)):
            K.conv2d_bwd_weight(dy, x_dev, weight.shape, stride, pad, dw=dw_buf,
                                db=db_buf.reshape(-1) if want_db else None, accumulate=True)
        else:
            dw, db = K.conv2d_bwd_weight(dy, x_dev, weight.shape, stride, pad, want_db=want_db)
            if want_dw:
                _accumulate(weight, dw)
            if want_db:
                _accumulate(bias, db)
    if inputs.requires_grad:
        dx_buf = inputs.grad.eval
        if is_device(dx_buf):
            K.conv2d_bwd_data(dy, w_dev, inputs.shape, stride, pad, dx=dx_buf, accumulate=True, bf16=bf16,
                              keep_layout=w_dev is weight.eval)
        else:
            _accumulate(inputs, K.conv2d_bwd_data(dy, w_dev, inputs.shape, stride, pad, bf16=bf16))


def Maxpool2DBackward(outputs):
    """Routes the upstream gradient to each window's first maximum (replaces reference
    xs/nn/grad_fn.py:206-235; only its unfold/argmax mode exists there in practice)."""
    inputs, = outputs.in_bounds
    if not inputs.requires_grad:
        return
    k, stride, pad = outputs.cache['kernel_size'], outputs.cache['stride'], outputs.cache['padding']
    idx = outputs.cache['pool_argmax']              # uint8 device array, NCHW order
    dy = _f32_device(outputs.grad.eval)
    dx_buf = inputs.grad.eval
    if is_device(dx_buf):
        K.maxpool2d_bwd(dy, idx, inputs.shape, k, stride, pad, dx=dx_buf, accumulate=True)
    else:
        # host gradient buffer: the kernel adds in float64 and rounds once, so upload the old value too
        old = _f32_device(dx_buf)
        K.maxpool2d_bwd(dy, idx, inputs.shape, k, stride, pad, dx=old, accumulate=True)
        dx_buf[...] = old.numpy()


# --------------------------------------------------------------------------- neighbours
def ReLUBackward(outputs):
    """Reference xs/nn/grad_fn.py:146-157, both the in-place and the out-of-place form."""
    if outputs.cache.get('inplace'):
        g, mask = outputs.grad.eval, outputs.cache['neg_mask_inplace']
        prev = outputs.cache['grad_fn'].pop()
        outputs.cache['inplace'] = bool(outputs.cache['grad_fn'])
        outputs.grad_fn = prev
        if prev is AddBackward and is_device(g) and not outputs.retain_grad() and _both_addends_on_device(outputs, g):
            # ReLU applied in place to a sum: the masked gradient goes to both addends in one pass
            a, b = outputs.in_bounds
            K.relu_mask_bwd2(g, mask, a.grad.eval, b.grad.eval, accumulate=True)
            return
        if is_device(g):
            K.relu_mask_bwd(g, mask, dx=g)                 # in place on the gradient
        else:
            g[mask] = 0
        if prev is not None:
            prev(outputs)
    else:
        inputs, = outputs.in_bounds
        if inputs.requires_grad:
            _accumulate(inputs, A.relu_grad(outputs.grad.eval, inputs.eval))


def SigmoidBackward(outputs):
    """Reference xs/nn/grad_fn.py:161-164."""
    inputs, = outputs.in_bounds
    if inputs.requires_grad:
        _accumulate(inputs, A.activation_grad(outputs.grad.eval, outputs.eval, 'sigmoid'))


def TanhBackward(outputs):
    """Reference xs/nn/grad_fn.py:167-170."""
    inputs, = outputs.in_bounds
    if inputs.requires_grad:
        _accumulate(inputs, A.activation_grad(outputs.grad.eval, outputs.eval, 'tanh'))


def _both_addends_on_device(outputs, g):
    """Two distinct addends of the output's shape that both want a gradient and keep it in aligned device memory."""
    if len(outputs.in_bounds) != 2:
        return False
    a, b = outputs.in_bounds
    if a is b or not (a.requires_grad and b.requires_grad):
        return False
    for t in (a, b):
        d = t.grad.eval if t.grad is not None else None
        if d is None or not is_device(d) or d.dtype != np.float32 or tuple(t.shape) != tuple(outputs.shape) or d.address() % 16:
            return False
    return a.grad.eval.address() != b.grad.eval.address() and g.address() % 16 == 0


def AddBackward(outputs):
    for t in outputs.in_bounds:
        if t.requires_grad:
            g = outputs.grad.eval
            if tuple(t.shape) != tuple(outputs.shape):
                g = A.sum_leading(g) if t.eval.size == outputs.shape[-1] else A.total(g)
            _accumulate(t, g)


def SubBackward(outputs):
    lhs, rhs = outputs.in_bounds
    if lhs.requires_grad:
        _accumulate(lhs, outputs.grad.eval)
    if rhs.requires_grad:
        _accumulate(rhs, A.scale(outputs.grad.eval, -1.0))


def MultiplyBackward(outputs):
    lhs, rhs = outputs.in_bounds
    g = outputs.grad.eval
    for a, b in ((lhs, rhs), (rhs, lhs)):
        if a.requires_grad:
            if is_device(g):
                raise NotImplementedError('element-wise product backward on device tensors')
            prod = g * b.eval
            if a.eval.size == 1:
                prod = np.asarray(prod.sum()).reshape(a.eval.shape)
            _accumulate(a, prod)


def PowBackward(outputs):
    inputs, = outputs.in_bounds
    if inputs.requires_grad:
        e = outputs.cache['exp']
        _accumulate(inputs, outputs.grad.eval * e * np.power(inputs.eval, e - 1))


def MMBackward(outputs):
    x1, x2 = outputs.in_bounds
    g = outputs.grad.eval
    if x1.requires_grad:
        if not _product_into_fresh_grad(x1, g, x2.eval, trans_b=True):
            _accumulate(x1, A.mm_nt(g, x2.eval))
    if x2.requires_grad:
        if not _product_into_fresh_grad(x2, x1.eval, g, trans_a=True):
            _accumulate(x2, A.mm_tn(x1.eval, g))


def AddmmBackward(outputs):
    """Reference xs/nn/grad_fn.py:86-99."""
    x1, x2, b = outputs.in_bounds
    g = outputs.grad.eval
    if b is not None and b.requires_grad:
        _accumulate(b, A.sum_leading(g) if b.eval.size != g.size else g)
    if x1.requires_grad:
        if not _product_into_fresh_grad(x1, g, x2.eval, trans_b=True):
            _accumulate(x1, A.mm_nt(g, x2.eval))
    if x2.requires_grad:
        if not _product_into_fresh_grad(x2, x1.eval, g, trans_a=True):
            _accumulate(x2, A.mm_tn(x1.eval, g))


def FlattenBackward(outputs):
    inputs, = outputs.in_bounds
    if inputs.requires_grad:
        _accumulate(inputs, outputs.grad.eval.reshape(inputs.shape))


ViewBackward = FlattenBackward


def SumBackward(outputs):
    inputs, = outputs.in_bounds
    if inputs.requires_grad:
        g = outputs.grad.eval
        if outputs.cache.get('axis') is None:
            val = float((g.numpy() if is_device(g) else np.asarray(g)).reshape(-1)[0])
            _accumulate(inputs, A.fill_like(inputs.eval, val))
        else:
            gh = g.numpy() if is_device(g) else np.asarray(g)
            if not outputs.cache['keepdims']:
                gh = np.expand_dims(gh, outputs.cache['axis'])
            _accumulate(inputs, np.broadcast_to(gh, inputs.shape).astype(gh.dtype))


def MeanBackward(outputs):
    inputs, = outputs.in_bounds
    if inputs.requires_grad:
        g = outputs.grad.eval
        gh = g.numpy() if is_device(g) else np.asarray(g)
        if outputs.cache.get('axis') is None:
            _accumulate(inputs, A.fill_like(inputs.eval, float(gh.reshape(-1)[0]) / inputs.eval.size))
        else:
            ax = outputs.cache['axis']
            if not outputs.cache['keepdims']:
                gh = np.expand_dims(gh, ax)
            _accumulate(inputs, (np.broadcast_to(gh, inputs.shape) / inputs.shape[ax]).astype(gh.dtype))


def Avgpool2DBackward(outputs):
    inputs, = outputs.in_bounds
    if inputs.requires_grad:
        _accumulate(inputs, A.avg_pool_blocks_grad(outputs.grad.eval, inputs.shape, outputs.cache['kernel_size'],
                                                    outputs.cache['stride']))


def _fresh_grad(t):
    """The gradient buffer of ``t`` if it is a device array still pending its clear, so that a kernel may
    write its result straight into it; None otherwise (the result then goes through _accumulate)."""
    if t is None or not t.requires_grad or t.grad is None:
        return None
    g = t.grad.eval
    return g if is_device(g) and g.take_fresh() else None


def BatchNormBackward(outputs):
    """Reference xs/nn/grad_fn.py:379-411."""
    inputs, gamma, beta = outputs.in_bounds
    dy = outputs.grad.eval
    if is_device(dy):
        out_dx, out_dg, out_db = _fresh_grad(inputs), _fresh_grad(gamma), _fresh_grad(beta)
        gam = A.same_place(dy, gamma.eval)
        xhat, mean = outputs.cache['normalized_x'], outputs.cache.get('batch_mean')
        if xhat is None:                             # not stored by the forward: x and the batch mean stand in
            xhat = inputs.eval
        dx, dgamma, dbeta = K.bn_bwd(dy, xhat, outputs.cache['sqrtvar'], gam,
                                     dx=out_dx, dgamma=None if out_dg is None else out_dg.reshape(-1),
                                     dbeta=None if out_db is None else out_db.reshape(-1),
                                     neg_mask=outputs.cache.get('neg_mask'),       # fused ReLU: strict mask on dy
                                     mean=mean if outputs.cache['normalized_x'] is None else None)
    else:
        out_dx = out_dg = out_db = None
        dx, dgamma, dbeta = A.batch_norm_backward(dy, outputs.cache['normalized_x'], outputs.cache['sqrtvar'], gamma.eval)
    if gamma.requires_grad and out_dg is None:
        _accumulate(gamma, dgamma)
    if beta.requires_grad and out_db is None:
        _accumulate(beta, dbeta)
    if inputs.requires_grad and out_dx is None:
        _accumulate(inputs, dx)


def CrossEntropyLossBackward(outputs):
    """Reference xs/nn/grad_fn.py:604-620."""
    logits, labels = outputs.in_bounds
    if not logits.requires_grad:
        return
    up = outputs.grad.eval
    if is_device(up) and not is_device(logits.cache['softmax'].eval):
        up = up.numpy()
    g = A.softmax_cross_entropy_grad(logits.cache['softmax'].eval, labels.eval, outputs.cache['reduction'], up)
    if logits.grad is None:
        logits.grad = Tensor(g)
    else:
        _accumulate(logits, g)


def MSELossBackward(outputs):
    pred, target = outputs.in_bounds
    if is_device(pred.eval):
        raise NotImplementedError('mse_loss backward on device tensors')
    up = float(np.asarray(outputs.grad.eval).reshape(-1)[0])
    diff = pred.eval - np.asarray(target.eval).reshape(pred.shape)
    if outputs.cache['reduction'] == 'mean':
        diff = diff / pred.eval.size
    g = diff * up                                   # the reference's loss is 0.5 * (pred - target)^2
    if pred.requires_grad:
        _accumulate(pred, g)
    if target.requires_grad:
        _accumulate(target, -g)
