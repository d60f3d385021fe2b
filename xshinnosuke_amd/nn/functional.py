"""Functional API (counterpart of the reference's xs/nn/functional.py).

``conv2d`` and ``max_pool2d`` keep the reference signatures, graph wiring,
``cache`` keys and accumulate-into-grad convention, but their arithmetic is done
by the HIP kernels of libxsmi355.so -- for device tensors in place, for host
(NumPy-backed) tensors by staging through device memory.  There is no NumPy
implementation of these two ops in this package: without the library or a
gfx950 device they raise.

The remaining functions are the small set of neighbours the README networks and
ResNet-18 need; they run in NumPy for host tensors and through element-wise /
reduction kernels for device tensors.
"""
import weakref

import numpy as np

from ..core import state as GLOBAL
from ..core.base import Tensor, Parameter, is_device
from ..backend import kernels as K, to_device
from ..backend import array as dev
from . import array_ops as A
from .grad_fn import *  # noqa: F401,F403  (backward functions are part of this module's namespace, as in the reference)
from .grad_fn import initialize_ops_grad, _f32_device


# Folded (conv + inference batch norm) filters kept between forwards, keyed by the conv's weight Parameter.  They
# live here and not on the Parameter: a checkpoint pickles the graph, and a kept filter holds device addresses
# that mean nothing in another process.
_FOLDED = weakref.WeakKeyDictionary()


def _mark_input(t):
    if GLOBAL.INPUTS is None:
        GLOBAL.INPUTS = t


def _wire(out, *ins):
    """Dynamic-graph bookkeeping: out.in_bounds = ins (None kept as a placeholder), ins[i].out_bounds += out."""
    if out.is_dynamic:
        if out.in_bounds:                # a reused output tensor (forward without backward): re-wire, do not append
            del out.in_bounds[:]
        out.add_in_bounds(*ins)
        for t in ins:
            if t is not None:
                t.add_out_bounds(out)


def _pair(v):
    if isinstance(v, (tuple, list)):
        return int(v[0]), int(v[1])
    return int(v), int(v)


# --------------------------------------------------------------------------- hot path
def conv2d(inputs, weight, bias=None, stride=(1, 1), padding=0, out=None, activation=None):
    """2-D cross-correlation, NCHW (reference xs/nn/functional.py:405-442).

    ``stride`` is a pair, ``padding`` one symmetric int, no dilation or groups.  Output
    ``(N, K, (H+2p-R)//sh+1, (W+2p-S)//sw+1)`` has the dtype of ``inputs``.  ``out`` may be a
    preallocated (possibly batch-sliced) Tensor that is written in place.
    ``activation='relu'`` is this package's extension: it fuses ``max(0, .)`` into the
    kernel epilogue (what ``Conv2D(activation='relu')`` computes in the reference with a
    second pass, xs/layers/convolutional.py:76-77) and keeps the strict ``pre < 0`` mask
    for the backward.
    """
    _mark_input(inputs)
    if activation not in (None, 'relu'):
        raise ValueError("conv2d can only fuse activation='relu'")
    x = inputs.eval
    if len(x.shape) != 4 or len(weight.shape) != 4:
        raise ValueError('conv2d expects NCHW input and KCRS weight, got %s and %s' % (x.shape, weight.shape))
    stride = _pair(stride)
    if isinstance(padding, (tuple, list)) or int(padding) != padding:
        raise TypeError('padding must be a single integer')
    padding = int(padding)
    on_device = is_device(x)
    x_dev = _f32_device(x)
    w_dev = _f32_device(weight.eval)
    b_dev = None if bias is None else _f32_device(bias.eval).reshape(-1)
    n, c, h, w = x.shape
    k, _, r, s = weight.shape
    oh, ow = K.conv_out_hw(h, w, r, s, stride, padding)
    requires_grad = bool(inputs.requires_grad or weight.requires_grad or (bias is not None and bias.requires_grad))
    track = GLOBAL.COMPUTE_GRAD and requires_grad
    neg_mask = dev.empty((n, k, oh, ow), np.uint8) if (activation == 'relu' and track) else None
    bf16 = bool(GLOBAL.CONV_BF16)

    # without gradients a bf16 result may stay in channels-last form for the next bf16 consumer (DeviceArray.channels_last)
    cl = bf16 and not track and on_device
    # a tracked forward on a device-resident filter is a training step's: the filter's layout is kept between calls
    keep = track and w_dev is weight.eval
    if out is None:
        y_dev = K.conv2d_fwd(x_dev, w_dev, b_dev, stride, padding, relu=activation == 'relu', neg_mask=neg_mask, bf16=bf16,
                             channels_last=cl, keep_layout=keep)
        out = Tensor(y_dev if on_device else y_dev.numpy().astype(x.dtype, copy=False))
    else:
        dst = out.eval
        if is_device(dst):
            K.conv2d_fwd(x_dev, w_dev, b_dev, stride, padding, relu=activation == 'relu', out=dst, neg_mask=neg_mask, bf16=bf16,
                         channels_last=cl, keep_layout=keep)
        else:
            y_dev = K.conv2d_fwd(x_dev, w_dev, b_dev, stride, padding, relu=activation == 'relu', neg_mask=neg_mask, bf16=bf16)
            out.eval = y_dev.numpy()              # cast to the buffer's dtype on store
    out.requires_grad = requires_grad
    _wire(out, inputs, weight, bias)
    if track:
        out.cache['x'] = x_dev                    # the reference keeps the unfolded matrix 'col' here
        out.cache['stride'] = stride
        out.cache['bf16'] = bf16
        out.cache['padding'] = padding
        if neg_mask is not None:
            out.cache['neg_mask'] = neg_mask
        out.grad_fn = Conv2DBackward
        initialize_ops_grad(inputs, weight, bias)
    return out


def conv2d_batch_norm_inference(inputs, weight, bias, stride, padding, gamma, beta, moving_mean, moving_variance,
                                epsilon=1e-5, out=None, activation=None):
    """``batch_norm(conv2d(inputs, ...), ..., training=False)`` (and the ReLU after it) on device tensors as ONE
    convolution: with given statistics the normalisation is a per-filter scale and shift, which is folded into the
    filter and the bias first (this package's extension; values equal the two-step form up to float rounding).
    Forward only: the result carries no ``grad_fn``."""
    _mark_input(inputs)
    if activation not in (None, 'relu'):
        raise ValueError("conv2d_batch_norm_inference can only fuse activation='relu'")
    x = inputs.eval
    if not is_device(x):
        raise NotImplementedError('the folded convolution needs device tensors')
    if len(x.shape) != 4 or len(weight.shape) != 4:
        raise ValueError('conv2d expects NCHW input and KCRS weight, got %s and %s' % (x.shape, weight.shape))
    stride = _pair(stride)
    padding = int(padding)
    dst = out.eval if (out is not None and is_device(out.eval)) else None
    bf16 = bool(GLOBAL.CONV_BF16)
    relu = activation == 'relu'
    sources = [t.eval for t in (weight, bias, gamma, beta, moving_mean, moving_variance) if t is not None]
    kept = _FOLDED.get(weight)
    x = _f32_device(x)
    if all(is_device(a) and a.dtype == np.float32 for a in sources):
        # Frozen parameters: the folded filter, its bias and its packed form (in a workspace of this filter's own) are
        # kept while nobody has taken the address of a parameter since they were made (DeviceArray.state).
        # (the batch size is part of the key: it decides which kernel, hence which packed layout, the library picks)
        # (and so is the count of step-graph recordings and replays: those change parameters without taking addresses)
        now = (tuple(a.state() for a in sources), float(epsilon), bf16, stride, padding, tuple(x.shape), dev._EPOCH[0])
        need = K.conv2d_workspace_bytes(x.shape, weight.shape, stride, padding)
        if kept is not None and kept['key'] == now and kept['ws'].holds(need):
            y = K.conv2d_fwd(x, kept['w'], kept['b'], stride, padding, relu=relu, out=dst, bf16=bf16, packed=True,
                             workspace=kept['ws'], channels_last=bf16)
        else:
            stats = [a.reshape(-1) for a in sources[-4:]]
            b_dev = None if bias is None else bias.eval.reshape(-1)
            w2, b2 = K.bn_fold(weight.eval, b_dev, *stats, epsilon)
            ws = kept['ws'] if kept is not None else K.Workspace()
            y = K.conv2d_fwd(x, w2, b2, stride, padding, relu=relu, out=dst, bf16=bf16, workspace=ws, channels_last=bf16)
            # the fold has read the parameters: their state as of now is what the kept filter belongs to
            key = (tuple(a.state() for a in sources), float(epsilon), bf16, stride, padding, tuple(x.shape), dev._EPOCH[0])
            _FOLDED[weight] = {'key': key, 'w': w2, 'b': b2, 'ws': ws, 'of': sources}   # 'of' keeps the ids in the key alive
    else:
        stats = [_f32_device(t.eval).reshape(-1) for t in (gamma, beta, moving_mean, moving_variance)]
        b_dev = None if bias is None else _f32_device(bias.eval).reshape(-1)
        w2, b2 = K.bn_fold(_f32_device(weight.eval), b_dev, *stats, epsilon)
        y = K.conv2d_fwd(x, w2, b2, stride, padding, relu=relu, out=dst, bf16=bf16, channels_last=bf16)
    if out is None:
        out = Tensor(y)
    elif y is not dst:
        out.eval = y
    out.requires_grad = False
    out.grad_fn = None                               # a reused output tensor may carry one from a tracked forward
    _wire(out, inputs, weight, bias)
    return out


def max_pool2d(inputs, kernel_size=2, stride=None, padding=0, out=None):
    """Max pooling with zero-valued padding that takes part in the max and first-maximum
    tie-breaking (reference xs/nn/functional.py:445-491).

    ``kernel_size`` is an int (an equal pair is accepted, which the reference's README
    shows but its code rejects); ``stride`` defaults to the kernel size.
    """
    _mark_input(inputs)
    if isinstance(kernel_size, (tuple, list)):
        if len(kernel_size) != 2 or kernel_size[0] != kernel_size[1]:
            raise ValueError('max_pool2d supports square windows only')
        kernel_size = kernel_size[0]
    kernel_size = int(kernel_size)
    stride = (kernel_size, kernel_size) if stride is None else _pair(stride)
    padding = int(padding)
    x = inputs.eval
    if len(x.shape) != 4:
        raise ValueError('max_pool2d expects an NCHW input, got shape %s' % (x.shape,))
    on_device = is_device(x)
    x_dev = _f32_device(x)
    track = GLOBAL.COMPUTE_GRAD and inputs.requires_grad
    if out is None:
        y_dev, idx = K.maxpool2d_fwd(x_dev, kernel_size, stride, padding, want_idx=track)
        out = Tensor(y_dev if on_device else y_dev.numpy().astype(x.dtype, copy=False))
    else:
        dst = out.eval
        if is_device(dst):
            _, idx = K.maxpool2d_fwd(x_dev, kernel_size, stride, padding, out=dst, want_idx=track)
        else:
            y_dev, idx = K.maxpool2d_fwd(x_dev, kernel_size, stride, padding, want_idx=track)
            out.eval = y_dev.numpy()
    out.requires_grad = inputs.requires_grad
    _wire(out, inputs)
    if track:
        out.cache['pool_argmax'] = idx            # uint8, NCHW order, value ky*k + kx
        out.cache['kernel_size'] = kernel_size
        out.cache['mode'] = 'im2col'
        out.cache['stride'] = stride
        out.cache['padding'] = padding
        out.grad_fn = Maxpool2DBackward
        initialize_ops_grad(inputs)
    return out


# --------------------------------------------------------------------------- neighbours
def _binary(lhs, rhs, fn, backward_fn, out):
    _mark_input(lhs)
    res = fn(lhs.eval, rhs.eval, None if out is None else out.eval)
    if out is None:
        out = Tensor(res)
    out.requires_grad = bool(lhs.requires_grad or rhs.requires_grad)
    _wire(out, lhs, rhs)
    if GLOBAL.COMPUTE_GRAD and out.requires_grad:
        initialize_ops_grad(lhs, rhs)
        out.grad_fn = backward_fn
    return out


def add(lhs, rhs, out=None):
    # The launch of a device add into a new tensor is held back until the next operation: the in-place ReLU of a
    # residual block then computes max(0, lhs + rhs) (and its sign mask) in one pass; anything else sees the plain
    # sum (see backend/kernels.add).
    return _binary(lhs, rhs, lambda a, b, o: A.add(a, b, o, defer=o is None), AddBackward, out)


def sub(lhs, rhs, out=None):
    def f(a, b, o):
        if is_device(a):
            return A.add(a, A.scale(A.same_place(a, b), -1.0), o)
        r = np.subtract(a, A.same_place(a, b))
        if o is not None:
            o[...] = r
            return o
        return r
    return _binary(lhs, rhs, f, SubBackward, out)


def mul(lhs, rhs, out=None):
    def f(a, b, o):
        if is_device(a):
            b = A.same_place(a, b)
            if b.size == 1:
                return A.scale(a, float(b.numpy().reshape(-1)[0]))
            raise NotImplementedError('element-wise product of device tensors')
        r = np.multiply(a, A.same_place(a, b))
        if o is not None:
            o[...] = r
            return o
        return r
    return _binary(lhs, rhs, f, MultiplyBackward, out)


def pow(inputs, exp, out=None):
    """Element-wise power with a Python scalar exponent (host tensors)."""
    _mark_input(inputs)
    if is_device(inputs.eval):
        raise NotImplementedError('pow on device tensors')
    res = np.power(inputs.eval, exp)
    out = Tensor(res)
    out.requires_grad = inputs.requires_grad
    _wire(out, inputs)
    if GLOBAL.COMPUTE_GRAD and out.requires_grad:
        out.cache['exp'] = exp
        out.grad_fn = PowBackward
        initialize_ops_grad(inputs)
    return out


def mm(x1, x2, out=None):
    _mark_input(x1)
    res = A.addmm(x1.eval, x2.eval, None, None if out is None else out.eval)
    if out is None:
        out = Tensor(res)
    out.requires_grad = bool(x1.requires_grad or x2.requires_grad)
    _wire(out, x1, x2)
    if GLOBAL.COMPUTE_GRAD and out.requires_grad:
        initialize_ops_grad(x1, x2)
        out.grad_fn = MMBackward
    return out


def addmm(b, x1, x2, out=None):
    """x1 @ x2 + b (reference xs/nn/functional.py:99-120); in_bounds order is (x1, x2, b)."""
    _mark_input(x1)
    res = A.addmm(x1.eval, x2.eval, None if b is None else b.eval, None if out is None else out.eval)
    if out is None:
        out = Tensor(res)
    out.requires_grad = bool(x1.requires_grad or x2.requires_grad or (b is not None and b.requires_grad))
    _wire(out, x1, x2, b)
    if GLOBAL.COMPUTE_GRAD and out.requires_grad:
        initialize_ops_grad(b, x1, x2)
        out.grad_fn = AddmmBackward
    return out


def relu(inputs, inplace=False, out=None):
    """max(0, x) (reference xs/nn/functional.py:297-313).  The in-place form overwrites ``inputs``
    and chains its backward in front of the tensor's existing grad_fn, as the reference's ReLU layer
    does (xs/layers/activators.py:37-50)."""
    _mark_input(inputs)
    if inplace:
        x = inputs.eval
        if GLOBAL.COMPUTE_GRAD and inputs.requires_grad:
            # the strict mask needs the sign of the pre-activation; y == 0 cannot tell x == 0 from x < 0
            if is_device(x):
                _, inputs.cache['neg_mask_inplace'] = K.relu_fwd_mask(x, x)
            else:
                inputs.cache['neg_mask_inplace'] = x < 0
                A.relu(x, x)
            inputs.cache.setdefault('grad_fn', []).append(inputs.grad_fn)
            inputs.cache['inplace'] = True
            inputs.grad_fn = ReLUBackward
        else:
            A.relu(x, x)
        return inputs
    res = A.relu(inputs.eval, None if out is None else out.eval)
    if out is None:
        out = Tensor(res)
    out.requires_grad = inputs.requires_grad
    _wire(out, inputs)
    if GLOBAL.COMPUTE_GRAD and out.requires_grad:
        out.grad_fn = ReLUBackward
        initialize_ops_grad(inputs)
    return out


def _activation(inputs, kind, backward_fn, out):
    _mark_input(inputs)
    res = A.activation(inputs.eval, kind, None if out is None else out.eval)
    if out is None:
        out = Tensor(res)
    out.requires_grad = inputs.requires_grad
    _wire(out, inputs)
    if GLOBAL.COMPUTE_GRAD and out.requires_grad:
        out.grad_fn = backward_fn
        initialize_ops_grad(inputs)
    return out


def sigmoid(inputs, out=None):
    """1 / (1 + exp(-x)) (reference xs/nn/functional.py:316-329)."""
    return _activation(inputs, 'sigmoid', SigmoidBackward, out)


def tanh(inputs, out=None):
    """Reference xs/nn/functional.py:332-345."""
    return _activation(inputs, 'tanh', TanhBackward, out)


def flatten(inputs, start=1, out=None):
    _mark_input(inputs)
    x = inputs.eval
    shape = tuple(x.shape[:start]) + (-1,)
    res = x.reshape(shape)
    if out is None:
        out = Tensor(res)
    else:
        out.eval = res
    out.requires_grad = inputs.requires_grad
    _wire(out, inputs)
    if GLOBAL.COMPUTE_GRAD and out.requires_grad:
        out.grad_fn = FlattenBackward
        initialize_ops_grad(inputs)
    return out


def view(inputs, shape, out=None):
    _mark_input(inputs)
    if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
        shape = tuple(shape[0])
    res = inputs.eval.reshape(tuple(shape))
    out = Tensor(res)
    out.requires_grad = inputs.requires_grad
    _wire(out, inputs)
    if GLOBAL.COMPUTE_GRAD and out.requires_grad:
        out.grad_fn = ViewBackward
        initialize_ops_grad(inputs)
    return out


def _reduce(inputs, axis, keepdims, mean):
    _mark_input(inputs)
    x = inputs.eval
    if axis is None:
        res = A.total(x)
        if mean:
            res = A.scale(res, 1.0 / x.size)
    else:
        xh = x.numpy() if is_device(x) else x
        res = (np.mean if mean else np.sum)(xh, axis=axis, keepdims=keepdims)
        res = A.same_place(x, np.asarray(res, dtype=xh.dtype))
    out = Tensor(res)
    out.requires_grad = inputs.requires_grad
    _wire(out, inputs)
    if GLOBAL.COMPUTE_GRAD and out.requires_grad:
        out.cache['axis'] = axis
        out.cache['keepdims'] = keepdims
        out.grad_fn = MeanBackward if mean else SumBackward
        initialize_ops_grad(inputs)
    return out


def sum(inputs, axis=None, keepdims=False):
    return _reduce(inputs, axis, keepdims, mean=False)


def mean(inputs, axis=None, keepdims=False):
    return _reduce(inputs, axis, keepdims, mean=True)


def avg_pool2d(inputs, kernel_size, stride=None, padding=0, out=None):
    """Mean over k x k windows at ``stride`` (default: the window size), reference xs/nn/functional.py:539-583 in
    its im2col mode, which is the only live one there (it compares the int window with the stride pair).  The
    reference's padded mode counts the padding twice in the output size and is not reproduced: padding must be 0."""
    _mark_input(inputs)
    k = int(kernel_size[0] if isinstance(kernel_size, (tuple, list)) else kernel_size)
    st = (k, k) if stride is None else _pair(stride)
    if padding != 0:
        raise NotImplementedError('avg_pool2d supports padding == 0 only')
    res = A.avg_pool_blocks(inputs.eval, k, st)
    if out is None:
        out = Tensor(res)
    else:
        out.eval = res
    out.requires_grad = inputs.requires_grad
    _wire(out, inputs)
    if GLOBAL.COMPUTE_GRAD and out.requires_grad:
        out.cache['kernel_size'] = k
        out.cache['mode'] = 'im2col'
        out.cache['stride'] = st
        out.cache['padding'] = padding
        out.grad_fn = Avgpool2DBackward
        initialize_ops_grad(inputs)
    return out


def batch_norm(inputs, gamma, beta, moving_mean, moving_variance, axis=1, training=True, epsilon=1e-5,
               momentum=0.9, out=None, activation=None):
    """Per-channel batch normalisation over axis 1 (reference xs/nn/functional.py:676-740).

    ``activation='relu'`` (device tensors only) is this package's extension, the counterpart of conv2d's: the
    ReLU that follows the normalisation is applied by the same kernel and its strict ``pre < 0`` mask is kept for
    the backward, which then needs no pass of its own either."""
    _mark_input(inputs)
    if axis != 1:
        raise NotImplementedError('batch_norm normalises over axis 1 only')
    x = inputs.eval
    if activation not in (None, 'relu'):
        raise ValueError("batch_norm can only fuse activation='relu'")
    if activation == 'relu' and not is_device(x):
        raise NotImplementedError('the fused ReLU needs device tensors')
    relu = activation == 'relu'
    xhat = sqrtvar = None
    dst = None if out is None else out.eval
    if training:
        mm, mv = moving_mean.eval, moving_variance.eval
        fused = is_device(x) and is_device(mm) and is_device(mv)      # the normalisation kernel updates them
        track = GLOBAL.COMPUTE_GRAD and bool(inputs.requires_grad or gamma.requires_grad or beta.requires_grad)
        neg_mask = dev.empty(x.shape, np.uint8) if relu else None
        # The device launch is held back until the next operation: at the end of a residual block that is the add of
        # the shortcut and then the in-place ReLU, behind the first convolution of a ResNet the 3x3/2 max-pool, and
        # either runs inside the normalisation's second pass (backend/kernels.bn_fwd); anything else sees the plain result.
        y, xhat, sqrtvar, mean_, var_ = A.batch_norm_train(x, gamma.eval, beta.eval, epsilon, dst,
                                                           (mm.reshape(-1), mv.reshape(-1)) if fused else None, momentum,
                                                           neg_mask, want_xhat=False,
                                                           defer=fused and track)
        if not track:
            neg_mask = None
        if not fused:
            for mov, cur in ((moving_mean, mean_), (moving_variance, var_)):
                m = mov.eval
                cur = A.same_place(m, cur)
                if is_device(m):
                    K.lerp_(m, cur, momentum)                   # m = momentum*m + (1-momentum)*cur
                else:
                    m *= momentum
                    m += (1 - momentum) * np.asarray(cur).reshape(m.shape)
    else:
        neg_mask = None
        y = A.batch_norm_infer(x, gamma.eval, beta.eval, moving_mean.eval, moving_variance.eval, epsilon, dst, relu)
    if out is None:
        out = Tensor(y)
    elif y is not dst:
        out.eval = y
    out.requires_grad = bool(inputs.requires_grad or gamma.requires_grad or beta.requires_grad)
    _wire(out, inputs, gamma, beta)
    if GLOBAL.COMPUTE_GRAD and out.requires_grad and training:
        out.cache['sqrtvar'] = sqrtvar
        out.cache['normalized_x'] = xhat
        # on the device the normalised input is not stored: the backward forms it again from x and the mean
        out.cache['batch_mean'] = mean_ if xhat is None else None
        if neg_mask is not None:
            out.cache['neg_mask'] = neg_mask
        else:
            out.cache.pop('neg_mask', None)
        out.grad_fn = BatchNormBackward
        initialize_ops_grad(inputs, gamma, beta)
    return out


def cross_entropy(x1, x2, reduction='mean', out=None):
    """Softmax + negative log-likelihood on integer labels (reference xs/nn/functional.py:984-1010)."""
    _mark_input(x1)
    if reduction not in ('mean', 'sum'):
        raise TypeError('unknown type for reduction')
    loss, sm = A.softmax_cross_entropy(x1.eval, x2.eval, reduction)
    x1.cache['softmax'] = Tensor(sm)
    if out is None:
        out = Tensor(loss)
    else:
        out.eval = loss
    _wire(out, x1, x2)
    if out.is_dynamic:
        out.is_leaf = True
    out.requires_grad = bool(x1.requires_grad or x2.requires_grad)
    if GLOBAL.COMPUTE_GRAD and out.requires_grad:
        out.cache['reduction'] = reduction
        out.grad_fn = CrossEntropyLossBackward
        initialize_ops_grad(x1)
    return out


def mse_loss(x1, x2, reduction='mean', out=None):
    """0.5 * (x1 - x2)^2, mean or sum (the reference halves the squared error)."""
    _mark_input(x1)
    if is_device(x1.eval):
        raise NotImplementedError('mse_loss on device tensors')
    d = x1.eval - np.asarray(x2.eval).reshape(x1.shape)
    val = 0.5 * (d * d)
    val = val.mean() if reduction == 'mean' else val.sum()
    res = np.asarray(val, dtype=x1.eval.dtype).reshape(1)
    if out is None:
        out = Tensor(res)
    else:
        out.eval = res
    _wire(out, x1, x2)
    if out.is_dynamic:
        out.is_leaf = True
    out.requires_grad = bool(x1.requires_grad or x2.requires_grad)
    if GLOBAL.COMPUTE_GRAD and out.requires_grad:
        out.cache['reduction'] = reduction
        out.grad_fn = MSELossBackward
        initialize_ops_grad(x1, x2)
    return out
