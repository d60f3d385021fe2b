"""NumPy restatement of the reference's conv / max-pool arithmetic.

TEST INFRASTRUCTURE ONLY -- see ``oracle/__init__.py``.

Every function works on plain ``numpy.ndarray`` values (no Tensor class) and
follows the reference's order of operations, including the facts that

* the unfolded matrix is always float64 (``np.zeros`` default dtype,
  reference ``xs/utils/common.py:37``), so the GEMMs run in float64 and the
  result is rounded once when it is stored into the destination array
  (``xs/core/base.py:73-75``);
* gradients are *accumulated* into existing buffers (``np.add(.., out=)``,
  ``xs/nn/grad_fn.py:194,197,202,235``);
* max-pool pads with the constant 0 and the pad cells take part in the max
  (``xs/nn/functional.py:452-453``), ``np.argmax`` picks the first maximum.

How each function is pinned (none of them has a stored golden vector in the
reference's own tests, which only print distances to PyTorch):

* ``conv2d_fwd``/``conv2d_bwd``: brute-force loops in ``oracle/brute.py``,
  ``torch.nn.functional.conv2d`` + autograd on the reference's own test shapes
  (``tests/gradient_check/xs_pytorch/cnn.py:4-8``), adjoint identities,
  central differences (the technique of ``xs/utils/toolkit.py:160-194``),
  special kernels (1x1 = GEMM, delta = shift, ones = box sum).
* ``max_pool2d_fwd``/``max_pool2d_bwd``: brute-force window scan with an
  explicit strict-greater rule, torch for ``padding=0`` (the case
  ``tests/gradient_check/xs_pytorch/pooling.py:18,43`` uses), invariants.
* ``im2col``/``col2im``: adjointness ``<im2col(x), c> == <x, col2im(c)>`` and
  the explicit index formula.
See ``tests/test_oracle.py``.
"""
import numpy as np


def out_size(size, kernel, stride, pad):
    """Output extent of a window op (reference ``xs/nn/functional.py:415-416``)."""
    return (size - kernel + 2 * pad) // stride + 1


def _zero_pad(x, pad):
    # reference: np.pad(..., 'constant') at xs/nn/functional.py:412 and :453
    if pad == 0:
        return x
    return np.pad(x, ((0, 0), (0, 0), (pad, pad), (pad, pad)), mode="constant")


def im2col(xpad, oh, ow, kh, kw, stride):
    """Unfold a (padded) NCHW array into a float64 ``(N*OH*OW, C*KH*KW)`` matrix.

    Rows are ordered (n, oh, ow), columns (c, ky, kx) -- reference
    ``xs/utils/common.py:35-46``.  The container is float64 whatever the input
    dtype is (``common.py:37``).
    """
    n, c = xpad.shape[:2]
    sh, sw = stride
    slab = np.zeros((n, c, kh, kw, oh, ow))            # float64 on purpose
    for ky in range(kh):
        for kx in range(kw):
            slab[:, :, ky, kx] = xpad[:, :, ky:ky + sh * oh:sh, kx:kx + sw * ow:sw]
    return slab.transpose(0, 4, 5, 1, 2, 3).reshape(n * oh * ow, c * kh * kw)


def col2im(x_shape, pad, kh, kw, stride, dcol):
    """Scatter-add a ``(N*OH*OW, C*KH*KW)`` matrix back onto the (unpadded) input.

    Reference ``xs/utils/common.py:49-65``: float64 canvas of the padded size
    (+ stride-1 slack), taps added in ascending (ky, kx) order, then the pad
    border is cropped away.
    """
    n, c, h, w = x_shape
    sh, sw = stride
    oh = out_size(h, kh, sh, pad)
    ow = out_size(w, kw, sw, pad)
    taps = dcol.reshape(n, oh, ow, c, kh, kw).transpose(0, 3, 4, 5, 1, 2)
    canvas = np.zeros((n, c, h + 2 * pad + sh - 1, w + 2 * pad + sw - 1))
    for ky in range(kh):
        for kx in range(kw):
            canvas[:, :, ky:ky + sh * oh:sh, kx:kx + sw * ow:sw] += taps[:, :, ky, kx]
    return canvas[:, :, pad:pad + h, pad:pad + w]


def conv2d_fwd(x, w, bias=None, stride=(1, 1), padding=0, keep_col=True):
    """Forward of reference ``conv2d`` (``xs/nn/functional.py:405-442``).

    Returns ``(y, col)``: ``y`` has ``x.dtype`` (one rounding of the float64
    GEMM + bias), ``col`` is the float64 unfolded input the backward reuses
    (the reference keeps it in ``out.cache['col']``, line 437).
    """
    n, c, h, wd = x.shape
    k, c2, kh, kw = w.shape
    if c2 != c:
        raise ValueError("channel mismatch: x has %d, weight expects %d" % (c, c2))
    oh = out_size(h, kh, stride[0], padding)
    ow = out_size(wd, kw, stride[1], padding)
    col = im2col(_zero_pad(x, padding), oh, ow, kh, kw, stride)
    flat = np.dot(col, w.reshape(k, -1).T)              # float64 GEMM (line 423)
    if bias is not None:
        flat = flat + np.asarray(bias).reshape(1, k)     # lines 424-425
    y = np.empty((n, k, oh, ow), dtype=x.dtype)
    y[...] = flat.reshape(n, oh, ow, k).transpose(0, 3, 1, 2)   # line 426: cast on store
    return (y, col) if keep_col else (y, None)


def conv2d_bwd(dy, x_shape, w, col, stride, padding, dx=None, dw=None, db=None):
    """Backward of reference ``Conv2DBackward`` (``xs/nn/grad_fn.py:186-203``).

    ``dx``/``dw``/``db`` are existing gradient buffers that are accumulated
    into in place (pass zeros for a fresh gradient); any of them may be
    ``None`` to skip that gradient.  Returns ``(dx, dw, db)``.
    """
    k, c, kh, kw = w.shape
    g = dy.transpose(1, 0, 2, 3).reshape(k, -1)          # line 191
    if dw is not None:
        np.add(dw, np.dot(g, col).reshape(k, c, kh, kw), out=dw)           # 192-194
    if db is not None:
        np.add(db, dy.sum(axis=(0, 2, 3)).reshape(db.shape[-1:]), out=db)  # 196-197
    if dx is not None:
        dcol = np.dot(g.T, w.reshape(k, -1))             # line 199
        np.add(dx, col2im(x_shape, padding, kh, kw, stride, dcol), out=dx)  # 201-203
    return dx, dw, db


def max_pool2d_fwd(x, kernel_size=2, stride=None, padding=0):
    """Forward of reference ``max_pool2d`` (``xs/nn/functional.py:445-491``).

    Only the unfold + argmax branch is live in the reference (the
    ``kernel_size == stride`` test at line 463 compares an int with a tuple).
    Returns ``(y, argmax)`` where ``argmax`` is the reference's flat int64
    vector over rows ordered (n, oh, ow, c), values ``ky*k + kx``.
    """
    if stride is None:
        stride = (kernel_size, kernel_size)
    elif isinstance(stride, int):
        stride = (stride, stride)
    xp = _zero_pad(x, padding)
    n, c, hp, wp = xp.shape
    oh = (hp - kernel_size) // stride[0] + 1
    ow = (wp - kernel_size) // stride[1] + 1
    rows = im2col(xp, oh, ow, kernel_size, kernel_size, stride)
    rows = rows.reshape(-1, kernel_size * kernel_size)   # (n,oh,ow,c) x (ky,kx)
    argmax = np.argmax(rows, axis=1)
    best = np.max(rows, axis=1)
    y = np.empty((n, c, oh, ow), dtype=x.dtype)
    y[...] = best.reshape(n, oh, ow, c).transpose(0, 3, 1, 2)
    return y, argmax


def max_pool2d_bwd(dy, argmax, x_shape, kernel_size, stride, padding, dx):
    """Backward of reference ``Maxpool2DBackward`` (``xs/nn/grad_fn.py:224-235``).

    One-hot scatter of ``dy`` into a zero float64 ``(rows, k*k)`` matrix, fold
    with ``col2im`` (gradient on pad cells is cropped), accumulate into ``dx``.
    """
    if isinstance(stride, int):
        stride = (stride, stride)
    g = dy.transpose(0, 2, 3, 1)
    onehot = np.zeros((g.size, kernel_size * kernel_size))
    onehot[np.arange(argmax.size), argmax.ravel()] = g.ravel()
    np.add(dx, col2im(x_shape, padding, kernel_size, kernel_size, stride, onehot), out=dx)
    return dx


def relu_fwd(x):
    """``np.maximum(0., x)`` -- reference ``xs/nn/td_functional.py:59-60``."""
    return np.maximum(0., x).astype(x.dtype, copy=False)


def relu_bwd(dy, pre):
    """Strict mask of reference ``ReLUBackward`` (``xs/nn/grad_fn.py:155-157``):
    gradient is dropped only where the pre-activation is < 0."""
    g = dy.copy()
    g[pre < 0] = 0
    return g
