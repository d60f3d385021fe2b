"""Brute-force definitions of the same operations, for tiny shapes only.

TEST INFRASTRUCTURE ONLY -- see ``oracle/__init__.py``.

These are written straight from the index formulas (cross-correlation with a
symmetric zero border; first maximum in row-major window order) with scalar
loops, sharing no code with ``xs_oracle``'s unfold/GEMM/fold route, so that a
transposed operand, a flipped kernel or a wrong fold offset in either one shows
up as a disagreement.
"""
import numpy as np


def _at(x, n, c, i, j):
    """Value of the zero-bordered input at (possibly out-of-range) (i, j)."""
    if 0 <= i < x.shape[2] and 0 <= j < x.shape[3]:
        return float(x[n, c, i, j])
    return 0.0


def conv2d_fwd_brute(x, w, bias, stride, pad):
    n_, c_, h_, w_ = x.shape
    k_, _, r_, s_ = w.shape
    sh, sw = stride
    oh_ = (h_ + 2 * pad - r_) // sh + 1
    ow_ = (w_ + 2 * pad - s_) // sw + 1
    y = np.zeros((n_, k_, oh_, ow_), dtype=np.float64)
    for n in range(n_):
        for k in range(k_):
            for oh in range(oh_):
                for ow in range(ow_):
                    acc = 0.0
                    for c in range(c_):
                        for r in range(r_):
                            for s in range(s_):
                                acc += _at(x, n, c, oh * sh + r - pad, ow * sw + s - pad) * float(w[k, c, r, s])
                    if bias is not None:
                        acc += float(np.asarray(bias).ravel()[k])
                    y[n, k, oh, ow] = acc
    return y


def conv2d_bwd_brute(dy, x, w, stride, pad):
    """Returns float64 (dx, dw, db) for zero-initialised gradients."""
    n_, c_, h_, w_ = x.shape
    k_, _, r_, s_ = w.shape
    sh, sw = stride
    _, _, oh_, ow_ = dy.shape
    dx = np.zeros(x.shape, dtype=np.float64)
    dw = np.zeros(w.shape, dtype=np.float64)
    db = np.zeros((k_,), dtype=np.float64)
    for n in range(n_):
        for k in range(k_):
            for oh in range(oh_):
                for ow in range(ow_):
                    g = float(dy[n, k, oh, ow])
                    db[k] += g
                    for c in range(c_):
                        for r in range(r_):
                            for s in range(s_):
                                i = oh * sh + r - pad
                                j = ow * sw + s - pad
                                if 0 <= i < h_ and 0 <= j < w_:
                                    dw[k, c, r, s] += g * float(x[n, c, i, j])
                                    dx[n, c, i, j] += g * float(w[k, c, r, s])
    return dx, dw, db


def max_pool2d_fwd_brute(x, k, stride, pad):
    """Returns (y float64 NCHW, idx int64 NCHW) with idx = ky*k + kx of the first maximum."""
    n_, c_, h_, w_ = x.shape
    sh, sw = stride
    oh_ = (h_ + 2 * pad - k) // sh + 1
    ow_ = (w_ + 2 * pad - k) // sw + 1
    y = np.zeros((n_, c_, oh_, ow_), dtype=np.float64)
    idx = np.zeros((n_, c_, oh_, ow_), dtype=np.int64)
    for n in range(n_):
        for c in range(c_):
            for oh in range(oh_):
                for ow in range(ow_):
                    best = None
                    where = -1
                    for r in range(k):
                        for s in range(k):
                            v = _at(x, n, c, oh * sh + r - pad, ow * sw + s - pad)
                            if best is None or v > best:     # strict: the first maximum stays
                                best, where = v, r * k + s
                    y[n, c, oh, ow] = best
                    idx[n, c, oh, ow] = where
    return y, idx


def max_pool2d_bwd_brute(dy, idx, x_shape, k, stride, pad):
    """Returns float64 dx for a zero-initialised gradient; idx is NCHW-ordered."""
    n_, c_, h_, w_ = x_shape
    sh, sw = stride
    dx = np.zeros(x_shape, dtype=np.float64)
    for n in range(n_):
        for c in range(c_):
            for oh in range(dy.shape[2]):
                for ow in range(dy.shape[3]):
                    r, s = divmod(int(idx[n, c, oh, ow]), k)
                    i = oh * sh + r - pad
                    j = ow * sw + s - pad
                    if 0 <= i < h_ and 0 <= j < w_:          # gradient on a border cell is dropped
                        dx[n, c, i, j] += float(dy[n, c, oh, ow])
    return dx
