"""Preallocated output tensors of static graphs.

``fit`` / ``evaluate`` / ``predict`` give every layer one output Tensor sized for the largest batch seen so far.
A shorter batch re-slices it, the functional op writes into it through ``out=``, and the layer-wise backward
reads the gradient that the next layer left on it (reference behaviour: xs/layers/base.py:88-104).  On the
device this is what keeps a training step free of allocations.
"""
from ..core import state as GLOBAL
from ..nn.initializers import Zeros


def allocate(layer, x):
    """A zero-filled static tensor of ``x``'s batch size and the layer's output shape, placed where ``x`` lives
    and wired to its producers (the input tensor first, then the layer's parameters)."""
    t = Zeros()((x.shape[0],) + tuple(layer.shape), requires_grad=layer.trainable)
    if t.device != x.device:
        t.cuda_() if x.device == 'cuda' else t.cpu_()
    t.to('static')
    t.add_in_bounds(x)
    t.add_in_bounds(*layer.parameters())
    return t


def fit_to_batch(layer, buf, x):
    """The buffer to use for input ``x``: ``buf`` re-sliced when it is large enough, else a new one.  Outside
    training a smaller batch gets a buffer of its own size (predictions are returned to the caller, who may
    keep them)."""
    rows, capacity = x.shape[0], (buf.shape_capacity[0] if buf is not None else -1)
    if rows > capacity or (rows < capacity and not GLOBAL.TRAINING):
        return allocate(layer, x)
    buf.slices(slice(None, rows if rows < capacity else None, None))
    # The reference leaves a reused buffer wired to the tensor it was created with, which goes stale as soon as
    # another loader hands in different batch tensors (fit after predict, a second fit): follow the live input.
    if buf.in_bounds and buf.in_bounds[0] is not x:
        buf.in_bounds[0] = x
    return buf
