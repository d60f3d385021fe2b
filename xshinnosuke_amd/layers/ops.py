"""Input and Add (counterpart of xs/layers/ops.py)."""
from .base import Layer, F
from ..nn.grad_fn import initialize_ops_grad
from ..nn import array_ops as A


class Input(Layer):
    def __init__(self, input_shape, **kwargs):
        super().__init__(input_shape=tuple(input_shape), **kwargs)
        self._shape = tuple(input_shape)

    def init_layer_out_tensor(self, x=None):
        if x is not None:
            self._data = x

    def call(self, x, *args, **kwargs):
        self._data = x
        return self._data

    def backward(self, gradients=None):
        pass


class Add(Layer):
    """Sum of several layers' outputs in a static graph."""

    def __call__(self, inbounds, *args, **kwargs):
        for inbound in inbounds:
            self._in_bounds.append(inbound)
            inbound.add_out_bounds(self)
            self._shape = inbound.shape
        return self

    def compute_output_shape(self, input_shape=None):
        return self._shape

    def forward(self, x=None, *args, **kwargs):
        self._data.zero_()
        for inbound in self._in_bounds:
            src = inbound.data
            A.iadd(self._data.eval, src.eval)
            if src.requires_grad:
                initialize_ops_grad(src)
            self._data.requires_grad = bool(self._data.requires_grad or src.requires_grad)
        return self._data

    def backward(self, gradients=None):
        for inbound in self._in_bounds:
            if inbound.data.requires_grad:
                A.iadd(inbound.data.grad.eval, self._data.grad.eval)
        self._data.zero_grad()
