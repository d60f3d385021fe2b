"""Layer, the node type of both graph styles (the role of the reference's xs/layers/base.py:6-134).

Applied to a Tensor a layer works eagerly: parameters are created from the input's shape on first use and
``call`` runs the functional op.  Applied to another Layer it only records the edge and its output shape; the
model later drives ``forward`` / ``backward`` over those edges, with one preallocated output tensor per layer
(``static_buffer``).
"""
from ..core.base import Tensor, Parameter            # noqa: F401  (re-exported to the layer modules)
from ..nn import functional as F                     # noqa: F401
from . import static_buffer


class Layer:
    def __init__(self, trainable=True, name=None, in_bounds=None, input_shape=None, shape=None, parameters=None,
                 **kwargs):
        self.name = str(name)
        self.trainable = trainable
        self._shape, self._input_shape = shape, input_shape
        self._parameters = [] if parameters is None else parameters
        self._in_bounds = [] if in_bounds is None else list(in_bounds)
        self._out_bounds = []
        self._data = None

    # ------------------------------------------------------------------ applying a layer
    def __call__(self, x, *args, **kwargs):
        if not isinstance(x, Tensor):
            return self._chain_after(x)
        return self._run(x, args, kwargs, dynamic=True)

    def forward(self, x=None, *args, **kwargs):
        """Static graphs call this without an argument: the input is then the output of the layer's last inbound
        layer.  A Tensor argument is the dynamic form, as in ``__call__``."""
        src = self._in_bounds[-1] if x is None else x
        if isinstance(src, Tensor):
            return self._run(src, args, kwargs, dynamic=src.is_dynamic)
        if not self._parameters:
            self.init_params(None)
        return self.call(src.data, *args, **kwargs)

    def _run(self, x, args, kwargs, dynamic):
        if not self._parameters:
            self.init_params(tuple(x.shape[1:]))
        if dynamic:
            self._forget_stale_output(x)
            x.next_layers.append(self)           # autograd clears this layer's output after the backward sweep
        return self.call(x, *args, **kwargs)

    def _forget_stale_output(self, x):
        """A dynamic forward hands the previous output tensor to the op as ``out=`` so that it is written again.
        After a forward without backward (inference) that tensor is still there; when the batch size has
        changed since, it cannot be reused and a new one is made (the reference raises a shape error here)."""
        d = self._data
        if isinstance(d, Tensor) and d.is_dynamic and d.eval is not None and len(d.shape) and d.shape[0] != x.shape[0]:
            self._data = None

    def _chain_after(self, inbound):
        """Graph building, ``layer(previous_layer)``: record the edge, infer the output shape, return self."""
        self._input_shape = inbound.shape
        self._shape = self.compute_output_shape(inbound.shape)
        self._in_bounds.append(inbound)
        inbound.add_out_bounds(self)
        return self

    def connect(self, inbound=None):
        """``Sequential.compile`` links consecutive layers with this; the first layer needs ``input_shape``."""
        if inbound is not None:
            self._input_shape = inbound.shape
        elif self._input_shape is None:
            raise ValueError('must specify input_shape')
        self._shape = self.compute_output_shape(self._input_shape)
        if inbound is not None:
            self._in_bounds.append(inbound)
            inbound.add_out_bounds(self)

    def call(self, x, *args, **kwargs):
        raise NotImplementedError

    def backward(self, gradients=None):
        """Static-graph backward of this layer: run the output tensor's grad_fn (which adds into the inputs'
        gradients), then clear the output's own gradient for the next step."""
        out = self._data
        if gradients is not None:
            if not isinstance(gradients, Tensor) or gradients.shape != out.shape:
                raise ValueError('gradients must be a Tensor of the output shape %s' % (out.shape,))
            out.grad = gradients
        if out.grad_fn is not None:
            out.grad_fn(out)
            out.zero_grad()

    # ------------------------------------------------------------------ shapes, parameters, buffers
    def init_params(self, input_shape=None, *args):
        pass

    def compute_output_shape(self, input_shape=None):
        self._shape = (input_shape,) if isinstance(input_shape, int) else tuple(input_shape)
        return self._shape

    def init_layer_out_tensor(self, x=None):
        if x is None:
            x = self._in_bounds[0].data
        self._data = static_buffer.fit_to_batch(self, self._data, x)

    def parameters(self, parameters=None):
        if parameters is None:
            return self._parameters
        self._parameters = parameters

    def params_count(self):
        return sum(p.eval.size for p in self._parameters if p is not None)

    def add_out_bounds(self, *outs):
        self._out_bounds.extend(o for o in outs if isinstance(o, Layer))

    shape = property(lambda self: self._shape)
    in_bounds = property(lambda self: self._in_bounds)
    out_bounds = property(lambda self: self._out_bounds)

    @property
    def data(self):
        return self._data

    @data.setter
    def data(self, v):
        self._data = v
