"""Layer base class (counterpart of xs/layers/base.py:6-134).

A layer is called either with a Tensor (eager: create parameters lazily from the
input shape, run ``call``) or with another Layer (graph building: infer the
output shape and link).  In a static graph every layer owns one preallocated
output Tensor sized for the largest batch, re-sliced for a shorter last batch and
written in place through the ``out=`` argument of the functional op.
"""
from ..core import state as GLOBAL
from ..core.base import Tensor, Parameter
from ..nn.initializers import Zeros
from ..nn import functional as F


class Layer:
    def __init__(self, trainable=True, name=None, in_bounds=None, input_shape=None, shape=None, parameters=None,
                 **kwargs):
        self.trainable = trainable
        self._in_bounds = list(in_bounds) if in_bounds is not None else []
        self._out_bounds = []
        self._input_shape = input_shape
        self.name = str(name)
        self._shape = shape
        self._parameters = parameters if parameters is not None else []
        self._data = None

    def __call__(self, x, *args, **kwargs):
        if isinstance(x, Tensor):
            if len(self._parameters) == 0:
                self.init_params(tuple(x.shape[1:]))
            x.next_layers.append(self)
            return self.call(x, *args, **kwargs)
        self._shape = self.compute_output_shape(x.shape)
        self._in_bounds.append(x)
        self._input_shape = x.shape
        x.add_out_bounds(self)
        return self

    def connect(self, inbound=None):
        if inbound is None:
            if self._input_shape is None:
                raise ValueError('must specify input_shape')
        else:
            self._input_shape = inbound.shape
        self._shape = self.compute_output_shape(self._input_shape)
        if inbound is not None:
            self._in_bounds.append(inbound)
            inbound.add_out_bounds(self)

    def params_count(self):
        return sum(v.eval.size for v in self._parameters if v is not None)

    @property
    def shape(self):
        return self._shape

    @property
    def out_bounds(self):
        return self._out_bounds

    @property
    def in_bounds(self):
        return self._in_bounds

    @property
    def data(self):
        return self._data

    @data.setter
    def data(self, v):
        self._data = v

    def parameters(self, parameters=None):
        if parameters is None:
            return self._parameters
        self._parameters = parameters

    def add_out_bounds(self, *outs):
        for out in outs:
            if isinstance(out, Layer):
                self._out_bounds.append(out)

    def init_params(self, input_shape=None, *args):
        pass

    def _new_out_tensor(self, x):
        t = Zeros()((x.shape[0],) + tuple(self.shape), requires_grad=self.trainable)
        if x.device == 'cuda' and t.device != 'cuda':
            t.cuda_()
        elif x.device == 'cpu' and t.device != 'cpu':
            t.cpu_()
        t.to('static')
        return t

    def init_layer_out_tensor(self, x=None):
        x = self._in_bounds[0].data if x is None else x
        if self._data is None or x.shape[0] > self._data.shape_capacity[0] or \
                (x.shape[0] < self._data.shape_capacity[0] and not GLOBAL.TRAINING):
            self._data = self._new_out_tensor(x)
            self._data.add_in_bounds(x)
            self._data.add_in_bounds(*self.parameters())
        else:
            if x.shape[0] < self._data.shape_capacity[0]:
                self._data.slices(slice(None, x.shape[0], None))
            else:
                self._data.slices(slice(None, None, None))
            # a reused output tensor must read from the tensor that feeds it now: the reference keeps the
            # tensor it was created with (xs/layers/base.py:88-104), which goes stale as soon as a new
            # loader hands in different batch tensors (fit after predict, a second fit)
            if self._data.in_bounds and self._data.in_bounds[0] is not x:
                self._data.in_bounds[0] = x

    def compute_output_shape(self, input_shape=None):
        self._shape = (input_shape,) if isinstance(input_shape, int) else tuple(input_shape)
        return self._shape

    def call(self, x, *args, **kwargs):
        raise NotImplementedError

    def forward(self, x=None, *args, **kwargs):
        if x is None:
            x = self._in_bounds[-1]
        if len(self._parameters) == 0:
            self.init_params(tuple(x.shape[1:]) if isinstance(x, Tensor) else None)
        if isinstance(x, Tensor):
            if x.is_dynamic:
                x.next_layers.append(self)
            return self.call(x, *args, **kwargs)
        return self.call(x.data, *args, **kwargs)

    def backward(self, gradients=None):
        if gradients is not None:
            assert isinstance(gradients, Tensor) and gradients.shape == self._data.shape
            self._data.grad = gradients
        if self._data.grad_fn is not None:
            self._data.grad_fn(self._data)
            self._data.zero_grad()
