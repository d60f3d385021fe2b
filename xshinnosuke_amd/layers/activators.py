"""Activation layers (counterpart of xs/layers/activators.py:4-87): ReLU (optionally in place), Sigmoid, Tanh,
the name-driven ``Activation`` wrapper and ``get_activator``."""
import copy

from .base import Layer, F


class ReLU(Layer):
    def __init__(self, inplace=False, **kwargs):
        super().__init__(**kwargs)
        self.inplace = inplace

    def init_layer_out_tensor(self, x=None):
        if self.inplace:
            self._data = x if x is not None else self._in_bounds[0].data
        else:
            super().init_layer_out_tensor(x)

    def call(self, x, *args, **kwargs):
        if self.inplace:
            self._data = F.relu(x, True)
        else:
            self._data = F.relu(x, False, self._data)
        return self._data

    def backward(self, gradients=None):
        if gradients is not None:
            self._data.grad = gradients
        if self._data.grad_fn is not None:
            self._data.grad_fn(self._data)
            if not self.inplace:
                self._data.zero_grad()


class Sigmoid(Layer):
    def call(self, x, *args, **kwargs):
        self._data = F.sigmoid(x, self._data)
        return self._data


class Tanh(Layer):
    def call(self, x, *args, **kwargs):
        self._data = F.tanh(x, self._data)
        return self._data


class Activation(Layer):
    """``Activation('relu' | 'sigmoid' | 'tanh')``: a layer that forwards to the named activation layer and
    shares its output tensor with it."""

    def __init__(self, act_name='relu', **kwargs):
        self.activation = get_activator(act_name)
        if self.activation is None:
            raise ValueError('unknown activation %r' % (act_name,))
        super().__init__(**kwargs)

    def init_layer_out_tensor(self, x=None):
        super().init_layer_out_tensor(x)
        self.activation.data = self._data

    def call(self, x, *args, **kwargs):
        self._data = self.activation.call(x)
        return self._data


_BY_NAME = {'relu': ReLU, 'sigmoid': Sigmoid, 'tanh': Tanh}


def get_activator(activator):
    """A fresh activation layer for a name; None for None and, as in the reference (activators.py:74-87), for a
    name it does not know; a copy of an ``Activation`` instance."""
    if activator is None:
        return None
    if isinstance(activator, str):
        cls = _BY_NAME.get(activator.lower())
        return cls() if cls is not None else None
    if isinstance(activator, Activation):
        return copy.deepcopy(activator)
    raise TypeError('unknown activator type!')


class FusedActivation:
    """What ``Conv2D`` / ``Dense`` do with their ``activation=`` argument.  'relu' after a convolution is fused
    into the kernel's epilogue by the layer itself; every other case owns a child activation layer that runs on
    the layer's output, provides the tensor the next layer reads and is differentiated first in the layer-wise
    backward (the reference's Conv2D omits the second point in static graphs, xs/layers/base.py:66-68)."""

    def _set_activation(self, name, fuse_relu):
        self.activation = None                   # name of a fused activation ('relu'), for the functional op
        self._act_layer = None                   # child layer for everything else
        if name is None:
            return
        if fuse_relu and isinstance(name, str) and name.lower() == 'relu':
            self.activation = 'relu'
            return
        self._act_layer = get_activator(name)

    def _activate(self, out):
        return out if self._act_layer is None else self._act_layer.forward(out)

    def _static_act_buffer(self):
        if self._act_layer is not None:
            self._act_layer.compute_output_shape(self._shape)
            self._act_layer.init_layer_out_tensor(self._data)

    def _act_backward(self):
        if self._act_layer is not None:
            self._act_layer.backward()

    @property
    def data(self):
        return self._data if self._act_layer is None else self._act_layer.data

    @data.setter
    def data(self, v):
        if self._act_layer is None:
            self._data = v
        else:
            self._act_layer.data = v
            if v is None:
                self._data = None
