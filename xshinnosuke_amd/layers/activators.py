"""ReLU layer (counterpart of xs/layers/activators.py:18-59)."""
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


class Activation(ReLU):
    def __init__(self, act_name='relu', **kwargs):
        if str(act_name).lower() != 'relu':
            raise ValueError('only relu is available')
        super().__init__(False, **kwargs)


def get_activator(name):
    if name is None:
        return None
    if str(name).lower() == 'relu':
        return ReLU()
    raise ValueError('unknown activation %r' % (name,))
