"""Dense and Flatten (counterpart of xs/layers/linear.py)."""
from functools import reduce

from .base import Layer, F, Parameter
from ..nn.initializers import get_initializer


class Dense(Layer):
    """``y = x @ W + b`` with W ``(in, out)`` and b ``(1, out)``."""

    def __init__(self, out_features, activation=None, use_bias=True, kernel_initializer='normal',
                 bias_initializer='zeros', **kwargs):
        self.out_features = out_features
        self.use_bias = use_bias
        self.kernel_initializer = get_initializer(kernel_initializer)
        self.bias_initializer = get_initializer(bias_initializer)
        if activation is not None and str(activation).lower() != 'relu':
            raise ValueError("Dense supports activation='relu' or None")
        self.activation = None if activation is None else 'relu'
        super().__init__(**kwargs)

    def compute_output_shape(self, input_shape=None):
        self._shape = (self.out_features,)
        return self._shape

    def init_params(self, input_shape=None, *args):
        if input_shape is not None:
            self._input_shape = tuple(input_shape)
        self._parameters.append(Parameter(self.kernel_initializer(tuple(self._input_shape) + (self.out_features,),
                                                                  requires_grad=True)))
        if self.use_bias:
            self._parameters.append(Parameter(self.bias_initializer((1, self.out_features), requires_grad=True)))

    def call(self, x, *args, **kwargs):
        if self.use_bias:
            weight, bias = self._parameters
            self._data = F.addmm(bias, x, weight, self._data)
        else:
            self._data = F.mm(x, self._parameters[0], self._data)
        if self.activation == 'relu':
            return F.relu(self._data)
        return self._data


class Flatten(Layer):
    def __init__(self, start_dim=1, **kwargs):
        if start_dim < 1:
            raise ValueError('start_dim must be > 0')
        self.start_dim = start_dim
        super().__init__(**kwargs)

    def compute_output_shape(self, input_shape=None):
        flat = reduce(lambda a, b: a * b, input_shape[self.start_dim - 1:])
        self._shape = tuple(input_shape[:self.start_dim - 1]) + (flat,)
        return self._shape

    def call(self, x, *args, **kwargs):
        self._data = F.flatten(x, self.start_dim, self._data)
        return self._data
