"""Dense and Flatten (counterpart of xs/layers/linear.py)."""
import math

from .base import Layer, F, Parameter
from .activators import FusedActivation
from ..nn.initializers import get_initializer


class Dense(FusedActivation, Layer):
    """``y = act(x @ W + b)``, W ``(in, out)``, b ``(1, out)``; ``activation`` names 'relu', 'sigmoid' or
    'tanh' (a child activation layer on the product's output)."""

    def __init__(self, out_features, activation=None, use_bias=True, kernel_initializer='normal',
                 bias_initializer='zeros', **kwargs):
        self.out_features = out_features
        self.use_bias = use_bias
        self.kernel_initializer = get_initializer(kernel_initializer)
        self.bias_initializer = get_initializer(bias_initializer)
        self._set_activation(activation, fuse_relu=False)
        super().__init__(**kwargs)

    def compute_output_shape(self, input_shape=None):
        self._shape = (self.out_features,)
        return self._shape

    def init_params(self, input_shape=None, *args):
        if input_shape is not None:
            self._input_shape = tuple(input_shape)
        w_shape = tuple(self._input_shape) + (self.out_features,)
        self._parameters.append(Parameter(self.kernel_initializer(w_shape, requires_grad=True)))
        if self.use_bias:
            self._parameters.append(Parameter(self.bias_initializer((1, self.out_features), requires_grad=True)))

    def init_layer_out_tensor(self, x=None):
        super().init_layer_out_tensor(x)
        self._static_act_buffer()

    def call(self, x, *args, **kwargs):
        weight = self._parameters[0]
        if self.use_bias:
            self._data = F.addmm(self._parameters[1], x, weight, self._data)
        else:
            self._data = F.mm(x, weight, self._data)
        return self._activate(self._data)

    def backward(self, gradients=None):
        self._act_backward()
        super().backward(gradients)


class Flatten(Layer):
    def __init__(self, start_dim=1, **kwargs):
        if start_dim < 1:
            raise ValueError('start_dim must be > 0')
        self.start_dim = start_dim
        super().__init__(**kwargs)

    def compute_output_shape(self, input_shape=None):
        keep = self.start_dim - 1
        self._shape = tuple(input_shape[:keep]) + (math.prod(input_shape[keep:]),)
        return self._shape

    def call(self, x, *args, **kwargs):
        self._data = F.flatten(x, self.start_dim, self._data)
        return self._data
