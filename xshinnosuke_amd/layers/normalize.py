"""BatchNormalization (counterpart of xs/layers/normalize.py:22-56)."""
from ..core import state as GLOBAL
from .base import Layer, F, Parameter
from ..nn.initializers import get_initializer


class BatchNormalization(Layer):
    def __init__(self, epsilon=1e-6, momentum=0.99, axis=1, gamma_initializer='ones', beta_initializer='zeros',
                 moving_mean_initializer='zeros', moving_variance_initializer='ones', **kwargs):
        self.epsilon, self.momentum, self.axis = epsilon, momentum, axis
        self.gamma_initializer = get_initializer(gamma_initializer)
        self.beta_initializer = get_initializer(beta_initializer)
        self.moving_mean_initializer = get_initializer(moving_mean_initializer)
        self.moving_variance_initializer = get_initializer(moving_variance_initializer)
        self.moving_mean = None
        self.moving_variance = None
        super().__init__(**kwargs)

    def init_params(self, input_shape=None, *args):
        if input_shape is not None:
            self._input_shape = tuple(input_shape)
        n_in = self._input_shape[self.axis - 1]
        self._parameters.append(Parameter(self.gamma_initializer(n_in, requires_grad=True)))
        self._parameters.append(Parameter(self.beta_initializer(n_in, requires_grad=True)))
        self.moving_mean = self.moving_mean_initializer(n_in)
        self.moving_variance = self.moving_variance_initializer(n_in)

    def call(self, x, *args, fuse_relu=False, **kwargs):
        """``fuse_relu`` is set by Sequential when an in-place ReLU layer follows on a device-resident dynamic
        graph: the normalisation kernel then applies it."""
        gamma, beta = self._parameters
        self._data = F.batch_norm(x, gamma, beta, self.moving_mean, self.moving_variance, self.axis, GLOBAL.TRAINING,
                                  self.epsilon, self.momentum, self._data, 'relu' if fuse_relu else None)
        return self._data
