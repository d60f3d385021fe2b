"""Loss layers (counterpart of xs/nn/objectives.py)."""
import copy

import numpy as np

from ..layers.base import Layer
from . import functional as F


class _Loss(Layer):
    def __init__(self, reduction='mean', **kwargs):
        self.reduction = reduction
        super().__init__(**kwargs)

    def init_layer_out_tensor(self, inputs, target):
        pass                                # the scalar loss tensor is created by the functional op

    def forward(self, inputs, target):
        self._data = self.call(inputs, target)
        return self._data

    __call__ = forward

    def calc_acc(self, y_pred, y_true):
        return 0.

    def calc_loss(self, y_pred, y_true):
        raise NotImplementedError

    def metric(self, y_pred, y_true):
        return self.calc_acc(y_pred, y_true), self.calc_loss(y_pred, y_true)


class MSELoss(_Loss):
    def call(self, inputs, target):
        return F.mse_loss(inputs, target, self.reduction)

    def calc_loss(self, y_pred, y_true):
        d = y_pred.numpy() - y_true.numpy().reshape(y_pred.shape)
        v = 0.5 * d * d
        return float(v.mean() if self.reduction == 'mean' else v.sum())


class CrossEntropyLoss(_Loss):
    def __init__(self):
        super().__init__()

    def call(self, inputs, target):
        return F.cross_entropy(inputs, target, self.reduction)

    def calc_loss(self, y_pred, y_true):
        z = y_pred.numpy().astype(np.float64)
        z = z - z.max(axis=-1, keepdims=True)
        logp = z - np.log(np.exp(z).sum(axis=-1, keepdims=True))
        lab = y_true.numpy().astype(np.int64).reshape(-1)
        return float(-logp.reshape(-1, logp.shape[-1])[np.arange(lab.size), lab].mean())

    def calc_acc(self, y_pred, y_true):
        return float(np.mean(np.argmax(y_pred.numpy(), axis=-1).ravel() == y_true.numpy().ravel()))


def get_objective(objective):
    if isinstance(objective, str):
        name = objective.lower()
        if name in ('crossentropy', 'cross_entropy'):
            return CrossEntropyLoss()
        if name in ('meansquarederror', 'mean_squared_error', 'mse'):
            return MSELoss()
        raise ValueError('unknown objective %r' % objective)
    if isinstance(objective, _Loss):
        return copy.deepcopy(objective)
    raise ValueError('unknown objective type!')
