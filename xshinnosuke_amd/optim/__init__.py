"""Optimizers (counterpart of xs/optim).  Only SGD demonstrably works in the reference (the others use an
undefined ``np``, e.g. xs/optim/sgd.py:21), so only SGD is provided."""
from ..nn import array_ops as A


class Optimizer:
    def __init__(self, parameters=None, lr=0.01, weight_decay=0.):
        self._parameters = parameters
        self.lr = lr
        self.weight_decay = weight_decay
        self.iterations = 0

    def zero_grad(self):
        for v in self._parameters:
            v.zero_grad()

    def step(self):
        self.iterations += 1


class SGD(Optimizer):
    def step(self):
        """v -= lr * v.grad for every trainable parameter (reference xs/optim/sgd.py:4-9)."""
        A.sgd_step_all([(v.eval, v.grad.eval) for v in self._parameters if v.requires_grad and v.grad is not None],
                       self.lr)
        super().step()


def get_optimizer(optimizer, **kwargs):
    if isinstance(optimizer, str):
        if optimizer.lower() in ('sgd',):
            return SGD(**kwargs)
        raise ValueError('unknown optimizer %r (only sgd is available)' % optimizer)
    if isinstance(optimizer, Optimizer):
        if kwargs.get('parameters') is not None:
            optimizer._parameters = kwargs['parameters']
        return optimizer
    raise ValueError('unknown optimizer type!')
