"""Parameter initialisers (counterpart of xs/nn/initializers.py).  Values are drawn with NumPy's
global RNG in float64, as in the reference; when the device is the default placement
(``state.USE_CUDA``) the resulting tensor is uploaded as float32."""
import numpy as np

from ..core import state as GLOBAL
from ..core.base import Tensor


def _finish(arr, **kwargs):
    t = Tensor(arr, **kwargs)
    if GLOBAL.USE_CUDA:
        t.cuda_()
    return t


def fans(shape):
    """(fan_in, fan_out): for a KCRS filter fan_in = C*R*S (reference initializers.py:11-21)."""
    shape = tuple(int(s) for s in np.atleast_1d(shape))
    if len(shape) == 2:
        return shape[0], shape[1]
    if len(shape) in (4, 5):
        rf = int(np.prod(shape[2:]))
        return shape[1] * rf, shape[0] * rf
    n = int(np.sqrt(np.prod(shape)))
    return n, n


class Initializer:
    def __init__(self, seed=None):
        if seed is not None:
            np.random.seed(seed)

    def __call__(self, shape, **kwargs):
        raise NotImplementedError


class Zeros(Initializer):
    def __call__(self, shape, **kwargs):
        return _finish(np.zeros(shape), **kwargs)


class Ones(Initializer):
    def __call__(self, shape, **kwargs):
        return _finish(np.ones(shape), **kwargs)


class Empty(Initializer):
    def __call__(self, shape, **kwargs):
        return _finish(np.empty(shape), **kwargs)


class Uniform(Initializer):
    def __init__(self, scale=0.05, seed=None):
        self.scale = scale
        super().__init__(seed)

    def __call__(self, shape, **kwargs):
        return _finish(np.random.uniform(-self.scale, self.scale, size=shape), **kwargs)


class Normal(Initializer):
    def __init__(self, std=0.1, mean=0.0, seed=None):
        self.std, self.mean = std, mean
        super().__init__(seed)

    def __call__(self, shape, **kwargs):
        return _finish(np.random.normal(loc=self.mean, scale=self.std, size=shape), **kwargs)


class _Scaled(Initializer):
    kind, rule = 'normal', staticmethod(lambda fi, fo: 1.0)

    def __call__(self, shape, **kwargs):
        fi, fo = fans(shape)
        s = float(np.sqrt(self.rule(fi, fo)))
        return (Normal(s) if self.kind == 'normal' else Uniform(s))(shape, **kwargs)


class HeNormal(_Scaled):
    rule = staticmethod(lambda fi, fo: 2.0 / fi)


class HeUniform(_Scaled):
    kind, rule = 'uniform', staticmethod(lambda fi, fo: 6.0 / fi)


class GlorotNormal(_Scaled):
    rule = staticmethod(lambda fi, fo: 2.0 / (fi + fo))


class GlorotUniform(_Scaled):
    kind, rule = 'uniform', staticmethod(lambda fi, fo: 6.0 / (fi + fo))


class LecunNormal(_Scaled):
    rule = staticmethod(lambda fi, fo: 1.0 / fi)


class LecunUniform(_Scaled):
    kind, rule = 'uniform', staticmethod(lambda fi, fo: 3.0 / fi)


_BY_NAME = {
    'zeros': Zeros, 'ones': Ones, 'normal': Normal, 'uniform': Uniform,
    'henormal': HeNormal, 'he_normal': HeNormal, 'heuniform': HeUniform, 'he_uniform': HeUniform,
    'glorotnormal': GlorotNormal, 'glorot_normal': GlorotNormal, 'xaviernormal': GlorotNormal,
    'glorotuniform': GlorotUniform, 'glorot_uniform': GlorotUniform, 'xavieruniform': GlorotUniform,
    'lecunnormal': LecunNormal, 'lecun_normal': LecunNormal, 'lecununiform': LecunUniform, 'lecun_uniform': LecunUniform,
}


def get_initializer(initializer):
    if isinstance(initializer, str):
        try:
            return _BY_NAME[initializer.lower()]()
        except KeyError:
            raise ValueError('unknown initializer %r' % initializer)
    if isinstance(initializer, Initializer):
        return initializer
    raise TypeError('unknown initializer type %r' % type(initializer))
