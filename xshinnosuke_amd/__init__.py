"""xshinnosuke_amd -- an MI355X (gfx950) backend for xshinnosuke's conv / max-pool path, behind the same API.

    import xshinnosuke_amd as xs
    x = xs.randn(8, 3, 32, 32, requires_grad=True).to('cuda')
    y = xs.nn.functional.conv2d(x, w, b, stride=(1, 1), padding=1)

The conv2d / max_pool2d forward and backward always run the hand-written HIP kernels in
libxsmi355.so (``xshinnosuke_amd/csrc``); the rest of the package is the thin caller-side mirror of the
reference's Tensor / layer / model interface that those ops plug into.
"""
import numpy as _np

from . import backend  # noqa: F401
from .backend.graph import StepGraph
from .core import state as GLOBAL
from .core.state import no_grad, conv_precision
from .core.base import Tensor, Parameter
from . import nn, layers, optim, utils
from .utils import gradient_check

float16, float32, float64 = _np.dtype(_np.float16), _np.dtype(_np.float32), _np.dtype(_np.float64)
int8, uint8, int16, int32, int64 = (_np.dtype(t) for t in (_np.int8, _np.uint8, _np.int16, _np.int32, _np.int64))


def tensor(data, requires_grad=False, dtype=None, name=None):
    return Tensor(_np.array(data, dtype=dtype), requires_grad=requires_grad, name=name)


def manual_seed_all(seed):
    _np.random.seed(seed)


def _shape(size):
    return tuple(size[0]) if len(size) == 1 and isinstance(size[0], (tuple, list)) else tuple(size)


def randn(*size, requires_grad=False, dtype=None):
    return Tensor(_np.random.randn(*_shape(size)).astype(dtype or _np.float64), requires_grad=requires_grad)


def rand(*size, requires_grad=False, dtype=None):
    return Tensor(_np.random.rand(*_shape(size)).astype(dtype or _np.float64), requires_grad=requires_grad)


def randint(low, high=None, size=None, requires_grad=False):
    return Tensor(_np.random.randint(low, high, size), requires_grad=requires_grad)


def zeros(*size, requires_grad=False, dtype=None):
    return Tensor(_np.zeros(_shape(size), dtype=dtype or _np.float64), requires_grad=requires_grad)


def ones(*size, requires_grad=False, dtype=None):
    return Tensor(_np.ones(_shape(size), dtype=dtype or _np.float64), requires_grad=requires_grad)


def cuda_available():
    """True when libxsmi355.so loads and finds a gfx950 device."""
    try:
        backend.init(0)
        return True
    except Exception:
        return False
