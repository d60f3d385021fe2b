"""Pooling layers (counterpart of xs/layers/pooling.py)."""
from .base import Layer, F


def _size2(v):
    if isinstance(v, (int, float)):
        return int(v), int(v)
    return tuple(int(i) for i in v)


def _square(kernel_size):
    if isinstance(kernel_size, (tuple, list)):
        if len(kernel_size) != 2 or kernel_size[0] != kernel_size[1]:
            raise ValueError('pooling supports square windows only')
        return int(kernel_size[0])
    return int(kernel_size)


class MaxPooling2D(Layer):
    """``MaxPooling2D(kernel_size=2, stride=None, padding=0)`` (reference pooling.py:5-31).  A pair
    ``(k, k)`` is accepted for ``kernel_size``, as the reference's README writes it."""

    def __init__(self, kernel_size=2, stride=None, padding=0, **kwargs):
        self.kernel_size = _square(kernel_size)
        self.stride = _size2(self.kernel_size if stride is None else stride)
        self.padding = padding
        super().__init__(**kwargs)

    def compute_output_shape(self, input_shape=None):
        c, h, w = input_shape
        k, p = self.kernel_size, self.padding
        self._shape = (c, (h - k + 2 * p) // self.stride[0] + 1, (w - k + 2 * p) // self.stride[1] + 1)
        return self._shape

    def call(self, x, *args, **kwargs):
        self._data = F.max_pool2d(x, self.kernel_size, self.stride, self.padding, self._data)
        return self._data


class AvgPooling2D(Layer):
    def __init__(self, kernel_size=2, stride=None, padding=0, **kwargs):
        self.kernel_size = _square(kernel_size)
        self.stride = _size2(self.kernel_size if stride is None else stride)
        self.padding = padding
        super().__init__(**kwargs)

    def compute_output_shape(self, input_shape=None):
        c, h, w = input_shape
        k, p = self.kernel_size, self.padding
        self._shape = (c, (h - k + 2 * p) // self.stride[0] + 1, (w - k + 2 * p) // self.stride[1] + 1)
        return self._shape

    def call(self, x, *args, **kwargs):
        self._data = F.avg_pool2d(x, self.kernel_size, self.stride, self.padding, self._data)
        return self._data
