"""Conv2D layer (counterpart of xs/layers/convolutional.py:7-83)."""
from .base import Layer, F, Parameter
from .activators import FusedActivation
from ..nn.initializers import get_initializer


def _size2(v):
    if isinstance(v, (int, float)):
        return int(v), int(v)
    return tuple(int(i) for i in v)


class Conv2D(FusedActivation, Layer):
    """``Conv2D(out_channels, kernel_size, use_bias=True, stride=1, padding=0, activation=None, ...)``.

    weight ``(Cout, Cin, KH, KW)``, bias ``(1, Cout)``; parameters are created lazily from the first
    input.  ``padding`` is an int or 'same' / 'valid'.  With ``activation='relu'`` the activation is
    fused into the convolution kernel's epilogue and differentiated with the strict ``pre < 0`` mask,
    in static graphs as well (the reference applies it in a second pass and, in static graphs,
    loses it for downstream layers, xs/layers/base.py:66-68).  'sigmoid' and 'tanh' run as a child
    activation layer on the convolution's output; an unknown name means no activation, as in the
    reference (xs/layers/activators.py:74-87).
    """

    def __init__(self, out_channels, kernel_size, use_bias=True, stride=1, padding=0, activation=None,
                 kernel_initializer='Normal', bias_initializer='zeros', **kwargs):
        self.out_channels = out_channels
        self.kernel_size = _size2(kernel_size)
        self.use_bias = use_bias
        self.stride = _size2(stride)
        self.padding = padding
        self._set_activation(activation, fuse_relu=True)
        self.kernel_initializer = get_initializer(kernel_initializer)
        self.bias_initializer = get_initializer(bias_initializer)
        self.pad_size = padding if isinstance(padding, int) else 0
        super().__init__(**kwargs)

    def init_params(self, input_shape=None, *args):
        if input_shape is not None:
            self._input_shape = tuple(input_shape)
        if isinstance(self.padding, str):
            self.compute_output_shape(self._input_shape)
        kh, kw = self.kernel_size
        weight = Parameter(self.kernel_initializer((self.out_channels, self._input_shape[0], kh, kw), requires_grad=True))
        self._parameters.append(weight)
        if self.use_bias:
            self._parameters.append(Parameter(self.bias_initializer((1, self.out_channels), requires_grad=True)))
        else:
            self._parameters.append(None)

    def compute_output_shape(self, input_shape=None):
        assert len(input_shape) == 3
        _, h, w = input_shape
        kh, kw = self.kernel_size
        if isinstance(self.padding, str):
            mode = self.padding.upper()
            if mode == 'SAME':
                # the reference's formula (convolutional.py:45-49); exact for stride 1 and odd kernels
                self.pad_size = (self.stride[0] * (h - 1) - h + kh) // 2
            elif mode == 'VALID':
                self.pad_size = 0
            else:
                raise TypeError('Unknown padding type!plz inputs SAME or VALID or an integer')
        else:
            assert isinstance(self.padding, int)
            self.pad_size = self.padding
        oh = (h - kh + 2 * self.pad_size) // self.stride[0] + 1
        ow = (w - kw + 2 * self.pad_size) // self.stride[1] + 1
        self._shape = (self.out_channels, oh, ow)
        return self._shape

    def call(self, x, *args, **kwargs):
        weight, bias = self._parameters[0], (self._parameters[1] if self.use_bias else None)
        self._data = F.conv2d(x, weight, bias, self.stride, self.pad_size, self._data, activation=self.activation)
        return self._activate(self._data)

    def init_layer_out_tensor(self, x=None):
        super().init_layer_out_tensor(x)
        self._static_act_buffer()

    def backward(self, gradients=None):
        self._act_backward()
        super().backward(gradients)
