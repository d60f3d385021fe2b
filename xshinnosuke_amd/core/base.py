"""Tensor / Parameter: the calling convention of the conv / pool path.

Counterpart of the reference's xs/core/base.py:6-371 restricted to what the
functional ops, layers and models of this package use.  A Tensor's storage is
either a ``numpy.ndarray`` (host) or a :class:`DeviceArray` (MI355X HBM); the
``eval`` property hands out the active leading-axis slice of it, which is how a
static graph re-uses one preallocated buffer for a shorter last batch
(xs/layers/base.py:88-104).
"""
import weakref

import numpy as np

from . import state as GLOBAL
from ..backend import DeviceArray, to_device
from ..backend import array as _dev

_FULL = slice(None, None, None)


def is_device(a):
    return isinstance(a, DeviceArray)


class Tensor(object):
    def __new__(cls, *args, **kwargs):
        if len(args) and isinstance(args[0], Tensor):
            return args[0]                       # Tensor(t) is t, as in the reference (base.py:7-10)
        return super().__new__(cls)

    def __init__(self, data=None, requires_grad=False, dtype=None, name=None, **kwargs):
        if isinstance(data, Tensor):
            return
        self._data = None
        self.reset_(data, requires_grad, name, dtype, **kwargs)

    def reset_(self, data=None, requires_grad=False, name=None, dtype=None, **kwargs):
        if data is not None:
            if is_device(data):
                self._data = data
            else:
                self._data = np.asarray(data, dtype=dtype)
        self._grad = kwargs.pop('grad', None)
        self._in_bounds = []
        self._out_bounds = []
        self.name = name
        self.grad_fn = None
        self.requires_grad = requires_grad
        self._slices = kwargs.pop('slices', _FULL)
        self._static = kwargs.pop('static_graph_tensor', False)
        self._cache = {}
        self._retain = kwargs.pop('retain_grad', False)
        self._is_leaf = None
        self.next_layers = []

    def free_memory(self):
        self._data = None
        self._grad = None

    # ---- storage -------------------------------------------------------------
    @property
    def eval(self):
        d = self._data
        if d is None:
            return None
        if d.size == 1 or self._slices == _FULL:
            return d
        return d[self._slices]

    @eval.setter
    def eval(self, v):
        if isinstance(v, Tensor):
            v = v.eval
        if self._data is None:
            self._data = v if is_device(v) else np.asarray(v)
            return
        dst = self.eval
        if is_device(dst):
            if is_device(v):
                dst.copy_from(v)
            else:
                dst.set(np.asarray(v))
        else:
            if is_device(v):
                v = v.numpy()
            self._data[self._slices] = np.asarray(v)          # casts to the buffer's dtype on store

    @property
    def data(self):
        if self._data is None:
            return None
        return Tensor(self._data, slices=self._slices, static_graph_tensor=self._static, grad=self._grad)

    @data.setter
    def data(self, v):
        if not isinstance(v, Tensor):
            raise TypeError('Unknown data type {}'.format(type(v)))
        self.eval = v.eval

    @property
    def shape_capacity(self):
        return self._data.shape

    @property
    def shape(self):
        s = self.eval.shape
        return s if len(s) != 0 else (1,)

    @property
    def dtype(self):
        return str(self._data.dtype)

    @property
    def device(self):
        return "cuda" if is_device(self._data) else "cpu"

    def slices(self, slices=None):
        if slices is None:
            return self._slices
        assert isinstance(slices, slice)
        self._slices = slices

    # ---- graph ---------------------------------------------------------------
    @property
    def is_leaf(self):
        return self._is_leaf if self._is_leaf is not None else len(self._in_bounds) == 0

    @is_leaf.setter
    def is_leaf(self, flag):
        self._is_leaf = flag

    @property
    def grad(self):
        if self._grad is not None:
            self._grad.slices(self._slices)
        return self._grad

    @grad.setter
    def grad(self, g):
        self._grad = g if isinstance(g, Tensor) or g is None else Tensor(g)

    @property
    def cache(self):
        return self._cache

    @property
    def is_static(self):
        return self._static

    @property
    def is_dynamic(self):
        return not self._static

    def retain_grad(self, retain=None):
        if retain is None:
            return self._retain
        self._retain = retain

    @property
    def in_bounds(self):
        return self._in_bounds

    @property
    def out_bounds(self):
        """The tensors computed from this one that are still alive.  The links are weak: a tensor that outlives a
        training loop (a loader's batch tensor, a static layer output feeding the loss) must not keep every
        result ever derived from it, and that result's device memory, alive."""
        live = [t for t in (r() for r in self._out_bounds) if t is not None]
        if len(live) != len(self._out_bounds):
            self._out_bounds = [weakref.ref(t) for t in live]
        return live

    def __getstate__(self):
        state = dict(self.__dict__)
        state['_out_bounds'] = []                # weak links are rebuilt by the next forward
        return state

    def add_in_bounds(self, *ins):
        for i in ins:
            if isinstance(i, Tensor) or i is None:
                self._in_bounds.append(i)
            else:
                raise TypeError('Not a Tensor')

    def add_out_bounds(self, *outs):
        for o in outs:
            if not isinstance(o, Tensor):
                raise TypeError('Not a Tensor')
            refs = self._out_bounds
            if refs and refs[-1]() is o:         # a reused output tensor, wired again by the next forward
                continue
            if len(refs) >= 32:
                refs[:] = [r for r in refs if r() is not None]
            refs.append(weakref.ref(o))

    def requires_grad_(self, flag):
        self.requires_grad = flag

    # ---- placement -----------------------------------------------------------
    def to(self, dst='static'):
        if dst == 'static':
            self._static = True
            return self
        if dst == 'dynamic':
            self._static = False
            return self
        if dst == 'cuda':
            GLOBAL.USE_CUDA = True
            ret = Tensor(self._device_copy(self._data), requires_grad=self.requires_grad, name=self.name)
            if self._grad is not None:
                ret.grad = Tensor(self._device_copy(self._grad._data))
            return ret
        if dst == 'cpu':
            ret = Tensor(self._host_copy(self._data), requires_grad=self.requires_grad, name=self.name)
            if self._grad is not None:
                ret.grad = Tensor(self._host_copy(self._grad._data))
            return ret
        raise ValueError('unknown destination %r' % (dst,))

    @staticmethod
    def _device_copy(a):
        if is_device(a):
            return a
        a = np.asarray(a)
        return to_device(a, np.float32 if a.dtype.kind == 'f' else a.dtype)

    @staticmethod
    def _host_copy(a):
        return a.numpy() if is_device(a) else a

    def cuda(self):
        return self.to('cuda')

    def cpu(self):
        return self.to('cpu')

    def cuda_(self):
        GLOBAL.USE_CUDA = True
        self._data = self._device_copy(self._data)
        if self._grad is not None:
            self._grad._data = self._device_copy(self._grad._data)

    def cpu_(self):
        self._data = self._host_copy(self._data)
        if self._grad is not None:
            self._grad._data = self._host_copy(self._grad._data)

    def numpy(self):
        e = self.eval
        return e.numpy() if is_device(e) else np.asarray(e)

    # ---- misc ----------------------------------------------------------------
    def __getitem__(self, item):
        ret = Tensor(self.eval[item], requires_grad=self.requires_grad)
        ret.add_out_bounds(self)
        return ret

    def __setitem__(self, key, value):
        if is_device(self._data):
            raise TypeError('item assignment is not supported on device tensors')
        self.eval[key] = np.asarray(value, dtype=self._data.dtype)

    def __repr__(self):
        rg = ", requires_grad=True" if self.requires_grad else ""
        fn = ", grad_fn=<%s>" % self.grad_fn.__name__ if self.grad_fn else ""
        body = self._data if not is_device(self._data) else repr(self._data)
        return "%s(%s%s%s)" % (self.__class__.__name__, body, rg, fn)

    __str__ = __repr__

    def _F(self):
        from ..nn import functional
        return functional

    def __add__(self, other):
        return self._F().add(self, Tensor(other))

    __radd__ = __add__

    def __sub__(self, other):
        return self._F().sub(self, Tensor(other))

    def __mul__(self, other):
        return self._F().mul(self, Tensor(other))

    __rmul__ = __mul__

    def __pow__(self, power, modulo=None):
        return self._F().pow(self, power)

    def __matmul__(self, other):
        return self._F().mm(self, Tensor(other))

    def mm(self, other):
        return self.__matmul__(other)

    dot = mm

    def numel(self):
        return self._data.size

    def item(self):
        assert self._data.size == 1
        return float(self.numpy().reshape(-1)[0])

    def zero_(self):
        if is_device(self._data):
            self._data.fill_zero(lazy=True)
        else:
            self._data = np.zeros_like(self._data)

    def fill_(self, value):
        if is_device(self._data):
            d = self._data
            if d.dtype == np.float32 and d.size:       # a fill kernel: nothing for the host to wait for
                d.take_fresh()
                d._overwritten()
                _dev.lib.call("xsmi_fill", d.cptr, float(value), d.size)
            else:
                d.set(np.full(d.shape, value, dtype=d.dtype))
        else:
            self._data.fill(value)

    def zero_grad(self):
        """Allocate a zero gradient of this tensor's (active) shape, or clear the existing one
        (reference xs/core/base.py:312-316)."""
        if self._grad is None:
            if is_device(self._data):
                self._grad = Tensor(_dev.zeros(self.shape, self._data.dtype, lazy=True))
            else:
                self._grad = Tensor(np.zeros(self.shape, dtype=self._data.dtype))
        else:
            self._grad.zero_()

    def sum(self, axis=None, keepdims=False):
        return self._F().sum(self, axis, keepdims)

    def mean(self, axis=None, keepdims=False):
        return self._F().mean(self, axis, keepdims)

    def view(self, *shapes):
        return self._F().view(self, shapes)

    def size(self, *dims):
        if len(dims) == 0:
            return self.shape
        if len(dims) == 1:
            return self.shape[dims[0]]
        return tuple(self.shape[d] for d in dims)

    def backward(self, gradients=None, retain_graph=False):
        """Reverse-mode sweep from this tensor (reference xs/core/base.py:343-357)."""
        from . import autograd
        if self.grad_fn is None:
            raise ValueError('can not solve grad on %s' % self)
        if gradients is not None:
            g = gradients.eval if isinstance(gradients, Tensor) else gradients
            if is_device(self._data):
                self._grad = Tensor(g if is_device(g) else to_device(np.asarray(g), np.float32))
            else:
                g = np.asarray(g.numpy() if is_device(g) else g, dtype=self._data.dtype)
                assert g.shape == tuple(self.shape)
                self._grad = Tensor(g)
        elif self._data.size == 1:
            if self._grad is None:
                if is_device(self._data) and self._data.dtype == np.float32:
                    from ..backend import kernels as K
                    self._grad = Tensor(K.full(self._data.shape, 1.0))      # written on the device: no host wait
                else:
                    one = np.array(1., dtype=self._data.dtype).reshape(self._data.shape)
                    self._grad = Tensor(to_device(one) if is_device(self._data) else one)
        else:
            raise ValueError('grad can be implicitly created only for scalar outputs')
        GLOBAL.OUTPUTS = self
        autograd.backward(self, GLOBAL.INPUTS, retain_graph)


class Parameter(Tensor):
    """A trainable leaf (reference xs/core/base.py:360-371)."""

    def __new__(cls, *args, **kwargs):
        if len(args) and isinstance(args[0], Parameter):
            return args[0]
        return object.__new__(cls)

    def __init__(self, t=None, **kwargs):
        if isinstance(t, Parameter):
            return
        if isinstance(t, Tensor):
            Tensor.__init__(self, t._data, t.requires_grad, None, t.name, **kwargs)
        else:
            Tensor.__init__(self, t, requires_grad=True)
