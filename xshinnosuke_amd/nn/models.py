"""Sequential / Model (static graph) and Module (dynamic graph), counterparts of xs/nn/models.py.

These are callers of the conv / pool path, not part of it; they reproduce the behaviours that
path depends on: lazily created parameters, per-layer preallocated output tensors re-sliced for a
shorter last batch (written through ``out=``), ``layer.backward()`` in reverse order for static
graphs, and parameter discovery by graph walk for ``Module``.
"""
import contextlib
import pickle
import time

import numpy as np

from ..core import state as GLOBAL
from ..core import autograd
from ..core.base import Tensor, Parameter
from ..layers.base import Layer
from ..layers.normalize import BatchNormalization
from ..layers.convolutional import Conv2D
from ..layers.activators import ReLU
from ..optim import get_optimizer
from ..utils.data import DataSet, DataLoader
from .objectives import get_objective
from . import functional as F
from ..backend.graph import StepGraph


class _Base:
    def __init__(self):
        self._parameters = set()
        self._device = 'cuda' if GLOBAL.USE_CUDA else 'cpu'

    def train(self):
        GLOBAL.TRAINING = True      # the reference sets an unused flag here (models.py:18-22); layers read TRAINING

    def eval(self):
        GLOBAL.TRAINING = False

    def parameters(self, parameters=None):
        if parameters is None:
            return self._parameters
        self._parameters = set(parameters)

    def to(self, dst):
        """'cuda' makes the device the default placement of parameters created from now on and moves the
        existing ones (reference models.py:30-43 swaps the global array module instead)."""
        if dst == 'cuda':
            GLOBAL.USE_CUDA = True
            self._device = 'cuda'
            for p in self._parameters:
                p.cuda_()
        elif dst == 'cpu':
            GLOBAL.USE_CUDA = False
            self._device = 'cpu'
            for p in self._parameters:
                p.cpu_()
        else:
            raise ValueError('unknown destination %r' % (dst,))
        return self


class _Model(_Base):
    def __init__(self):
        super().__init__()
        self.loss = None
        self.optimizer = None
        self._graph = None

    def __call__(self, x, *args, **kwargs):
        return self.forward(x)

    def init_graph_out_tensor(self, x, y):
        raise NotImplementedError

    def _place(self, t):
        return t.cuda() if self._device == 'cuda' and t.device != 'cuda' else t

    def fit(self, x, y, batch_size=None, epochs=1, verbose=1, shuffle=True, validation_data=None,
            validation_split=0., initial_epoch=0):
        x, y = np.asarray(x), np.asarray(y)
        if validation_data is None and 0. < validation_split < 1.:
            split = int(x.shape[0] * validation_split)
            validation_data = (x[-split:], y[-split:])
            x, y = x[:-split], y[:-split]
        loader = DataLoader(DataSet(x, y), batch_size, shuffle, device=self._device)
        history = {'train_loss': [], 'train_acc': [], 'validation_loss': [], 'validation_acc': []}
        self.train()
        # GLOBAL.STEP_GRAPH: the loader refills the same two device tensors for every batch and the static graph
        # writes the same buffers every step, so the third full-batch step is recorded instead of run and every
        # later full batch is one replay; `pred` and `loss` are then the recording's tensors.
        graph, recorded, eager_steps = None, None, 0
        want_graph = GLOBAL.STEP_GRAPH and self._device == 'cuda'
        for epoch in range(initial_epoch, epochs):
            t0 = time.time()
            losses, accs = [], []
            for idx, (bx, by) in enumerate(loader):
                bx, by = self._place(bx), self._place(by)
                if idx == 0 or idx == len(loader) - 1:
                    self.init_graph_out_tensor(bx, by)
                full = bx.shape[0] == loader.batch_size
                record = want_graph and graph is None and full and eager_steps >= 2
                if graph is not None and full:
                    pred, loss = recorded
                    graph.replay()
                    self.optimizer.iterations += 1
                else:
                    if record:
                        graph = StepGraph()
                    with (graph.capture() if record else contextlib.nullcontext()):
                        self.optimizer.zero_grad()
                        pred = self.forward(bx)
                        loss = self.loss.forward(pred, by)
                        self.backward(loss)
                        self.optimizer.step()
                    if record:
                        recorded = (pred, loss)
                        graph.replay()
                    eager_steps += 1
                losses.append(loss.item())
                accs.append(self.loss.calc_acc(pred, by))
            history['train_loss'].append(float(np.mean(losses)))
            history['train_acc'].append(float(np.mean(accs)))
            msg = 'epoch %d/%d - %.2fs - loss %.4f - acc %.4f' % (epoch + 1, epochs, time.time() - t0,
                                                                  history['train_loss'][-1], history['train_acc'][-1])
            if validation_data is not None:
                vacc, vloss = self.evaluate(validation_data[0], validation_data[1], batch_size)
                history['validation_loss'].append(vloss)
                history['validation_acc'].append(vacc)
                msg += ' - val_loss %.4f - val_acc %.4f' % (vloss, vacc)
                self.train()
            if verbose:
                print(msg)
        return history

    def backward(self, loss):
        """Static-graph sweep: the loss's grad_fn, then every layer in reverse (reference models.py:138-144)."""
        if loss.grad is None:
            loss.zero_grad()
            loss.grad.fill_(1.)
        loss.grad_fn(loss)
        for layer in reversed(self._graph):
            layer.backward()
        GLOBAL.INPUTS = None

    def evaluate(self, x, y, batch_size=None):
        self.eval()
        x, y = np.asarray(x), np.asarray(y)
        accs, losses = [], []
        with GLOBAL.no_grad():
            loader = DataLoader(DataSet(x, y), batch_size if batch_size is not None else x.shape[0], device=self._device)
            for idx, (bx, by) in enumerate(loader):
                bx, by = self._place(bx), self._place(by)
                if idx == 0 or idx == len(loader) - 1:
                    self.init_graph_out_tensor(bx, by)
                pred = self.forward(bx)
                acc, loss = self.loss.metric(pred, by)
                accs.append(acc)
                losses.append(loss)
        GLOBAL.INPUTS = None
        return float(np.mean(accs)), float(np.mean(losses))

    def predict(self, x, batch_size=None):
        self.eval()
        x = np.asarray(x)
        outs = []
        with GLOBAL.no_grad():
            loader = DataLoader(DataSet(x), batch_size if batch_size is not None else x.shape[0], device=self._device)
            for idx, bx in enumerate(loader):
                bx = self._place(bx)
                if idx == 0 or idx == len(loader) - 1:
                    self.init_graph_out_tensor(bx, None)
                outs.append(self.forward(bx).numpy().copy())
        GLOBAL.INPUTS = None
        return Tensor(np.concatenate(outs, axis=0))

    def save(self, save_path):
        """Pickle ``[graph, optimizer, loss]`` (reference xs/nn/models.py:188-192).  Device arrays are
        written as host arrays, so a checkpoint made on the GPU loads anywhere."""
        if not save_path.endswith('.pkl'):
            save_path += '.pkl'
        with open(save_path, 'wb') as f:
            pickle.dump([self._graph, self.optimizer, self.loss], f)

    def load(self, model_path):
        """Counterpart of reference xs/nn/models.py:194-202; additionally re-collects the parameter set
        from the loaded layers.  Only load files this package wrote: unpickling runs code."""
        if not model_path.endswith('.pkl'):
            model_path += '.pkl'
        with open(model_path, 'rb') as f:
            graph, optimizer, loss = pickle.load(f)
        self._graph = graph
        self.optimizer = optimizer
        self.loss = loss
        self._parameters = set()
        for layer in self._graph:
            for v in (layer.parameters() if hasattr(layer, 'parameters') else []):
                if v is not None:
                    self._parameters.add(v)
        if any(p.device == 'cuda' for p in self._parameters):
            self._device = 'cuda'

    def __str__(self):
        rows = ['%-24s %-20s %10s' % ('Layer', 'Output shape', 'Params')]
        total = 0
        for layer in self._graph or []:
            n = layer.params_count() if isinstance(layer, Layer) else 0
            total += n
            rows.append('%-24s %-20s %10d' % (layer.__class__.__name__, (None,) + tuple(layer.shape or ()), n))
        rows.append('Total params: %d' % total)
        return '\n'.join(rows)


def _owns_static_output(*layers):
    """True if one of the layers holds a preallocated static-graph output tensor.  fit / evaluate / predict give
    every layer one before the first forward; such layers are driven one by one (their outputs are distinct
    buffers that the layer-wise backward relies on), so the fused forms below leave them alone -- also when the
    graph's first input, a loader's batch tensor, is a dynamic tensor."""
    return any(isinstance(l, Layer) and isinstance(l._data, Tensor) and l._data.is_static for l in layers)


class Sequential(_Model):
    def __init__(self, *layers):
        super().__init__()
        self._graph = list(layers)
        self._initialized = False

    def add(self, layer):
        self._graph.append(layer)

    def pop(self, index=-1):
        return self._graph.pop(index)

    def init_graph_out_tensor(self, x, y):
        for layer in self._graph:
            layer.init_layer_out_tensor(x)
            x = layer.data

    def init_params(self, input_shape=None):
        for layer in self._graph:
            if isinstance(layer, _Model):
                continue
            if len(layer.parameters()) == 0:
                layer.init_params(input_shape)
            for v in layer.parameters():
                if v is not None:
                    self._parameters.add(v)
            input_shape = layer.compute_output_shape(input_shape)
        self._initialized = True

    def compile(self, optimizer, loss, **kwargs):
        assert self._graph
        prev = None
        for layer in self._graph:
            layer.connect(prev)
            prev = layer
        self.init_params(self._graph[0]._input_shape)
        self.loss = get_objective(loss)
        self.optimizer = get_optimizer(optimizer, parameters=self._parameters, **kwargs)
        if GLOBAL.USE_CUDA:
            self.to('cuda')

    def forward(self, x, *args, **kwargs):
        layers = self._graph
        i, n = 0, len(layers)
        while i < n:
            layer = layers[i]
            nxt = layers[i + 1] if i + 1 < n else None
            # BatchNormalization followed by an in-place ReLU on a device-resident dynamic graph: one kernel does
            # both (same values and gradients as the two layers; the ReLU layer's output is the same tensor, as
            # an in-place activation's is).  Static graphs drive the layers' backward one by one and are left alone.
            if (isinstance(layer, BatchNormalization) and isinstance(nxt, ReLU) and nxt.inplace and
                    isinstance(x, Tensor) and x.is_dynamic and x.device == 'cuda' and not _owns_static_output(layer, nxt)):
                x = layer.forward(x, fuse_relu=True)
                nxt.data = x
                i += 2
            # Inference (moving statistics, nothing to differentiate) of Conv2D -> BatchNormalization [-> ReLU] on a
            # device-resident dynamic graph: the normalisation is a per-filter scale and shift, folded into the
            # convolution.  All the layers involved then hold the same output tensor.
            elif (isinstance(layer, Conv2D) and layer.activation is None and layer._act_layer is None and
                    isinstance(nxt, BatchNormalization) and
                    nxt.axis == 1 and not GLOBAL.TRAINING and not GLOBAL.COMPUTE_GRAD and isinstance(x, Tensor) and
                    x.is_dynamic and x.device == 'cuda' and len(layer._parameters) and len(nxt._parameters) and
                    not _owns_static_output(layer, nxt, layers[i + 2] if i + 2 < n else None)):
                relu = layers[i + 2] if i + 2 < n and isinstance(layers[i + 2], ReLU) else None
                x.next_layers.append(layer)
                weight, bias = layer._parameters[0], (layer._parameters[1] if layer.use_bias else None)
                gamma, beta = nxt._parameters
                # as in the layers' own calls, the previous output tensor is written again when it still fits
                prev = layer.data if isinstance(layer.data, Tensor) and layer.data.device == 'cuda' else None
                if prev is not None:
                    oh, ow = F.K.conv_out_hw(x.shape[2], x.shape[3], weight.shape[2], weight.shape[3], layer.stride, layer.pad_size)
                    if tuple(prev.shape) != (x.shape[0], weight.shape[0], oh, ow):
                        prev = None
                x = F.conv2d_batch_norm_inference(x, weight, bias, layer.stride, layer.pad_size, gamma, beta, nxt.moving_mean,
                                                  nxt.moving_variance, nxt.epsilon, prev, 'relu' if relu is not None else None)
                layer.data = x
                nxt.data = x
                i += 2
                if relu is not None:
                    relu.data = x
                    i += 1
            else:
                x = layer.forward(x)
                i += 1
        return x


class Model(_Model):
    def __init__(self, inputs=None, outputs=None):
        super().__init__()
        self.inputs = inputs
        self.outputs = outputs

    def init_graph_out_tensor(self, x, y):
        self.inputs._data = x
        for layer in self._graph[1:]:
            layer.init_layer_out_tensor()

    def compile(self, optimizer, loss, **kwargs):
        assert self.inputs is not None and self.outputs is not None
        self._graph = autograd.topological_sort(self.inputs, self.outputs)
        for g in self._graph:
            if len(g.parameters()) == 0:
                g.init_params(g._input_shape)
            for v in g.parameters():
                if v is not None:
                    self._parameters.add(v)
        self.loss = get_objective(loss)
        self.optimizer = get_optimizer(optimizer, parameters=self._parameters, **kwargs)
        if GLOBAL.USE_CUDA:
            self.to('cuda')

    def forward(self, x, *args, **kwargs):
        self.inputs._data = x
        out = None
        for layer in self._graph[1:]:
            out = layer.forward()
        return out


class Module(_Base):
    """Dynamic graph: subclasses define ``forward``; parameters are collected after each call by walking
    the graph from the input along ``out_bounds`` (reference models.py:341-360)."""

    def __call__(self, x, *args, **kwargs):
        out = self.forward(x)
        self._collect(x)
        out.is_leaf = True
        return out

    def _collect(self, x):
        queue, seen = [x], {id(x)}
        while queue:
            v = queue.pop(0)
            for n in v.out_bounds:
                if id(n) not in seen:
                    for p in n.in_bounds:
                        if isinstance(p, Parameter):
                            self._parameters.add(p)
                    queue.append(n)
                    seen.add(id(n))

    def forward(self, x):
        raise NotImplementedError
