"""Reverse-mode sweep over the dynamic graph (counterpart of xs/core/autograd.py:5-45)."""
from . import state as GLOBAL
from .base import Parameter
from ..backend import capi as _capi


def topological_sort(ins, outs):
    """Nodes reachable from ``outs`` through in_bounds (Parameters excluded), inputs first."""
    order, seen = [], set()

    def visit(v):
        if ins is not None and v is ins:
            if id(v) not in seen:
                seen.add(id(v))
                order.append(v)
            return
        if id(v) in seen:
            return
        seen.add(id(v))
        for child in v.in_bounds:
            if child is None or isinstance(child, Parameter):
                continue
            visit(child)
        order.append(v)

    visit(outs)
    return order


def _sweep(graph, retain_graph):
    for node in reversed(graph):
        if node.grad_fn is not None:
            node.grad_fn(node)
        for layer in node.next_layers:
            layer.data = None
        keep = retain_graph or node.is_leaf or node.retain_grad()
        kwargs = dict(requires_grad=node.requires_grad, name=node.name, slices=node.slices(),
                      static_graph_tensor=node.is_static)
        if keep:
            node.reset_(retain_grad=node.retain_grad(), grad=node._grad, **kwargs)
        else:
            node.free_memory()
            node.reset_(**kwargs)


def backward(outputs, inputs, retain_graph=False):
    graph = topological_sort(inputs, outputs)
    try:
        _sweep(graph, retain_graph)
    finally:
        _capi.join_side()        # weight gradients that conv layers left on the backend's second stream
    if retain_graph:
        GLOBAL.GRAPH = graph
    else:
        GLOBAL.INPUTS = None
        GLOBAL.OUTPUTS = None
        GLOBAL.GRAPH = None
