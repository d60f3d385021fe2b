"""Array-level wrappers of the conv / max-pool entry points.

Each function takes and returns :class:`DeviceArray` values, checks shapes on
the host before anything is launched, and raises ``ValueError`` for geometry
the reference would also reject.
"""
import ctypes
import os
import weakref

import numpy as np

from . import capi
from .capi import lib, CONV_RELU, CONV_BF16, CONV_WS_PACKED, CONV_DW_ASYNC
from . import array as _array
from .array import DeviceArray, Workspace, empty

_ws = Workspace()
_ws_dw = Workspace()        # weight-gradient scratch of conv2d_bwd: lives beside _ws because the two kernels overlap


def conv_out_hw(h, w, r, s, stride, pad):
    if stride[0] < 1 or stride[1] < 1 or pad < 0:
        raise ValueError("stride must be positive and padding non-negative (got %s, %s)" % (stride, pad))
    return (h + 2 * pad - r) // stride[0] + 1, (w + 2 * pad - s) // stride[1] + 1


def _dims(x_shape, w_shape, stride, pad):
    n, c, h, w = x_shape
    k, c2, r, s = w_shape
    if c2 != c:
        raise ValueError("conv2d: input has %d channels, weight expects %d" % (c, c2))
    return [int(v) for v in (n, c, h, w, k, r, s, stride[0], stride[1], pad)]


_NEED = {}                  # geometry -> xsmi_conv2d_workspace_bytes (a pure function of the ten numbers)


def _need(dims):
    key = tuple(dims)
    need = _NEED.get(key)
    if need is None:
        need = _NEED[key] = lib.raw("xsmi_conv2d_workspace_bytes")(*dims)
    return need


def _need_pass(dims, pass_):
    """Workspace of one fp32 pass alone (0 forward, 1 backward-data): what a filter's layout workspace holds."""
    key = (pass_,) + tuple(dims)
    need = _NEED.get(key)
    if need is None:
        need = _NEED[key] = lib.raw("xsmi_conv2d_pass_workspace_bytes")(*dims, pass_, 0)
    return need


def conv2d_workspace_bytes(x_shape, w_shape, stride, pad):
    """Bytes of workspace the conv entry points want for this geometry."""
    return _need(_dims(x_shape, w_shape, stride, pad))


def _workspace(dims):
    return _ws.get(_need(dims))


# ---- filter layouts made ahead of time -----------------------------------------------------------------------
# Every conv call first rewrites its filter into the layout its kernel reads: a launch of a few microseconds in
# front of each of the ~40 convolution passes of a ResNet-18 training step, on the critical path although the
# filters only change once per step.  A training forward / backward therefore works in a workspace of its own per
# (filter, pass, geometry), and right after an optimizer step `refresh_layouts` lays all filters used since the
# previous one out again on the library's second stream (xsmi_conv2d_pack), beside the start of the next step.  A
# call that finds its workspace's layout still belonging to the filter's current contents (DeviceArray.state)
# skips the layout launch (XSMI_CONV_WS_PACKED).  XSMI_PREPACK=0 switches this off.
_PREPACK = os.environ.get("XSMI_PREPACK", "1") not in ("", "0")
_LAYOUTS = weakref.WeakKeyDictionary()        # filter's memory block -> {(pass, dims): _Layout}


def _filter_key(w):
    """What a layout of filter ``w`` is valid for: the filter's hand-out count, and the count of step-graph replays
    (a replay changes parameters without Python taking their address)."""
    return (w.state(), _array._REPLAYS[0])


class _Layout:
    __slots__ = ("ws", "key", "used", "ahead")

    def __init__(self):
        self.ws = Workspace()
        self.key = None       # _filter_key of the filter when the workspace's layout was made
        self.used = False     # a convolution ran in this workspace since the last refresh
        self.ahead = True     # False once xsmi_conv2d_pack reported that this geometry has nothing to lay out ahead


def _layout_for(w, pass_, dims):
    """(entry, current): the layout workspace of this filter, pass and geometry, and whether it already holds the
    layout of the filter's present contents.  Waits for layouts still on the second stream."""
    blk = w._block
    if w._offset or blk.lazy_zero or (blk.cl is not None and blk.cl.valid):
        return None, False
    entries = _LAYOUTS.get(blk)
    if entries is None:
        entries = _LAYOUTS[blk] = {}
    key = (pass_,) + tuple(dims)
    entry = entries.get(key)
    if entry is None:
        entry = entries[key] = _Layout()
    entry.used = True
    if capi._layouts_pending[0]:                  # the workspace may still be written on the second stream
        capi.join_side()
    return entry, entry.key is not None and entry.key == _filter_key(w)


_plan = {"sig": None, "jobs": None}


def _options_changed():
    """A kernel-selection switch of the library changed: sizes and layouts made for the old selection are void."""
    _NEED.clear()
    for entries in list(_LAYOUTS.values()):
        entries.clear()
    _plan["sig"] = _plan["jobs"] = None


capi._option_listeners.append(_options_changed)


def refresh_layouts(arrays):
    """After an update of ``arrays`` (an optimizer step): every filter among them whose layouts were used since the
    last refresh gets them made again, on the second stream, in one call; layouts that were not used are dropped."""
    if not _LAYOUTS:
        return
    todo = []
    for v in arrays:
        entries = _LAYOUTS.get(v._block)
        if not entries:
            continue
        for key in [k for k, e in entries.items() if not e.used]:
            del entries[key]
        for key, e in entries.items():
            e.used = False
            e.key = None
            if e.ahead:
                todo.append((v, e, key))
    if not todo:
        return
    # the job table is rebuilt only when the set of layouts changes (and while a step graph records, which must see
    # every buffer's address being taken)
    sig = tuple((v.address(), e.ws.address(), key) for v, e, key in todo)
    if sig != _plan["sig"] or _array._CAPTURE[0] is not None:
        jobs = (capi.PackJob * len(todo))()
        for job, (v, e, (pass_, *dims)) in zip(jobs, todo):
            ws, ws_bytes = e.ws.get(_need_pass(dims, pass_))
            job.w, job.workspace, job.workspace_bytes = v.ptr, ws.value, ws_bytes
            job.N, job.C, job.H, job.W, job.K, job.R, job.S, job.sh, job.sw, job.pad = dims
            job.pass_ = pass_
        _plan["sig"], _plan["jobs"] = sig, jobs
    jobs = _plan["jobs"]
    lib.call("xsmi_conv2d_pack", len(todo), ctypes.cast(jobs, ctypes.c_void_p))
    if _array._CAPTURE[0] is not None:
        # The recorded step reads these workspaces as already laid out and lays them out again at its end; whoever
        # changes a filter between two replays leaves them stale, so the graph keeps the jobs to redo them first.
        _array._CAPTURE[0].note_layout_jobs(jobs, len(todo), [v for v, _, _ in todo])
        _plan["sig"] = _plan["jobs"] = None       # the table now belongs to the graph
    held = []
    for job, (v, e, _) in zip(jobs, todo):
        if job.packed:
            e.key = _filter_key(v)
            held.append((v, e.ws))
        else:
            e.ahead = False
    if held:
        capi.layouts_enqueued(*held)


def _f32(a, what):
    if not isinstance(a, DeviceArray) or a.dtype != np.float32:
        raise TypeError("%s must be a float32 DeviceArray" % what)
    return a


def conv2d_fwd(x, w, bias=None, stride=(1, 1), pad=0, relu=False, out=None, neg_mask=None, bf16=False, packed=False,
               workspace=None, channels_last=False, keep_layout=False):
    """``keep_layout=True`` (training steps; fp32, the shared workspace): the call works in a workspace that belongs
    to this filter, pass and geometry, whose layout ``refresh_layouts`` renews after each update of the filter.
    ``packed=True`` promises that the previous conv call on this workspace was this same forward with the same
    geometry and filter values (the workspace still holds the filter's packed form), so it is not laid out again.
    ``workspace``: a ``Workspace`` of the caller's instead of the shared one (a layer that keeps its packed filter).
    ``channels_last=True`` (with ``bf16``, no mask): the result may be left in channels-last bf16 form, and an input
    that lives in that form is read as it is (``DeviceArray.channels_last``); results equal the plain bf16 path's up
    to the bf16 rounding of the stored activations."""
    _f32(x, "x"); _f32(w, "w")
    dims = _dims(x.shape, w.shape, stride, pad)
    n, c, h, wd, k, r, s = dims[:7]
    oh, ow = conv_out_hw(h, wd, r, s, stride, pad)
    if oh <= 0 or ow <= 0:
        raise ValueError("conv2d: filter %dx%d does not fit the padded input %dx%d" % (r, s, h + 2 * pad, wd + 2 * pad))
    if bias is not None:
        _f32(bias, "bias")
        if bias.size != k:
            raise ValueError("conv2d: bias has %d elements for %d filters" % (bias.size, k))
    if out is None:
        out = empty((n, k, oh, ow))
    elif out.shape != (n, k, oh, ow):
        raise ValueError("conv2d: out has shape %s, expected %s" % (out.shape, (n, k, oh, ow)))
    if neg_mask is not None and (neg_mask.dtype != np.uint8 or neg_mask.size != out.size):
        raise ValueError("conv2d: neg_mask must be uint8 with one byte per output element")
    layout = None
    if keep_layout and _PREPACK and not bf16 and not packed and workspace is None:
        layout, packed = _layout_for(w, 0, dims)
        if layout is not None:
            workspace = layout.ws
    flags = (CONV_RELU if relu else 0) | (CONV_BF16 if bf16 else 0) | (CONV_WS_PACKED if packed else 0)
    if layout is not None:
        ws, ws_bytes = workspace.get(_need_pass(dims, 0))
    else:
        ws, ws_bytes = _workspace(dims) if workspace is None else workspace.get(_need(dims))
    if channels_last and bf16 and neg_mask is None:
        xcl = x.channels_last()
        if xcl is not None and not (c % 32 == 0 and xcl.border >= pad):
            xcl = None                                # read through the float32 form (x.cptr converts)
        if xcl is not None or c % 32 == 0 or c <= 8:
            ycl = out.channels_last_out(1) if k % 8 == 0 else None
            lib.call("xsmi_conv2d_fwd_cl", None if xcl is not None else x.cptr, xcl.buf.cptr if xcl is not None else None,
                     xcl.border if xcl is not None else 0, w.cptr, bias.cptr if bias is not None else None,
                     None if ycl is not None else out.cptr, ycl.buf.cptr if ycl is not None else None, 1, *dims,
                     flags & ~CONV_BF16, ws, ws_bytes)
            return out
    out._overwritten()
    # a filter whose layout is in place is not read: its address goes along without counting as handed out
    wptr = ctypes.c_void_p(w.address()) if layout is not None and packed else w.cptr
    lib.call("xsmi_conv2d_fwd", x.cptr, wptr, bias.cptr if bias is not None else None, out.cptr,
             neg_mask.cptr if neg_mask is not None else None, *dims, flags, ws, ws_bytes)
    if layout is not None and not packed:
        layout.key = _filter_key(w)               # the call has laid the present filter out in this workspace
    return out


def _beta(accumulate, *outs):
    """1.0 to add into the outputs, 0.0 to overwrite them.  Outputs that are all pending all-zero
    buffers are overwritten instead of cleared and added to; in a mix the pending ones are cleared
    for real when their pointer is taken."""
    outs = [o for o in outs if o is not None]
    if accumulate and not all(o.is_fresh() for o in outs):
        return 1.0
    for o in outs:
        o.take_fresh()
    return 0.0


def conv2d_bwd_data(dy, w, x_shape, stride=(1, 1), pad=0, dx=None, accumulate=False, bf16=False, packed=False,
                    keep_layout=False):
    _f32(dy, "dy"); _f32(w, "w")
    dims = _dims(x_shape, w.shape, stride, pad)
    n, c, h, wd, k, r, s = dims[:7]
    oh, ow = conv_out_hw(h, wd, r, s, stride, pad)
    if dy.shape != (n, k, oh, ow):
        raise ValueError("conv2d backward: dy has shape %s, expected %s" % (dy.shape, (n, k, oh, ow)))
    if dx is None:
        dx = empty(x_shape)
        accumulate = False
    elif dx.shape != tuple(x_shape):
        raise ValueError("conv2d backward: dx has shape %s, expected %s" % (dx.shape, tuple(x_shape)))
    layout = None
    if keep_layout and _PREPACK and not bf16 and not packed:
        layout, packed = _layout_for(w, 1, dims)
    ws, ws_bytes = _workspace(dims) if layout is None else layout.ws.get(_need_pass(dims, 1))
    beta = _beta(accumulate, dx)
    wptr = ctypes.c_void_p(w.address()) if layout is not None and packed else w.cptr
    lib.call("xsmi_conv2d_bwd_data", dy.cptr, wptr, dx.cptr, *dims, beta,
             (CONV_BF16 if bf16 else 0) | (CONV_WS_PACKED if packed else 0), ws, ws_bytes)
    if layout is not None and not packed:
        layout.key = _filter_key(w)
    return dx


def conv2d_bwd_weight(dy, x, w_shape, stride=(1, 1), pad=0, dw=None, db=None, accumulate=False, want_db=False,
                      bf16=False):
    _f32(dy, "dy"); _f32(x, "x")
    dims = _dims(x.shape, w_shape, stride, pad)
    n, c, h, wd, k, r, s = dims[:7]
    oh, ow = conv_out_hw(h, wd, r, s, stride, pad)
    if dy.shape != (n, k, oh, ow):
        raise ValueError("conv2d backward: dy has shape %s, expected %s" % (dy.shape, (n, k, oh, ow)))
    if dw is None:
        dw = empty(w_shape)
        if db is None and want_db:
            db = empty((k,))
        accumulate = False
    elif dw.shape != tuple(w_shape):
        raise ValueError("conv2d backward: dw has shape %s, expected %s" % (dw.shape, tuple(w_shape)))
    if db is not None and db.size != k:
        raise ValueError("conv2d backward: db has %d elements for %d filters" % (db.size, k))
    ws, ws_bytes = _workspace(dims)
    beta = _beta(accumulate, dw, db)
    lib.call("xsmi_conv2d_bwd_weight", dy.cptr, x.cptr, dw.cptr, db.cptr if db is not None else None, *dims,
             beta, CONV_BF16 if bf16 else 0, ws, ws_bytes)
    return dw, db


def conv2d_bwd(dy, x, w, dx, dw, db=None, stride=(1, 1), pad=0, accumulate=False, bf16=False, async_dw=False,
               keep_layout=False):
    """Both gradients of one layer in one call, into existing device buffers.  Same results as ``conv2d_bwd_weight``
    followed by ``conv2d_bwd_data``.  ``async_dw=True`` leaves the weight gradient running on the library's second
    stream beside whatever is enqueued next; dw and db are complete after ``capi.join_side()``, which every call into
    the library performs by itself except the passes of a backward sweep that cannot touch them."""
    _f32(dy, "dy"); _f32(x, "x"); _f32(w, "w")
    dims = _dims(x.shape, w.shape, stride, pad)
    n, c, h, wd, k, r, s = dims[:7]
    oh, ow = conv_out_hw(h, wd, r, s, stride, pad)
    if dy.shape != (n, k, oh, ow):
        raise ValueError("conv2d backward: dy has shape %s, expected %s" % (dy.shape, (n, k, oh, ow)))
    if dx.shape != tuple(x.shape) or dw.shape != tuple(w.shape):
        raise ValueError("conv2d backward: dx %s / dw %s do not match x %s / w %s" % (dx.shape, dw.shape, x.shape, w.shape))
    if db is not None and db.size != k:
        raise ValueError("conv2d backward: db has %d elements for %d filters" % (db.size, k))
    need = _need(dims)
    if capi.side_pending() and not _ws_dw.holds(need):
        capi.join_side()                        # the block about to be replaced may still be in use
    layout, packed = None, False
    if keep_layout and _PREPACK and not bf16:
        layout, packed = _layout_for(w, 1, dims)          # the data gradient's filter layout
    ws, ws_bytes = _ws.get(need) if layout is None else layout.ws.get(_need_pass(dims, 1))
    ws_dw, ws_dw_bytes = _ws_dw.get(need)
    beta_dw = _beta(accumulate, dw, db)
    beta_dx = _beta(accumulate, dx)
    flags = (CONV_BF16 if bf16 else 0) | (CONV_DW_ASYNC if async_dw else 0) | (CONV_WS_PACKED if packed else 0)
    wptr = ctypes.c_void_p(w.address()) if layout is not None and packed else w.cptr
    lib.call("xsmi_conv2d_bwd", dy.cptr, x.cptr, wptr, dx.cptr, dw.cptr, db.cptr if db is not None else None, *dims,
             beta_dx, beta_dw, flags, ws, ws_bytes, ws_dw, ws_dw_bytes)
    if layout is not None and not packed:
        layout.key = _filter_key(w)
    if async_dw:
        capi.hold_side(dy, x, dw, db)
    return dx, dw, db


def pool_out_hw(h, w, k, stride, pad):
    if stride[0] < 1 or stride[1] < 1 or pad < 0:
        raise ValueError("stride must be positive and padding non-negative (got %s, %s)" % (stride, pad))
    return (h + 2 * pad - k) // stride[0] + 1, (w + 2 * pad - k) // stride[1] + 1


def maxpool2d_fwd(x, k, stride, pad=0, out=None, idx=None, want_idx=True):
    _f32(x, "x")
    n, c, h, w = x.shape
    oh, ow = pool_out_hw(h, w, k, stride, pad)
    if oh <= 0 or ow <= 0:
        raise ValueError("max_pool2d: window %d does not fit the padded input %dx%d" % (k, h + 2 * pad, w + 2 * pad))
    # a normalisation of x that has not been launched yet is taken out of the queue first (an allocation below may
    # call into the library, which would launch it)
    entry = capi.take_deferred_bn(x, None)
    try:
        if out is None:
            out = empty((n, c, oh, ow))
        elif out.shape != (n, c, oh, ow):
            raise ValueError("max_pool2d: out has shape %s, expected %s" % (out.shape, (n, c, oh, ow)))
        if idx is None and want_idx:
            idx = empty((n, c, oh, ow), np.uint8)
    except Exception:
        if entry is not None:
            entry.launch()                            # what was asked for before this call still happens
        raise
    if entry is not None:
        # the input is a normalisation with a ReLU that has not been launched yet: the head of a ResNet in one pass
        if (entry.relu_mask is not None and k == 3 and tuple(stride) == (2, 2) and pad == 1 and h % 2 == 0 and w % 4 == 0
                and out.is_whole()):
            out.take_fresh()
            entry.launch(pooled=out, idx=idx)
            return out, idx
        entry.launch()
    xcl = x.channels_last() if idx is None else None
    if xcl is not None and xcl.border >= pad:         # no argmax wanted and the input lives in channels-last form
        ycl = out.channels_last_out(1)
        if ycl is not None:
            lib.call("xsmi_cl_maxpool2d", xcl.buf.cptr, xcl.border, ycl.buf.cptr, ycl.border, n, c, h, w, int(k),
                     int(stride[0]), int(stride[1]), int(pad))
            return out, None
    lib.call("xsmi_maxpool2d_fwd", x.cptr, out.cptr, idx.cptr if idx is not None else None,
             n, c, h, w, int(k), int(stride[0]), int(stride[1]), int(pad))
    return out, idx


def maxpool2d_bwd(dy, idx, x_shape, k, stride, pad=0, dx=None, accumulate=False):
    _f32(dy, "dy")
    n, c, h, w = x_shape
    oh, ow = pool_out_hw(h, w, k, stride, pad)
    if dy.shape != (n, c, oh, ow) or idx.size != dy.size or idx.dtype != np.uint8:
        raise ValueError("max_pool2d backward: dy/idx do not match the pooled shape %s" % ((n, c, oh, ow),))
    if dx is None:
        dx = empty(x_shape)
        accumulate = False
    elif dx.shape != tuple(x_shape):
        raise ValueError("max_pool2d backward: dx has shape %s, expected %s" % (dx.shape, tuple(x_shape)))
    beta = _beta(accumulate, dx)
    if (FUSE_BN_ADD_RELU and beta == 0.0 and k == 3 and tuple(stride) == (2, 2) and pad == 1 and h % 2 == 0 and w % 4 == 0
            and dx.is_whole()):
        # held back: if the next call is the backward of the normalisation that fed the pool, the routed gradient is
        # formed inside that backward (bn_bwd) and never stored
        e = PoolBwdEntry()
        e.dy, e.idx, e.dx, e.dims = dy, idx, dx, (n, c, h, w)
        dy.ptr; idx.ptr                               # pending clears are settled now
        capi.defer_pool_bwd(e)
        return dx
    lib.call("xsmi_maxpool2d_bwd", dy.cptr, idx.cptr, dx.cptr, n, c, h, w, int(k), int(stride[0]), int(stride[1]),
             int(pad), beta)
    return dx


class PoolBwdEntry:
    """The gradient of a 3x3 / stride 2 / pad 1 max-pool into a buffer that is overwritten, asked for and not launched
    yet (see capi._deferred)."""

    __slots__ = ("dy", "idx", "dx", "dims")

    def arrays(self):
        return (self.dy, self.idx, self.dx)

    def launch(self):
        n, c, h, w = self.dims
        lib.call("xsmi_maxpool2d_bwd", self.dy.cptr, self.idx.cptr, self.dx.cptr, n, c, h, w, 3, 2, 2, 1, 0.0)


def relu_mask_bwd(dy, neg_mask, dx=None, accumulate=False):
    _f32(dy, "dy")
    if dx is None:
        dx = empty(dy.shape)
        accumulate = False
    beta = 0.0 if dx is dy else _beta(accumulate, dx)
    lib.call("xsmi_relu_mask_bwd", dy.cptr, neg_mask.cptr, dx.cptr, dy.size, beta)
    return dx


def relu_mask_bwd2(dy, neg_mask, dx1, dx2, accumulate=True):
    """The masked gradient (0 where neg_mask is set, else dy) added into (or written over) two tensors at once."""
    _f32(dy, "dy")
    if dx1.size != dy.size or dx2.size != dy.size or dx1 is dx2:
        raise ValueError("relu_mask_bwd2: needs two different outputs of dy's size")
    b1, b2 = _beta(accumulate, dx1), _beta(accumulate, dx2)
    lib.call("xsmi_relu_mask_bwd2", dy.cptr, neg_mask.cptr, dx1.cptr, b1, dx2.cptr, b2, dy.size)
    return dx1, dx2


def copy_kernel(dst, src):
    lib.call("xsmi_copy_kernel", dst.cptr, src.cptr, src.nbytes)


# ---- neighbours of conv / pool (device-resident element-wise, normalisation, reduction ops) ----
def _like(a, out):
    if out is None:
        return empty(a.shape)
    if out.size != a.size:
        raise ValueError("output has %d elements, expected %d" % (out.size, a.size))
    return out


def axpy(y, x, a):
    """y += a * x"""
    _f32(y, "y"); _f32(x, "x")
    if x.size != y.size:
        raise ValueError("axpy: %s vs %s" % (x.shape, y.shape))
    if y.take_fresh():                        # y is a pending all-zero buffer: y = a * x, no clear, no read of y
        if float(a) == 1.0:
            return y.copy_from(x)
        lib.call("xsmi_scale_shift", x.cptr, y.cptr, float(a), 0.0, y.size)
        return y
    lib.call("xsmi_axpy", y.cptr, x.cptr, float(a), y.size)
    return y


def axpy_multi(ys, xs, a):
    """y += a * x for every pair, in one launch per 48 tensors (one optimizer step over all parameters)."""
    n = len(ys)
    if n == 0:
        return
    for y, x in zip(ys, xs):
        _f32(y, "y"); _f32(x, "x")
        if x.size != y.size:
            raise ValueError("axpy_multi: %s vs %s" % (x.shape, y.shape))
    yp = (ctypes.c_void_p * n)(*[y.ptr for y in ys])
    xp = (ctypes.c_void_p * n)(*[x.ptr for x in xs])
    ns = (ctypes.c_size_t * n)(*[y.size for y in ys])
    lib.call("xsmi_axpy_multi", n, yp, xp, ns, float(a))


def add(a, b, out=None, defer=False):
    """``defer=True`` (new result array only) holds the launch back until the next call into the library, so that
    an in-place ReLU of the result can run in the same pass; any other call enqueues the add first."""
    _f32(a, "a"); _f32(b, "b")
    if defer and out is None and a.size == b.size:
        entry = capi.take_deferred_bn(a, b) if a is not b else None
        if entry is not None and entry.relu_mask is not None:       # a normalisation with a ReLU of its own: as it is
            entry.launch()
            entry = None
        try:
            out = empty(a.shape)
        except Exception:
            if entry is not None:
                entry.launch()                        # what was asked for before this call still happens
            raise
        if entry is not None:
            # one operand is a normalisation that has not been launched yet: both wait for the call after this one
            (b if entry.y is a else a).ptr            # the other operand: a pending clear is carried out now
            capi.defer_bn_add(entry, a, b, out)
            return out
        acl, bcl = a.channels_last(), b.channels_last()
        if acl is None or bcl is None or not acl.same_layout(bcl):
            a.ptr; b.ptr                              # operands with a pending clear are cleared now
        capi.defer_add(a, b, out)
        return out
    out = _like(a, out)
    lib.call("xsmi_add", a.cptr, b.cptr, out.cptr, a.size)
    return out


def scale(a, s, t=0.0, out=None):
    _f32(a, "a")
    out = _like(a, out)
    lib.call("xsmi_scale_shift", a.cptr, out.cptr, float(s), float(t), a.size)
    return out


def add_scalar(a, t, out=None):
    return scale(a, 1.0, t, out)


def relu_fwd(x, out=None):
    _f32(x, "x")
    if out is x:                                      # in place: a held-back add that produced x joins this pass
        ops = capi.take_deferred_add(x)
        if ops is not None:
            acl, bcl = ops[0].channels_last(), ops[1].channels_last()
            if acl is not None and bcl is not None and acl.same_layout(bcl):
                xcl = x.channels_last_out(acl.border)     # both operands live in channels-last form: so does the sum
                if xcl is not None:
                    lib.call("xsmi_cl_add", acl.buf.cptr, bcl.buf.cptr, xcl.buf.cptr, xcl.buf.size, 1)
                    return x
            lib.call("xsmi_add_relu", ops[0].cptr, ops[1].cptr, x.cptr, None, x.size)
            return x
    out = _like(x, out)
    lib.call("xsmi_relu_fwd", x.cptr, out.cptr, x.size)
    return out


def relu_fwd_mask(x, out=None):
    """Returns (max(0, x), uint8 mask of x < 0); ``out`` may be ``x`` itself."""
    _f32(x, "x")
    if out is x:                                      # in place: a held-back add that produced x joins this pass
        ops = capi.take_deferred_add(x, with_bn=True)
        if ops is not None:
            mask = empty(x.shape, np.uint8)
            if len(ops) == 3:                         # ... and the normalisation that produced one of its operands
                entry = ops[2]
                entry.launch(residual=ops[1] if entry.y is ops[0] else ops[0], out=x, neg_mask=mask)
                return x, mask
            lib.call("xsmi_add_relu", ops[0].cptr, ops[1].cptr, x.cptr, mask.cptr, x.size)
            return x, mask
    out = _like(x, out)
    mask = empty(x.shape, np.uint8)
    lib.call("xsmi_relu_fwd_mask", x.cptr, out.cptr, mask.cptr, x.size)
    return out, mask


def relu_bwd(dy, pre, dx=None):
    _f32(dy, "dy"); _f32(pre, "pre")
    dx = _like(dy, dx)
    lib.call("xsmi_relu_bwd", dy.cptr, pre.cptr, dx.cptr, dy.size)
    return dx


ACT_KINDS = {'sigmoid': 1, 'tanh': 2}


def act_fwd(x, kind, out=None):
    """sigmoid or tanh of x (``out`` may be x)."""
    _f32(x, "x")
    out = _like(x, out)
    lib.call("xsmi_act_fwd", x.cptr, out.cptr, x.size, ACT_KINDS[kind])
    return out


def act_bwd(dy, y, kind, dx=None):
    """Gradient of sigmoid / tanh through the forward's output y."""
    _f32(dy, "dy"); _f32(y, "y")
    if y.size != dy.size:
        raise ValueError("act_bwd: %s vs %s" % (dy.shape, y.shape))
    dx = _like(dy, dx)
    lib.call("xsmi_act_bwd", dy.cptr, y.cptr, dx.cptr, dy.size, ACT_KINDS[kind])
    return dx


def lerp_(m, cur, momentum):
    """m = momentum*m + (1-momentum)*cur"""
    lib.call("xsmi_lerp", m.cptr, cur.cptr, float(momentum), m.size)
    return m


def _nchw3(shape):
    n, c = shape[0], shape[1]
    hw = 1
    for d in shape[2:]:
        hw *= d
    return int(n), int(c), int(hw)


FUSE_BN_ADD_RELU = os.environ.get("XSMI_FUSE_BN_ADD_RELU", "1") != "0"


class BnEntry:
    """A training batch normalisation that has been asked for and not launched yet (see capi._deferred)."""

    __slots__ = ("x", "gamma", "beta", "eps", "y", "sqrtvar", "mean", "var", "mm", "mv", "momentum", "dims", "ws",
                 "relu_mask")

    def arrays(self):
        return (self.x, self.gamma, self.beta, self.y, self.sqrtvar, self.mean, self.var, self.mm, self.mv, self.relu_mask)

    def launch(self, residual=None, out=None, neg_mask=None, pooled=None, idx=None):
        """Plain: y = gamma * xhat + beta (clipped at zero, with the sign mask, when the entry has a ReLU of its own).
        With ``residual``: out = max(0, y + residual) and its sign mask in one pass.  With ``pooled``: the 3x3/2
        max-pool of the clipped y (and ``idx``) in one pass.  In both fused forms y itself is never written, and
        reading it raises."""
        n, c, hw = self.dims
        ws, ws_bytes = self.ws
        mm, mv = self.mm, self.mv
        stats = (self.sqrtvar.cptr, self.mean.cptr, self.var.cptr, mm.cptr if mm is not None else None,
                 mv.cptr if mv is not None else None, float(self.momentum))
        if pooled is not None:
            _, _, h, w = self.x.shape
            self.y.never_written("this batch normalisation's result was consumed by the max-pool that followed it, in one "
                                 "pass, and was not stored (XSMI_FUSE_BN_ADD_RELU=0 keeps the passes apart)")
            lib.call("xsmi_bn_relu_maxpool_fwd", self.x.cptr, self.gamma.cptr, self.beta.cptr, pooled.cptr,
                     idx.cptr if idx is not None else None, self.relu_mask.cptr, *stats, n, c, h, w, float(self.eps),
                     ws, ws_bytes)
            return
        if residual is None:
            lib.call("xsmi_bn_fwd", self.x.cptr, self.gamma.cptr, self.beta.cptr, self.y.cptr, None, *stats,
                     self.relu_mask.cptr if self.relu_mask is not None else None, n, c, hw, float(self.eps), ws, ws_bytes)
            return
        self.y.never_written("this batch normalisation's result was consumed by the add and ReLU that followed it, in "
                             "one pass, and was not stored (XSMI_FUSE_BN_ADD_RELU=0 keeps the three passes apart)")
        lib.call("xsmi_bn_add_relu_fwd", self.x.cptr, self.gamma.cptr, self.beta.cptr, residual.cptr, out.cptr, *stats,
                 neg_mask.cptr, n, c, hw, float(self.eps), ws, ws_bytes)


def bn_fwd(x, gamma, beta, eps, y=None, moving=None, momentum=0.0, neg_mask=None, want_xhat=True, defer=False):
    """``moving=(moving_mean, moving_var)`` device arrays are updated in place: m = momentum*m + (1-momentum)*stat.
    A uint8 ``neg_mask`` of x's size fuses a ReLU: it receives pre-activation < 0 and y is clipped at 0.
    ``want_xhat=False`` skips the store of the normalised input (None is returned for it): ``bn_bwd`` forms it
    again from x and the batch mean.  ``defer=True`` (without mask and normalised input) holds the launch back until
    the next call into the library: an add of y and another tensor followed by the in-place ReLU of the sum then runs
    inside the normalisation's second pass, and so does (with ``neg_mask``, i.e. a ReLU of the normalisation's own) a
    3x3 / stride 2 / pad 1 max-pool of y; any other call enqueues the normalisation first."""
    _f32(x, "x")
    n, c, hw = _nchw3(x.shape)
    y = _like(x, y); xhat = empty(x.shape) if want_xhat else None
    y.take_fresh()
    sqrtvar = empty((c,)); mean = empty((c,)); var = empty((c,))
    mm, mv = moving if moving is not None else (None, None)
    if mm is not None and (mm.size != c or mv.size != c):
        raise ValueError("bn_fwd: moving statistics must have %d elements" % c)
    ws, ws_bytes = _ws.get(lib.raw("xsmi_bn_workspace_bytes")(c))
    if defer and FUSE_BN_ADD_RELU and not want_xhat and y.is_whole():
        e = BnEntry()
        e.relu_mask = neg_mask
        e.x, e.gamma, e.beta, e.eps, e.y = x, gamma, beta, eps, y
        e.sqrtvar, e.mean, e.var, e.mm, e.mv, e.momentum = sqrtvar, mean, var, mm, mv, momentum
        e.dims, e.ws = (n, c, hw), (ws, ws_bytes)
        for a in (x, gamma, beta) + ((mm, mv) if mm is not None else ()):
            a.ptr                                     # pending clears and channels-last forms are settled now
        capi.defer_bn(e)
        return y, None, sqrtvar, mean, var
    lib.call("xsmi_bn_fwd", x.cptr, gamma.cptr, beta.cptr, y.cptr, xhat.cptr if want_xhat else None, sqrtvar.cptr,
             mean.cptr, var.cptr,
             mm.cptr if mm is not None else None, mv.cptr if mv is not None else None, float(momentum),
             neg_mask.cptr if neg_mask is not None else None, n, c, hw, float(eps), ws, ws_bytes)
    return y, xhat, sqrtvar, mean, var


def bn_infer(x, gamma, beta, mean, var, eps, y=None, relu=False):
    n, c, hw = _nchw3(x.shape)
    y = _like(x, y)
    y.take_fresh()
    lib.call("xsmi_bn_infer", x.cptr, gamma.cptr, beta.cptr, mean.cptr, var.cptr, y.cptr, n, c, hw, float(eps),
             1 if relu else 0)
    return y


def bn_fold(w, bias, gamma, beta, mean, var, eps):
    """Filter and bias of the convolution that equals conv(w, bias) followed by the inference normalisation."""
    _f32(w, "w")
    k = w.shape[0]
    for a in (gamma, beta, mean, var):
        if a.size != k:
            raise ValueError("bn_fold: %d statistics for %d filters" % (a.size, k))
    if bias is not None and bias.size != k:
        raise ValueError("bn_fold: bias has %d elements for %d filters" % (bias.size, k))
    w_out, b_out = empty(w.shape), empty((k,))
    lib.call("xsmi_bn_fold", w.cptr, bias.cptr if bias is not None else None, gamma.cptr, beta.cptr, mean.cptr, var.cptr,
             w_out.cptr, b_out.cptr, k, w.size // k, float(eps))
    return w_out, b_out


def bn_bwd(dy, xhat, sqrtvar, gamma, dx=None, dgamma=None, dbeta=None, neg_mask=None, mean=None):
    """dx, dgamma, dbeta; buffers passed in are overwritten completely.  ``neg_mask`` is the byte mask of a fused
    ReLU: the upstream gradient counts as 0 where it is set.  With ``mean`` (the batch mean of the forward),
    ``xhat`` is the forward's input x instead of its normalised form."""
    if xhat.size != dy.size or (mean is not None and mean.size != dy.shape[1]):
        raise ValueError("bn_bwd: operands do not match %s" % (dy.shape,))
    n, c, hw = _nchw3(dy.shape)
    # dy may be the gradient of a max-pool that has not been launched yet: it is taken out of the queue first (an
    # allocation below may call into the library, which would launch it)
    pool = capi.take_deferred_pool_bwd(dy)
    try:
        dx = empty(dy.shape) if dx is None else dx
        dgamma = empty((c,)) if dgamma is None else dgamma
        dbeta = empty((c,)) if dbeta is None else dbeta
        if dx.size != dy.size or dgamma.size != c or dbeta.size != c:
            raise ValueError("bn_bwd: output buffers do not match %s" % (dy.shape,))
        for o in (dx, dgamma, dbeta):
            o.take_fresh()
        ws, ws_bytes = _ws.get(lib.raw("xsmi_bn_workspace_bytes")(c))
    except Exception:
        if pool is not None:
            pool.launch()                             # what was asked for before this call still happens
        raise
    if pool is not None:
        if mean is not None and len(dy.shape) == 4 and dx is not dy and dx.is_whole():
            # pool gradient and normalisation gradient as two passes over (pooled gradient, indices, x, mask)
            pn, pc, ph, pw = pool.dims
            dy.never_written("this max-pool gradient was consumed by the batch-norm backward that followed it and was not "
                             "stored (XSMI_FUSE_BN_ADD_RELU=0 keeps the passes apart)")
            lib.call("xsmi_bn_bwd_maxpool", pool.dy.cptr, pool.idx.cptr, xhat.cptr, mean.cptr, sqrtvar.cptr, gamma.cptr,
                     neg_mask.cptr if neg_mask is not None else None, dx.cptr, dgamma.cptr, dbeta.cptr, pn, pc, ph, pw,
                     ws, ws_bytes)
            return dx, dgamma, dbeta
        pool.launch()
    lib.call("xsmi_bn_bwd", dy.cptr, xhat.cptr, mean.cptr if mean is not None else None, sqrtvar.cptr, gamma.cptr,
             neg_mask.cptr if neg_mask is not None else None, dx.cptr, dgamma.cptr, dbeta.cptr, n, c, hw, ws, ws_bytes)
    return dx, dgamma, dbeta


def avgpool_fwd(x, k, stride=None):
    n, c, h, w = x.shape
    sh, sw = (int(k), int(k)) if stride is None else (int(stride[0]), int(stride[1]))
    if k > h or k > w or sh < 1 or sw < 1:
        raise ValueError("avg_pool2d: window %d does not fit the input %dx%d" % (k, h, w))
    y = empty((n, c, (h - k) // sh + 1, (w - k) // sw + 1))
    lib.call("xsmi_avgpool_fwd", x.cptr, y.cptr, n, c, h, w, int(k), sh, sw)
    return y


def avgpool_bwd(dy, x_shape, k, stride=None):
    n, c, h, w = x_shape
    sh, sw = (int(k), int(k)) if stride is None else (int(stride[0]), int(stride[1]))
    if dy.shape != (n, c, (h - k) // sh + 1, (w - k) // sw + 1):
        raise ValueError("avg_pool2d backward: dy %s does not match the pooled shape of %s" % (dy.shape, tuple(x_shape)))
    dx = empty(x_shape)
    lib.call("xsmi_avgpool_bwd", dy.cptr, dx.cptr, n, c, h, w, int(k), sh, sw)
    return dx


def gemm(a, b, bias=None, trans_a=False, trans_b=False, out=None):
    """op(a) @ op(b) (+ bias over rows); a and b are 2-D row-major."""
    _f32(a, "a"); _f32(b, "b")
    m, k = (a.shape[1], a.shape[0]) if trans_a else a.shape
    k2, n = (b.shape[1], b.shape[0]) if trans_b else b.shape
    if k != k2:
        raise ValueError("gemm: inner dimensions %d and %d differ" % (k, k2))
    if out is None:
        out = empty((m, n))
    elif out.size != m * n:
        raise ValueError("gemm: output has shape %s, expected %s" % (out.shape, (m, n)))
    # room for a split of K over the chip when the output is small (the dense layer's batch of rows)
    ws, ws_bytes = _ws.get(min(64 * m * n * 4, 1 << 24))
    lib.call("xsmi_gemm", a.cptr, b.cptr, bias.cptr if bias is not None else None, out.cptr, int(m), int(n), int(k),
             1 if trans_a else 0, 1 if trans_b else 0, ws, ws_bytes)
    return out


def dense_fwd(x, w, b=None, out=None):
    return gemm(x, w, None if b is None else b.reshape(-1), out=out)


def colsum(a):
    m, n = a.shape
    out = empty((n,))
    lib.call("xsmi_colsum", a.cptr, out.cptr, int(m), int(n))
    return out


def sum_all(a):
    out = empty((1,))
    lib.call("xsmi_sum_all", a.cptr, out.cptr, a.size)
    return out


def _labels(labels):
    if labels.dtype != np.int64:
        from .array import to_device
        labels = to_device(labels.numpy().astype(np.int64), np.int64)
    return labels


def softmax_ce_fwd(logits, labels, reduction):
    m, n = logits.reshape(-1, logits.shape[-1]).shape
    labels = _labels(labels)
    sm = empty(logits.shape)
    buf = empty((1 + m,))
    lib.call("xsmi_softmax_ce_fwd", logits.cptr, labels.cptr, sm.cptr, buf.cptr, int(m), int(n),
             1 if reduction == 'mean' else 0)
    return buf.leading(0, 1), sm


def softmax_ce_bwd(sm, labels, reduction, upstream):
    """``upstream``: the loss's gradient, a host scalar or a one-element device array (read on the device, so
    the host does not wait for the forward to finish)."""
    m, n = sm.reshape(-1, sm.shape[-1]).shape
    labels = _labels(labels)
    up_dev = upstream if isinstance(upstream, DeviceArray) else None
    if up_dev is not None and (up_dev.dtype != np.float32 or up_dev.size != 1):
        raise ValueError("softmax_ce_bwd: upstream must be one float32")
    up = 1.0 if up_dev is not None else float(np.asarray(upstream).reshape(-1)[0])
    scale_ = up / m if reduction == 'mean' else up
    dz = empty(sm.shape)
    lib.call("xsmi_softmax_ce_bwd", sm.cptr, labels.cptr, up_dev.cptr if up_dev is not None else None, dz.cptr,
             int(m), int(n), scale_)
    return dz


def full(shape, value):
    out = empty(shape)
    lib.call("xsmi_fill", out.cptr, float(value), out.size)
    return out
