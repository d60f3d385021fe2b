"""ctypes binding of ``libxsmi355.so`` (declared in ``include/xsmi355.h``).

The library is the only compute path for conv / max-pool: if it is missing or
cannot initialise a gfx950 device, the ops raise -- there is no CPU fallback.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# XSMI355_LIBRARY lets a developer load another build of the same ABI; the default is the in-tree one
_LIB_PATH = os.environ.get("XSMI355_LIBRARY") or os.path.join(os.path.dirname(_HERE), "lib", "libxsmi355.so")


class XsmiError(RuntimeError):
    """A call into libxsmi355.so failed."""


class DeviceInfo(ctypes.Structure):
    _fields_ = [
        ("device", ctypes.c_int),
        ("cu_count", ctypes.c_int),
        ("clock_khz", ctypes.c_int),
        ("lds_bytes_per_cu", ctypes.c_int),
        ("wavefront", ctypes.c_int),
        ("l2_bytes", ctypes.c_int),
        ("hbm_bytes", ctypes.c_uint64),
        ("name", ctypes.c_char * 128),
        ("arch", ctypes.c_char * 64),
    ]


class PackJob(ctypes.Structure):
    """xsmi_pack_job_t"""
    _fields_ = [("w", ctypes.c_void_p), ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t)] + \
               [(n, ctypes.c_int) for n in ("N", "C", "H", "W", "K", "R", "S", "sh", "sw", "pad", "pass_", "packed")]


_c = ctypes
_vp, _i, _sz, _f, _u = _c.c_void_p, _c.c_int, _c.c_size_t, _c.c_float, _c.c_uint
_CONV_DIMS = [_i] * 10   # N C H W K R S sh sw pad

# name -> (restype, argtypes); must list every symbol include/xsmi355.h declares
SIGNATURES = {
    "xsmi_init": (_i, [_i]),
    "xsmi_is_initialized": (_i, []),
    "xsmi_last_error": (_c.c_char_p, []),
    "xsmi_device_info": (_i, [_c.POINTER(DeviceInfo)]),
    "xsmi_scratch_bytes": (_sz, []),
    "xsmi_malloc": (_i, [_c.POINTER(_vp), _sz]),
    "xsmi_free": (_i, [_vp]),
    "xsmi_memcpy_h2d": (_i, [_vp, _vp, _sz]),
    "xsmi_memcpy_d2h": (_i, [_vp, _vp, _sz]),
    "xsmi_host_alloc": (_i, [_c.POINTER(_vp), _sz]),
    "xsmi_host_free": (_i, [_vp]),
    "xsmi_memcpy_h2d_async": (_i, [_vp, _vp, _sz]),
    "xsmi_memcpy_d2d": (_i, [_vp, _vp, _sz]),
    "xsmi_memset": (_i, [_vp, _i, _sz]),
    "xsmi_sync": (_i, []),
    "xsmi_set_option": (_i, [_c.c_char_p, _c.c_long]),
    "xsmi_get_option": (_i, [_c.c_char_p, _c.POINTER(_c.c_long)]),
    "xsmi_event_create": (_i, [_c.POINTER(_vp)]),
    "xsmi_event_record": (_i, [_vp]),
    "xsmi_event_synchronize": (_i, [_vp]),
    "xsmi_event_elapsed_ms": (_i, [_vp, _vp, _c.POINTER(_f)]),
    "xsmi_event_destroy": (_i, [_vp]),
    "xsmi_profiling": (_i, [_i]),
    "xsmi_last_kernel_ms": (_i, [_c.POINTER(_f)]),
    "xsmi_copy_kernel": (_i, [_vp, _vp, _sz]),
    "xsmi_conv2d_workspace_bytes": (_sz, _CONV_DIMS),
    "xsmi_conv2d_pass_workspace_bytes": (_sz, _CONV_DIMS + [_i, _u]),
    "xsmi_conv2d_fwd": (_i, [_vp, _vp, _vp, _vp, _vp] + _CONV_DIMS + [_u, _vp, _sz]),
    "xsmi_conv2d_fwd_noalloc": (_i, [_vp, _vp, _vp, _vp, _vp] + _CONV_DIMS + [_u]),
    "xsmi_conv2d_bwd_data": (_i, [_vp, _vp, _vp] + _CONV_DIMS + [_f, _u, _vp, _sz]),
    "xsmi_conv2d_bwd_weight": (_i, [_vp, _vp, _vp, _vp] + _CONV_DIMS + [_f, _u, _vp, _sz]),
    "xsmi_conv2d_bwd": (_i, [_vp] * 6 + _CONV_DIMS + [_f, _f, _u, _vp, _sz, _vp, _sz]),
    "xsmi_conv2d_bwd_join": (_i, []),
    "xsmi_conv2d_pack": (_i, [_i, _vp]),
    "xsmi_maxpool2d_fwd": (_i, [_vp, _vp, _vp] + [_i] * 8),
    "xsmi_maxpool2d_bwd": (_i, [_vp, _vp, _vp] + [_i] * 8 + [_f]),
    "xsmi_relu_mask_bwd": (_i, [_vp, _vp, _vp, _sz, _f]),
    "xsmi_relu_mask_bwd2": (_i, [_vp, _vp, _vp, _f, _vp, _f, _sz]),
    "xsmi_axpy": (_i, [_vp, _vp, _f, _sz]),
    "xsmi_axpy_multi": (_i, [_i, _c.POINTER(_vp), _c.POINTER(_vp), _c.POINTER(_sz), _f]),
    "xsmi_add": (_i, [_vp, _vp, _vp, _sz]),
    "xsmi_add_relu": (_i, [_vp, _vp, _vp, _vp, _sz]),
    "xsmi_scale_shift": (_i, [_vp, _vp, _f, _f, _sz]),
    "xsmi_relu_fwd": (_i, [_vp, _vp, _sz]),
    "xsmi_relu_fwd_mask": (_i, [_vp, _vp, _vp, _sz]),
    "xsmi_relu_bwd": (_i, [_vp, _vp, _vp, _sz]),
    "xsmi_conv2d_fwd_cl": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _i] + [_i] * 10 + [_u, _vp, _sz]),
    "xsmi_cl_add": (_i, [_vp, _vp, _vp, _sz, _i]),
    "xsmi_cl_maxpool2d": (_i, [_vp, _i, _vp, _i] + [_i] * 8),
    "xsmi_cl_to_nchw": (_i, [_vp, _i, _vp] + [_i] * 4),
    "xsmi_act_fwd": (_i, [_vp, _vp, _sz, _i]),
    "xsmi_act_bwd": (_i, [_vp, _vp, _vp, _sz, _i]),
    "xsmi_lerp": (_i, [_vp, _vp, _f, _sz]),
    "xsmi_bn_workspace_bytes": (_sz, [_i]),
    "xsmi_bn_fwd": (_i, [_vp] * 10 + [_f, _vp, _i, _i, _i, _f, _vp, _sz]),
    "xsmi_bn_add_relu_fwd": (_i, [_vp] * 10 + [_f, _vp, _i, _i, _i, _f, _vp, _sz]),
    "xsmi_bn_relu_maxpool_fwd": (_i, [_vp] * 11 + [_f, _i, _i, _i, _i, _f, _vp, _sz]),
    "xsmi_bn_bwd_maxpool": (_i, [_vp] * 10 + [_i, _i, _i, _i, _vp, _sz]),
    "xsmi_bn_infer": (_i, [_vp] * 6 + [_i, _i, _i, _f, _i]),
    "xsmi_bn_fold": (_i, [_vp] * 8 + [_i, _i, _f]),
    "xsmi_bn_bwd": (_i, [_vp] * 9 + [_i, _i, _i, _vp, _sz]),
    "xsmi_avgpool_fwd": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _i]),
    "xsmi_avgpool_bwd": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _i]),
    "xsmi_gemm": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _sz]),
    "xsmi_colsum": (_i, [_vp, _vp, _i, _i]),
    "xsmi_sum_all": (_i, [_vp, _vp, _sz]),
    "xsmi_softmax_ce_fwd": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "xsmi_softmax_ce_bwd": (_i, [_vp, _vp, _vp, _vp, _i, _i, _f]),
    "xsmi_fill": (_i, [_vp, _f, _sz]),
    "xsmi_graph_begin": (_i, []),
    "xsmi_graph_end": (_i, [_c.POINTER(_vp), _i]),
    "xsmi_graph_launch": (_i, [_vp]),
    "xsmi_graph_destroy": (_i, [_vp]),
}

CONV_RELU = 0x1
CONV_BF16 = 0x2
CONV_WS_PACKED = 0x4
CONV_DW_ASYNC = 0x8
NOALLOC_SCRATCH_BYTES = 16 << 20      # XSMI_NOALLOC_SCRATCH_BYTES of the header


def library_path():
    return _LIB_PATH


class _Lib:
    """Lazy handle: the shared object is opened on first use."""

    def __init__(self):
        self._dll = None

    def _open(self):
        if self._dll is not None:
            return self._dll
        if not os.path.exists(_LIB_PATH):
            raise XsmiError(
                "libxsmi355.so is not built (%s is missing); run "
                "`make -C xshinnosuke_amd/csrc` or __graft_entry__.build()" % _LIB_PATH)
        dll = ctypes.CDLL(_LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(dll, name)          # AttributeError if the export is missing
            fn.restype = res
            fn.argtypes = args
        self._dll = dll
        return dll

    def raw(self, name):
        """The bare ctypes function of a query that enqueues nothing and touches no device memory.  Everything
        else must go through ``call``, which is where a held-back add is enqueued and the second stream joined."""
        if name not in _QUERIES:
            raise XsmiError("%s launches work: call it through lib.call" % name)
        return getattr(self._open(), name)

    def call(self, name, *args):
        """Call an int-returning entry point; raise with the library's message on failure."""
        if _deferred:
            _flush_deferred()
        if _side_hold and name not in _SIDE_SAFE:
            join_side()
        dll = self._open()
        rc = getattr(dll, name)(*args)
        if rc != 0:
            msg = dll.xsmi_last_error().decode("utf-8", "replace")
            if rc == 1:
                raise ValueError(msg)
            raise XsmiError(msg)


_QUERIES = frozenset(("xsmi_scratch_bytes", "xsmi_conv2d_workspace_bytes", "xsmi_conv2d_pass_workspace_bytes", "xsmi_bn_workspace_bytes", "xsmi_is_initialized", "xsmi_last_error"))

lib = _Lib()

# Weight gradients that xsmi_conv2d_bwd left on the library's second stream (XSMI_CONV_DW_ASYNC).  The arrays they
# read and write are kept alive here, so their memory cannot be handed out again, and every call into the library
# joins the second stream first unless it is one of the passes of a backward sweep listed below: those write
# activation gradients only, never a filter gradient, a forward activation or an upstream gradient already consumed.
_side_hold = []
_SIDE_SAFE = frozenset(("xsmi_conv2d_bwd", "xsmi_bn_bwd", "xsmi_relu_mask_bwd", "xsmi_relu_mask_bwd2", "xsmi_relu_bwd",
                        "xsmi_maxpool2d_bwd", "xsmi_avgpool_bwd", "xsmi_conv2d_bwd_join"))


def hold_side(*arrays):
    _side_hold.append(arrays)


def side_pending():
    return bool(_side_hold)


def join_side():
    """The main stream waits for the second stream (weight gradients, filter layouts made ahead); the operands
    held for it are released."""
    if _side_hold or _layouts_pending[0]:
        try:
            lib.call("xsmi_conv2d_bwd_join")
        finally:
            del _side_hold[:]
            del _layouts_hold[:]
            _layouts_pending[0] = False


# Filter layouts that xsmi_conv2d_pack put on the second stream (kernels.refresh_layouts).  Unlike a weight
# gradient they do not force the next call into the library to join: only a convolution that is about to read
# one of those workspaces does (kernels._layout_for), so that the layouts run beside whatever comes first.
_layouts_pending = [False]
_layouts_hold = []          # the filters being read and the workspaces being written there stay allocated until the join


def layouts_enqueued(*held):
    _layouts_pending[0] = True
    _layouts_hold.extend(held)


# One operation may be held back until the next call into the library, so that the end of a residual block runs as
# few passes as it needs (kernels.bn_fwd / kernels.add / kernels.relu_fwd):
#   ("add", a, b, out)            an element-wise add into a new array; if the next call is the in-place ReLU of its
#                                 result, both run as one pass;
#   ("bn", entry)                 a training batch normalisation (kernels.BnEntry: operands, outputs, launch); with a
#                                 ReLU of its own, if the next call is the 3x3/2 max-pool of its result, both run as one
#                                 normalisation whose second pass pools; without one, if the
#                                 next call is a held-back add with its result as one operand, it becomes
#   ("bn_add", entry, a, b, out)  and if the call after that is the in-place ReLU (with mask) of the sum, the three run
#                                 as one normalisation whose second pass adds the other operand and clips.
#   ("pool_bwd", entry)           the gradient of a 3x3/2 max-pool into a fresh buffer (kernels.PoolBwdEntry); if the
#                                 next call is the backward of the normalisation that fed the pool, the routed gradient
#                                 is formed inside that backward's two passes instead of being stored.
# Every other call enqueues what is held back first, in order, so nothing can read or change the operands or the
# results between an operation and the point where it was asked for.
_deferred = []          # at most one entry


def _flush_deferred():
    op = _deferred.pop()
    if op[0] == "add":
        _, a, b, out = op
        lib.call("xsmi_add", a.cptr, b.cptr, out.cptr, a.size)
    elif op[0] in ("bn", "pool_bwd"):
        op[1].launch()
    else:
        _, entry, a, b, out = op
        entry.launch()
        lib.call("xsmi_add", a.cptr, b.cptr, out.cptr, a.size)


def _deferred_arrays():
    op = _deferred[0]
    if op[0] == "add":
        return op[1:]
    arrays = list(op[1].arrays())
    if op[0] == "bn_add":
        arrays.extend(op[2:])
    return arrays


def flush_deferred(block=None):
    """Enqueue what is held back, if anything (with ``block``: only if it uses that allocation).  For changes of an
    array's state that make no call into the library (a clear that is only noted): a held-back operation may still
    have to read the array as it was, or to write it first."""
    if _deferred and (block is None or any(a is not None and a._block is block for a in _deferred_arrays())):
        _flush_deferred()


def defer_add(a, b, out):
    if _deferred:
        _flush_deferred()
    _deferred.append(("add", a, b, out))


def defer_bn(entry):
    if _deferred:
        _flush_deferred()
    _deferred.append(("bn", entry))


def take_deferred_bn(a, b):
    """The held-back normalisation whose result is ``a`` or ``b`` (it is no longer pending: the caller launches it or
    holds it back again), or None (anything else that was pending is enqueued)."""
    if not _deferred:
        return None
    if _deferred[0][0] == "bn" and (_deferred[0][1].y is a or _deferred[0][1].y is b):
        return _deferred.pop()[1]
    _flush_deferred()
    return None


def defer_pool_bwd(entry):
    if _deferred:
        _flush_deferred()
    _deferred.append(("pool_bwd", entry))


def take_deferred_pool_bwd(dx):
    """The held-back max-pool gradient whose result is ``dx`` (no longer pending), or None (anything else that was
    pending is enqueued)."""
    if not _deferred:
        return None
    if _deferred[0][0] == "pool_bwd" and _deferred[0][1].dx is dx:
        return _deferred.pop()[1]
    _flush_deferred()
    return None


def defer_bn_add(entry, a, b, out):
    if _deferred:
        _flush_deferred()
    _deferred.append(("bn_add", entry, a, b, out))


def take_deferred_add(out, with_bn=False):
    """The operands ``(a, b)`` of the held-back add whose result is ``out``, or None (a different pending operation is
    enqueued).  ``with_bn``: a held-back normalisation + add is handed over too, as ``(a, b, entry)``; without it that
    pair is enqueued as two launches and reported as None."""
    if not _deferred:
        return None
    op = _deferred[0]
    if op[0] == "add" and op[3] is out:
        _deferred.pop()
        return op[1], op[2]
    if op[0] == "bn_add" and op[4] is out and with_bn:
        _deferred.pop()
        return op[2], op[3], op[1]
    _flush_deferred()
    return None


def drop_pending():
    """Forget a held-back add and the arrays kept for the second stream (a recording that is being discarded)."""
    del _deferred[:]
    del _side_hold[:]
    del _layouts_hold[:]
    _layouts_pending[0] = False


def init(device=0):
    lib.call("xsmi_init", int(device))


def is_initialized():
    return bool(lib.raw("xsmi_is_initialized")())


def ensure_init():
    if not is_initialized():
        init(0)


def device_info():
    ensure_init()
    info = DeviceInfo()
    lib.call("xsmi_device_info", ctypes.byref(info))
    return {
        "device": info.device, "cu_count": info.cu_count, "clock_khz": info.clock_khz,
        "lds_bytes_per_cu": info.lds_bytes_per_cu, "wavefront": info.wavefront,
        "l2_bytes": info.l2_bytes, "hbm_bytes": int(info.hbm_bytes),
        "name": info.name.decode(), "arch": info.arch.decode(),
    }


def profiling(on):
    ensure_init()
    lib.call("xsmi_profiling", 1 if on else 0)


def last_kernel_ms():
    ms = ctypes.c_float()
    lib.call("xsmi_last_kernel_ms", ctypes.byref(ms))
    return ms.value


def synchronize():
    try:
        lib.call("xsmi_sync")              # joins the second stream and waits for both
    finally:
        del _side_hold[:]
        del _layouts_hold[:]
        _layouts_pending[0] = False


# Kernel-selection switches of the library ("tap_sk", "sk_spin_limit", "tap_persist", ...).  What the host keeps
# that depends on them (workspace sizes, filter layouts made ahead) is dropped by the listeners.
_option_listeners = []


def set_option(name, value):
    """Set a tuning switch of the library; returns the previous value."""
    old = get_option(name)
    synchronize()
    lib.call("xsmi_set_option", name.encode(), int(value))
    for fn in _option_listeners:
        fn()
    return old


def get_option(name):
    v = ctypes.c_long()
    lib.call("xsmi_get_option", name.encode(), ctypes.byref(v))
    return v.value
