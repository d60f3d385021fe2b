"""Device-resident arrays owned by Python, allocated through the C ABI."""
import ctypes
import math
import weakref

import numpy as np

from .capi import lib, ensure_init, XsmiError, flush_deferred


_DTYPE_CLASS = np.dtype(np.float32).__class__

_POOL = {}            # rounded size -> list of free device pointers
_CL_POOL = {}         # (n, c, h, w, border) -> ChannelsLast forms of released arrays (their borders are zero)
_CL_POOL_DEPTH = 4
_POOL_BYTES = [0]
_POOL_LIMIT = 64 << 30
_CAPTURE = [None]     # the StepGraph whose step is being recorded (backend/graph.py), else None
_EPOCH = [0]          # moves whenever recorded work may have changed device memory behind Python's back
_REPLAYS = [0]          # step-graph replays so far: each may have changed parameters without Python taking their address


def _round_size(nbytes):
    nbytes = max(int(nbytes), 256)
    if nbytes <= (1 << 20):
        return (nbytes + 255) & ~255
    return (nbytes + (1 << 16) - 1) & ~((1 << 16) - 1)


def release_cached_memory():
    """Return every cached block to the driver."""
    _CL_POOL.clear()                      # their buffers return to _POOL first
    for ptrs in _POOL.values():
        for ptr in ptrs:
            lib.call("xsmi_free", ctypes.c_void_p(ptr))
    _POOL.clear()
    _POOL_BYTES[0] = 0


class _Block:
    """One device allocation shared by the views of an array.  Freed blocks are kept in a size-keyed
    pool and handed out again: a training step allocates the same sizes every iteration, all work
    runs in order on one stream, so reuse needs no synchronisation and avoids hipMalloc/hipFree
    (which serialise with the device) in the steady state."""

    __slots__ = ("ptr", "nbytes", "logical", "lazy_zero", "version", "cl", "owner", "unwritten", "__weakref__")

    def __init__(self, nbytes):
        ensure_init()
        self.logical = int(nbytes)
        self.lazy_zero = False
        self.unwritten = None                # why the contents were never produced (a message), see never_written()
        self.cl = None                       # ChannelsLast form of the array that fills this block, if it has one
        self.version = 0                     # counts every hand-out of the address and every pending clear
        size = _round_size(nbytes)
        # Memory handed out while a step is recorded belongs to that graph from then on: released blocks go to
        # the graph's own pool (later allocations of the same recording may take them, which a replay repeats
        # in the same order), never to code that runs between replays.
        graph = self.owner = _CAPTURE[0]
        free = graph._pool.get(size) if graph is not None else None
        if free:
            self.ptr = free.pop()
            self.nbytes = size
            return
        free = _POOL.get(size)
        if free:
            self.ptr = free.pop()
            _POOL_BYTES[0] -= size
        else:
            p = ctypes.c_void_p()
            try:
                lib.call("xsmi_malloc", ctypes.byref(p), size)
            except Exception:
                release_cached_memory()
                lib.call("xsmi_malloc", ctypes.byref(p), size)
            self.ptr = p.value
        self.nbytes = size

    def __reduce__(self):
        # a device address means nothing in another process; arrays pickle as host copies (DeviceArray.__reduce__)
        raise TypeError("a device memory block cannot be pickled")

    def __del__(self):
        try:
            cl = self.cl
            if cl is not None:               # keep the zero-bordered buffer for the next array of this geometry
                self.cl = None
                cl.valid = False
                if cl.buf._block.owner is None and _CAPTURE[0] is None:
                    kept = _CL_POOL.setdefault((cl.n, cl.c, cl.h, cl.w, cl.border), [])
                    if len(kept) < _CL_POOL_DEPTH:
                        kept.append(cl)
            if self.ptr:
                graph = self.owner
                if graph is not None and not graph._closed:
                    graph._pool.setdefault(self.nbytes, []).append(self.ptr)
                elif _POOL_BYTES[0] + self.nbytes <= _POOL_LIMIT:
                    _POOL.setdefault(self.nbytes, []).append(self.ptr)
                    _POOL_BYTES[0] += self.nbytes
                else:
                    lib.call("xsmi_free", ctypes.c_void_p(self.ptr))
                self.ptr = None
        except Exception:
            pass


class ChannelsLast:
    """A float32 NCHW array's contents held as bf16 [N][H + 2 border][W + 2 border][C] with a zero border (the operand
    layout of the bf16 convolution kernel; csrc/cl_ops.hip).  While ``valid`` the float32 memory of the owning
    block is stale: ``DeviceArray.ptr`` converts back before it hands the address out, so only the operations that
    ask for this form (conv, add + ReLU and max-pool without gradients under bf16 precision) ever see it."""

    __slots__ = ("buf", "n", "c", "h", "w", "border", "valid")

    def __init__(self, n, c, h, w, border):
        self.n, self.c, self.h, self.w, self.border = n, c, h, w, border
        # zeroed once: the kernels write the interior only, the border stays zero
        self.buf = DeviceArray((n, h + 2 * border, w + 2 * border, c), np.uint16).fill_zero()
        self.valid = False

    def same_layout(self, other):
        return (self.n, self.c, self.h, self.w, self.border) == (other.n, other.c, other.h, other.w, other.border)


def _rebuild_array(host):
    """Unpickling side of DeviceArray.__reduce__: back onto the device when one can be used, else the
    host array itself (tensors then simply live on the host).  Only "no library / no gfx950 device" selects
    the host: a failed allocation or copy is an error, not a reason to scatter a model over two places."""
    try:
        ensure_init()
    except (XsmiError, ValueError):              # library missing, no device, or device 0 out of range
        return host
    return to_device(host, host.dtype)


class DeviceArray:
    """Dense C-contiguous array in device memory (float32, uint8, int32 or int64).

    Only what the conv / pool path needs: shape/dtype bookkeeping, host copies,
    reshape, and slicing of the leading axis (the static graph re-slices its
    preallocated buffers to a shorter last batch).
    """

    def __init__(self, shape, dtype=np.float32, _block=None, _offset=0):
        self.shape = shape = tuple(map(int, shape))
        self.dtype = dtype if dtype.__class__ is _DTYPE_CLASS else np.dtype(dtype)
        self.size = math.prod(shape)
        self.nbytes = self.size * self.dtype.itemsize
        if _block is None:
            _block = _Block(max(self.nbytes, 16))
            _block.logical = self.nbytes
        self._block = _block
        self._offset = int(_offset)

    @property
    def ptr(self):
        blk = self._block
        if blk.unwritten is not None:
            raise XsmiError(blk.unwritten)
        blk.version += 1                     # whoever takes the address may write through it
        graph = _CAPTURE[0]
        if graph is not None and blk.owner is not graph:
            graph._refs[id(blk)] = blk       # recorded launches use this memory: it lives as long as the graph
        if blk.lazy_zero:                    # logically zero, memory not cleared yet: clear it on first use
            blk.lazy_zero = False
            lib.call("xsmi_memset", ctypes.c_void_p(blk.ptr), 0, blk.nbytes)
        cl = blk.cl
        if cl is not None and cl.valid:      # the contents live in channels-last form: convert back first
            cl.valid = False
            lib.call("xsmi_cl_to_nchw", cl.buf.cptr, cl.border, ctypes.c_void_p(blk.ptr), cl.n, cl.c, cl.h, cl.w)
        return blk.ptr + self._offset

    def state(self):
        """(allocation, version): equal to an earlier value exactly when the address has not been handed out (to a
        kernel, a copy, the host) and no clear was scheduled since, i.e. the contents cannot have changed.  Lets
        results derived from an array (a packed or folded filter) be kept for the next call."""
        return id(self._block), self._block.version

    def address(self):
        """The device address as an integer; unlike ``ptr`` it leaves a pending clear pending (for alignment and
        aliasing checks)."""
        return self._block.ptr + self._offset

    def channels_last(self):
        """The ChannelsLast form if that is where this array's contents currently live, else None (never converts)."""
        cl = self._block.cl
        if cl is not None and cl.valid and self._offset == 0 and self.shape == (cl.n, cl.c, cl.h, cl.w):
            return cl
        return None

    def channels_last_out(self, border=1):
        """Declare that this array (float32 NCHW, a whole allocation, channels a multiple of 8) is about to be
        produced in channels-last form: returns the ChannelsLast whose ``buf`` interior the producer writes, marked
        valid, or None if the array does not qualify.  A pending clear is dropped (everything is overwritten)."""
        blk = self._block
        if (len(self.shape) != 4 or self.dtype != np.float32 or self._offset != 0 or self.nbytes < blk.logical
                or self.shape[1] % 8 or self.size == 0):
            return None
        n, c, h, w = self.shape
        cl = blk.cl
        if cl is None or (cl.n, cl.c, cl.h, cl.w, cl.border) != (n, c, h, w, border):
            kept = _CL_POOL.get((n, c, h, w, border))
            cl = blk.cl = kept.pop() if kept else ChannelsLast(n, c, h, w, border)
        blk.lazy_zero = False
        blk.version += 1
        cl.valid = True
        return cl

    def _overwritten(self):
        """Called before the whole array is overwritten: a channels-last form need not be converted back, and contents
        that were never produced (never_written) no longer matter."""
        whole = self._offset == 0 and self.nbytes >= self._block.logical
        if whole:
            self._block.unwritten = None
        cl = self._block.cl
        if cl is not None and cl.valid and whole:
            cl.valid = False

    def is_fresh(self):
        """True if the array is a whole allocation whose clear is still pending."""
        blk = self._block
        return blk.lazy_zero and self._offset == 0 and self.nbytes >= blk.logical

    def is_whole(self):
        """True if the array fills its allocation (not a part of a larger buffer)."""
        return self._offset == 0 and self.nbytes >= self._block.logical

    def never_written(self, why):
        """Declare that the operation that was to produce this array (a whole allocation) ran fused into its consumer
        and stored nothing here: handing out the address raises ``why`` until the array is overwritten as a whole."""
        self._block.unwritten = str(why)
        self._block.version += 1

    def take_fresh(self):
        """True if this array is a pending all-zero buffer that the caller will now overwrite completely
        (the pending clear is dropped).  An array that covers only part of its allocation is cleared
        for real instead and reports False."""
        blk = self._block
        if self._offset == 0 and self.nbytes >= blk.logical:
            blk.unwritten = None
        if not blk.lazy_zero:
            return False
        if self._offset == 0 and self.nbytes >= blk.logical:
            blk.lazy_zero = False
            return True
        self.ptr                              # materialise the zeros
        return False

    def __reduce__(self):
        # checkpoints hold host arrays (reference xs/nn/models.py:188-202 pickles NumPy arrays)
        return _rebuild_array, (self.numpy(),)

    @property
    def cptr(self):
        return ctypes.c_void_p(self.ptr)

    @property
    def ndim(self):
        return len(self.shape)

    def numpy(self):
        if _CAPTURE[0] is not None:
            raise XsmiError("a device array cannot be read on the host while a step graph is being captured: "
                            "nothing recorded has run yet")
        out = np.empty(self.shape, dtype=self.dtype)
        if self.nbytes:
            lib.call("xsmi_memcpy_d2h", out.ctypes.data_as(ctypes.c_void_p), self.cptr, self.nbytes)
        return out

    def __array__(self, dtype=None, copy=None):
        a = self.numpy()
        return a if dtype is None else a.astype(dtype, copy=False)

    def set(self, host):
        if _CAPTURE[0] is not None:
            raise XsmiError("a blocking upload cannot be part of a step graph: fill the array before the capture, "
                            "or enqueue set_async from pinned memory")
        host = np.ascontiguousarray(host, dtype=self.dtype)
        if host.shape != self.shape:
            host = np.ascontiguousarray(np.broadcast_to(host, self.shape))
        self.take_fresh()                     # everything is overwritten: a pending clear is moot
        self._overwritten()
        if self.nbytes:
            lib.call("xsmi_memcpy_h2d", self.cptr, host.ctypes.data_as(ctypes.c_void_p), self.nbytes)
        return self

    def set_async(self, pinned, count=None):
        """Enqueue an upload of the first ``count`` leading rows (all by default) of a PinnedArray.  The
        caller keeps the pinned memory unchanged until an event recorded afterwards has completed."""
        rows = self.shape[0] if count is None else int(count)
        if pinned.dtype != self.dtype or pinned.shape[1:] != self.shape[1:] or rows > pinned.shape[0] or rows > self.shape[0]:
            raise ValueError("set_async: pinned %s %s does not fit device %s %s" % (pinned.shape, pinned.dtype, self.shape, self.dtype))
        nbytes = (self.nbytes // self.shape[0]) * rows if self.shape[0] else 0
        if rows == self.shape[0]:
            self.take_fresh()
        if nbytes:
            lib.call("xsmi_memcpy_h2d_async", self.cptr, ctypes.c_void_p(pinned._ptr), nbytes)
        return self

    def copy_from(self, other):
        if other.nbytes != self.nbytes:
            raise ValueError("size mismatch in device copy: %s vs %s" % (other.shape, self.shape))
        self.take_fresh()
        self._overwritten()
        if self.nbytes:
            lib.call("xsmi_memcpy_d2d", self.cptr, other.cptr, self.nbytes)
        return self

    def copy(self):
        return DeviceArray(self.shape, self.dtype).copy_from(self)

    def fill_zero(self, lazy=False):
        """Clear the array.  ``lazy=True`` only marks a whole allocation as zero: the memset happens on
        the first ordinary use, and not at all if the first use overwrites everything (take_fresh)."""
        blk = self._block
        flush_deferred(blk)                   # a held-back operation that uses this allocation comes first
        self._overwritten()
        if lazy and self._offset == 0 and self.nbytes >= blk.logical:
            blk.lazy_zero = True
            blk.version += 1
            return self
        if self.nbytes:
            lib.call("xsmi_memset", self.cptr, 0, self.nbytes)
        return self

    def reshape(self, *shape):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        shape = list(shape)
        if -1 in shape:
            known = math.prod(s for s in shape if s != -1)
            shape[shape.index(-1)] = self.size // max(known, 1)
        if math.prod(shape) != self.size:
            raise ValueError("cannot reshape %s into %s" % (self.shape, tuple(shape)))
        return DeviceArray(shape, self.dtype, _block=self._block, _offset=self._offset)

    def leading(self, start, stop):
        """View of rows [start, stop) of the leading axis."""
        n = self.shape[0]
        start = 0 if start is None else start
        stop = n if stop is None else min(stop, n)
        row = (self.size // n) * self.dtype.itemsize if n else 0
        return DeviceArray((stop - start,) + self.shape[1:], self.dtype, _block=self._block,
                           _offset=self._offset + start * row)

    def __getitem__(self, item):
        if isinstance(item, slice) and item.step in (None, 1):
            return self.leading(item.start, item.stop)
        raise TypeError("device arrays only support contiguous slices of the leading axis")

    def __repr__(self):
        return "DeviceArray(shape=%s, dtype=%s)" % (self.shape, self.dtype)


def empty(shape, dtype=np.float32):
    return DeviceArray(shape, dtype)


def zeros(shape, dtype=np.float32, lazy=False):
    return DeviceArray(shape, dtype).fill_zero(lazy)


def to_device(host, dtype=None):
    host = np.asarray(host)
    if dtype is None:
        dtype = np.float32 if host.dtype.kind == "f" else host.dtype
    return DeviceArray(host.shape, dtype).set(host)


class PinnedArray:
    """Page-locked host array (``.array`` is a NumPy view of it) for uploads that only enqueue on the
    stream.  The memory is returned when the object dies."""

    def __init__(self, shape, dtype=np.float32):
        ensure_init()
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = ctypes.c_void_p()
        lib.call("xsmi_host_alloc", ctypes.byref(p), max(self.nbytes, 16))
        self._ptr = p.value
        buf = (ctypes.c_char * max(self.nbytes, 1)).from_address(self._ptr)
        self.array = np.frombuffer(buf, dtype=self.dtype, count=self.nbytes // self.dtype.itemsize).reshape(self.shape)

    def __del__(self):
        try:
            if self._ptr:
                self.array = None
                lib.call("xsmi_host_free", ctypes.c_void_p(self._ptr))
                self._ptr = None
        except Exception:
            pass


_WORKSPACES = weakref.WeakSet()


def workspace_bytes():
    """Device bytes beside the tensors: all live workspaces (the shared ones and the per-filter layout workspaces)
    plus what the library holds itself (``xsmi_scratch_bytes``)."""
    ensure_init()
    return sum(w._block.nbytes for w in list(_WORKSPACES) if w._block is not None) + int(lib.raw("xsmi_scratch_bytes")())


class Workspace:
    """Grow-only scratch buffer handed to the conv entry points."""

    def __init__(self):
        self._block = None
        _WORKSPACES.add(self)

    def __reduce__(self):
        raise TypeError("a device workspace cannot be pickled")

    def address(self):
        """The present block's device address (0 before the first ``get``)."""
        return self._block.ptr if self._block is not None else 0

    def holds(self, nbytes):
        """True if ``get(nbytes)`` would hand out the present block (no reallocation)."""
        return self._block is not None and self._block.nbytes >= nbytes

    def get(self, nbytes):
        if self._block is None or self._block.nbytes < nbytes:
            self._block = None
            self._block = _Block(max(int(nbytes), 256))
        graph = _CAPTURE[0]
        if graph is not None and self._block.owner is not graph:
            graph._refs[id(self._block)] = self._block
        return ctypes.c_void_p(self._block.ptr), self._block.nbytes


class Event:
    def __init__(self):
        ensure_init()
        e = ctypes.c_void_p()
        lib.call("xsmi_event_create", ctypes.byref(e))
        self._e = e

    def record(self):
        lib.call("xsmi_event_record", self._e)
        return self

    def synchronize(self):
        lib.call("xsmi_event_synchronize", self._e)
        return self

    def elapsed_ms(self, stop):
        ms = ctypes.c_float()
        lib.call("xsmi_event_elapsed_ms", self._e, stop._e, ctypes.byref(ms))
        return ms.value

    def __del__(self):
        try:
            lib.call("xsmi_event_destroy", self._e)
        except Exception:
            pass
