"""Step graphs: one training or inference step recorded once and re-issued with a single call.

The host needs several microseconds of Python and ctypes per launch, and a ResNet-18 training step is more than
two hundred launches: issuing it takes the host about as long as running it takes the device.  A step whose
launches do not change between iterations (static shapes, the same tensors) can instead be recorded through
``xsmi_graph_begin`` / ``xsmi_graph_end`` and replayed with ``xsmi_graph_launch``:

    graph = StepGraph()
    with graph.capture():
        loss = step()          # ordinary code: zero_grad, forward, loss, backward, optimizer step
    for _ in range(n):
        x.eval.set_async(next_batch)   # new contents into the SAME device arrays the step read
        graph.replay()
        print(loss.item())             # the tensors made while recording now hold this replay's results

What the recording freezes, and what the caller therefore has to keep true:
  * nothing runs while recording: the recorded step has not happened when ``capture`` exits, and reading a
    device array on the host inside the block raises;
  * every decision Python took while recording (which kernel, overwrite or accumulate, learning rate and other
    scalars, shapes) is part of the graph; state that only Python advances (an optimizer's iteration counter)
    does not move on a replay;
  * device memory handed out while recording stays with the graph, and arrays that existed before and were
    used inside stay alive with it, until ``close()``;
  * a recorded training step reads its convolution filters in the layouts that the previous step's end left in
    per-filter workspaces, and renews them at its own end.  Code that changes a filter between two replays (an
    eager step on a short last batch, a loaded checkpoint, a host write) would leave them stale: ``replay`` notices
    that a filter's address has been handed out since and lays the filters out again before it launches.
"""
import contextlib
import ctypes

from . import array as _array
from . import capi as _capi
from .capi import lib, XsmiError


class StepGraph:
    def __init__(self):
        self._exec = None
        self._pool = {}           # rounded size -> free device pointers that belong to this graph
        self._refs = {}           # id -> pre-existing block that recorded launches read or write
        self._closed = False
        self.replays = 0
        self._layout_jobs = None  # (job table, count, filters) of the layouts the recording reads as already made
        self._filter_states = None

    @contextlib.contextmanager
    def capture(self):
        if self._exec is not None or self._closed:
            raise XsmiError("this step graph has already been captured")
        if _array._CAPTURE[0] is not None:
            raise XsmiError("another step graph is being captured")
        _capi.ensure_init()
        # channels-last buffers waiting for reuse carry contents eager code made; the recording makes its own
        _array._CL_POOL.clear()
        _array._EPOCH[0] += 1
        lib.call("xsmi_graph_begin")         # (enqueues a held-back add and joins the second stream first)
        _array._CAPTURE[0] = self
        keep = False
        try:
            yield self
            keep = True
        finally:
            handle = ctypes.c_void_p()
            try:
                if keep:
                    lib.call("xsmi_graph_end", ctypes.byref(handle), 1)
                else:                        # the step raised: close the recording, keep the step's own error
                    _capi.drop_pending()
                    try:
                        lib.call("xsmi_graph_end", ctypes.byref(handle), 0)
                    except Exception:
                        pass
            finally:
                _array._CAPTURE[0] = None
                _array._CL_POOL.clear()      # none of this graph's buffers may reach eager code
                _array._EPOCH[0] += 1
            self._exec = handle if handle.value else None
            if self._exec is None:
                self.close()
            elif self._layout_jobs is not None:
                self._filter_states = [v.state() for v in self._layout_jobs[2]]

    def note_layout_jobs(self, jobs, count, filters):
        """Called by the filter-layout bookkeeping while this graph records: the layouts made at the recorded step's
        end are the ones its next replay starts from."""
        self._layout_jobs = (jobs, count, list(filters))

    def replay(self):
        if self._exec is None:
            raise XsmiError("this step graph holds no recording")
        if self._layout_jobs is not None:
            jobs, count, filters = self._layout_jobs
            if [v.state() for v in filters] != self._filter_states:
                # a filter was touched outside the graph since the layouts were made: make them again (second
                # stream; the launch below waits for it)
                lib.call("xsmi_conv2d_pack", count, ctypes.cast(jobs, ctypes.c_void_p))
        lib.call("xsmi_graph_launch", self._exec)
        _array._EPOCH[0] += 1                # parameters may have changed without Python taking their address
        _array._REPLAYS[0] += 1
        self.replays += 1
        if self._layout_jobs is not None:
            self._filter_states = [v.state() for v in self._layout_jobs[2]]

    def close(self):
        """Release the executable graph and return the graph's memory to the common pool."""
        if self._closed:
            return
        self._closed = True
        if self._exec is not None:
            lib.call("xsmi_graph_destroy", self._exec)
            self._exec = None
        for size, ptrs in self._pool.items():
            for ptr in ptrs:
                _array._POOL.setdefault(size, []).append(ptr)
                _array._POOL_BYTES[0] += size
        self._pool.clear()
        self._refs.clear()
        self._layout_jobs = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
