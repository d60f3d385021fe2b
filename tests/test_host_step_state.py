"""Host-side bookkeeping behind step graphs and filter layouts made ahead, exercised without a GPU: the library is
replaced by a recorder that hands out made-up addresses, so only the Python logic runs (who owns a block of device
memory, which arrays a recording keeps alive, when a filter layout counts as current)."""
import ctypes
import gc

import pytest

from xshinnosuke_amd.backend import array as dev
from xshinnosuke_amd.backend import capi, kernels as K
from xshinnosuke_amd.backend.graph import StepGraph


class _Recorder:
    def __init__(self):
        self.calls = []
        self.next_address = 0x7000_0000_0000
        self.unpackable = set()          # passes whose jobs report "nothing to lay out ahead"

    def raw(self, name):
        if name == "xsmi_is_initialized":
            return lambda: 1
        if name == "xsmi_conv2d_workspace_bytes":
            return lambda *dims: 1 << 16
        if name == "xsmi_conv2d_pass_workspace_bytes":
            return lambda *dims_pass_flags: 1 << 12
        if name == "xsmi_last_error":
            return lambda: b""
        raise AssertionError(name)

    def call(self, name, *args):
        self.calls.append(name)
        if name == "xsmi_malloc":
            args[0]._obj.value = self.next_address
            self.next_address += 1 << 24
        elif name == "xsmi_graph_end":
            args[0]._obj.value = 0xBEEF if args[1] else None
        elif name == "xsmi_conv2d_pack":
            jobs = ctypes.cast(args[1], ctypes.POINTER(capi.PackJob))
            for i in range(args[0]):
                jobs[i].packed = 0 if jobs[i].pass_ in self.unpackable else 1


@pytest.fixture
def recorder(monkeypatch):
    rec = _Recorder()
    saved = (dict(dev._POOL), dev._POOL_BYTES[0], dict(dev._CL_POOL), dict(K._plan))
    dev._POOL.clear(); dev._POOL_BYTES[0] = 0; dev._CL_POOL.clear()
    monkeypatch.setattr(capi.lib, "call", rec.call)
    monkeypatch.setattr(capi.lib, "raw", rec.raw)
    monkeypatch.setattr(K, "_PREPACK", True)
    yield rec
    gc.collect()
    capi.drop_pending()
    K._LAYOUTS.clear()
    K._plan.update(saved[3])
    dev._POOL.clear(); dev._POOL.update(saved[0]); dev._POOL_BYTES[0] = saved[1]
    dev._CL_POOL.clear(); dev._CL_POOL.update(saved[2])


def _pooled():
    return sorted(p for ptrs in dev._POOL.values() for p in ptrs)


def test_memory_handed_out_while_recording_stays_with_the_graph(recorder):
    before = dev.empty((1024,))                       # exists before the recording
    graph = StepGraph()
    with graph.capture():
        a = dev.empty((1024,))
        a_ptr = a.address()
        before.ptr                                    # a recorded launch would use this array
        del a
        gc.collect()
        b = dev.empty((1024,))                        # same size: the recording reuses its own released block
        assert b.address() == a_ptr
        with pytest.raises(capi.XsmiError):
            b.numpy()                                 # nothing recorded has run
    assert recorder.calls.count("xsmi_graph_begin") == 1 and recorder.calls.count("xsmi_graph_end") == 1
    assert id(before._block) in graph._refs           # kept alive with the graph
    b_ptr = b.address()
    del b
    gc.collect()
    assert b_ptr not in _pooled()                     # eager code must never be handed the graph's memory
    c = dev.empty((1024,))
    assert c.address() != b_ptr
    graph.replay()
    assert recorder.calls[-1] == "xsmi_graph_launch" and graph.replays == 1
    graph.close()
    assert "xsmi_graph_destroy" in recorder.calls
    assert b_ptr in _pooled()                         # released with the graph
    with pytest.raises(capi.XsmiError):
        graph.replay()


def test_a_step_that_raises_closes_the_recording_and_keeps_nothing(recorder):
    graph = StepGraph()
    with pytest.raises(ZeroDivisionError):
        with graph.capture():
            dev.empty((256,))
            1 / 0
    assert dev._CAPTURE[0] is None
    assert recorder.calls[-1] == "xsmi_graph_end"
    with pytest.raises(capi.XsmiError):
        graph.replay()
    with pytest.raises(capi.XsmiError):
        with graph.capture():
            pass


def test_a_filter_layout_is_current_exactly_until_the_filter_address_is_handed_out(recorder):
    w = dev.empty((64, 64, 3, 3))
    dims = [32, 64, 56, 56, 64, 3, 3, 1, 1, 1]
    entry, current = K._layout_for(w, 0, dims)
    assert entry is not None and not current          # nothing has been laid out yet
    K.refresh_layouts([w])                            # what the optimizer step does after its update
    assert recorder.calls.count("xsmi_conv2d_pack") == 1 and capi._layouts_pending[0]
    again, current = K._layout_for(w, 0, dims)
    assert again is entry and current
    assert not capi._layouts_pending[0] and recorder.calls[-1] == "xsmi_conv2d_bwd_join"   # waited before the first use
    w.ptr                                             # someone may have written the filter
    _, current = K._layout_for(w, 0, dims)
    assert not current
    # another geometry of the same filter is a layout of its own
    other, current = K._layout_for(w, 0, [8] + dims[1:])
    assert other is not entry and not current


def test_refresh_reuses_its_job_table_and_drops_layouts_nobody_used(recorder):
    w1, w2 = dev.empty((64, 64, 3, 3)), dev.empty((128, 64, 3, 3))
    d1, d2 = [32, 64, 56, 56, 64, 3, 3, 1, 1, 1], [32, 64, 56, 56, 128, 3, 3, 2, 2, 1]
    recorder.unpackable.add(1)                        # backward-data jobs report nothing to prepare
    for step in range(3):
        K._layout_for(w1, 0, d1); K._layout_for(w2, 0, d2); K._layout_for(w2, 1, d2)
        K.refresh_layouts([w1, w2, dev.empty((64,))])
        if step == 0:
            table = K._plan["jobs"]
            assert len(table) == 3
        elif step == 1:
            assert len(K._plan["jobs"]) == 2          # the job that cannot be prepared ahead is not asked again
            table = K._plan["jobs"]
        else:
            assert K._plan["jobs"] is table           # same layouts as last time: same table
    assert K._layout_for(w2, 1, d2)[1] is False and K._layout_for(w2, 0, d2)[1] is True
    # a step that uses only w1: w2's layouts are dropped at the next refresh
    K.refresh_layouts([w1, w2])
    K._layout_for(w1, 0, d1)
    K.refresh_layouts([w1, w2])
    assert list(K._LAYOUTS[w1._block]) == [(0,) + tuple(d1)] and not K._LAYOUTS[w2._block]
    # the filter's memory goes away: so do its layouts (filters being laid out on the second stream are held until
    # the main stream has waited for it)
    blocks = len(K._LAYOUTS)
    del w1
    gc.collect()
    assert len(K._LAYOUTS) == blocks
    capi.join_side()
    gc.collect()
    assert len(K._LAYOUTS) == blocks - 1


def test_a_replay_after_an_eager_filter_update_lays_the_recorded_filters_out_again(recorder):
    """eager, eager, capture, replay, eager step on a short batch (other geometry), replay: the recording reads its
    filters in layouts made at the previous step's end, and the eager step in between changed the filter without
    renewing the full-batch layouts."""
    w = dev.empty((64, 64, 3, 3))
    full, short = [16, 64, 56, 56, 64, 3, 3, 1, 1, 1], [6, 64, 56, 56, 64, 3, 3, 1, 1, 1]

    def step(dims):
        entry, current = K._layout_for(w, 0, dims)    # what a training forward does
        w.ptr                                         # the optimizer step writes the filter
        K.refresh_layouts([w])
        return current

    assert step(full) is False                        # first step lays the filter out itself
    assert step(full) is True                         # second finds the layout made ahead
    graph = StepGraph()
    with graph.capture():
        assert step(full) is True                     # recorded as already laid out
    packs = recorder.calls.count("xsmi_conv2d_pack")
    graph.replay()
    graph.replay()
    assert recorder.calls.count("xsmi_conv2d_pack") == packs      # nothing touched the filter between replays
    # a replay changes the filter without Python seeing it: no layout made before it counts as current for eager code
    assert K._layout_for(w, 0, full)[1] is False
    assert step(short) is False                       # the eager step on the short last batch
    recorder.calls.clear()
    graph.replay()
    assert recorder.calls == ["xsmi_conv2d_pack", "xsmi_graph_launch"]          # laid out again, then launched
    jobs = ctypes.cast(graph._layout_jobs[0], ctypes.POINTER(capi.PackJob))
    assert graph._layout_jobs[1] == 1 and jobs[0].N == 16 and jobs[0].w == w.address()
    recorder.calls.clear()
    graph.replay()
    assert recorder.calls == ["xsmi_graph_launch"]
    graph.close()
