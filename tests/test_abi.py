"""CPU-side checks of the C-ABI library: it loads and exports what include/xsmi355.h declares."""
import ctypes
import os
import re

import pytest

from xshinnosuke_amd.backend import capi as libmod

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "xsmi355.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(xsmi_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_bound_and_exported():
    declared = _declared_symbols()
    assert len(declared) >= 20
    assert sorted(libmod.SIGNATURES) == declared          # the Python binding covers the whole header
    dll = ctypes.CDLL(libmod.library_path())
    for name in declared:
        assert hasattr(dll, name), name


def test_calls_before_init_fail_with_a_message():
    dll = ctypes.CDLL(libmod.library_path())
    dll.xsmi_last_error.restype = ctypes.c_char_p
    dll.xsmi_is_initialized.restype = ctypes.c_int
    if dll.xsmi_is_initialized():
        pytest.skip("library already initialised in this process")
    assert dll.xsmi_sync() == 3
    assert b"xsmi_init" in dll.xsmi_last_error()


def test_workspace_query_needs_no_device():
    f = libmod.lib.raw("xsmi_conv2d_workspace_bytes")
    c2 = f(32, 64, 56, 56, 64, 3, 3, 1, 1, 1)
    assert c2 >= 64 * 576 * 4
    assert f(32, 64, 56, 56, 64, 3, 3, 0, 1, 1) == 0      # invalid stride -> 0
    assert f(1, 1, 2, 2, 1, 5, 5, 1, 1, 0) == 0           # filter larger than the input -> 0


def test_per_pass_workspace_queries_need_no_device():
    """The size of one pass alone never exceeds the size for all passes, the maximum over passes and flags is that
    size, a pass outside 0..2 and a bad geometry give 0; what the library holds itself is a constant."""
    whole = libmod.lib.raw("xsmi_conv2d_workspace_bytes")
    one = libmod.lib.raw("xsmi_conv2d_pass_workspace_bytes")
    for dims in ((32, 64, 56, 56, 64, 3, 3, 1, 1, 1), (32, 64, 56, 56, 128, 3, 3, 2, 2, 1), (32, 3, 224, 224, 64, 7, 7, 2, 2, 3),
                 (2, 5, 9, 11, 70, 3, 2, 1, 2, 2), (32, 512, 7, 7, 512, 3, 3, 1, 1, 1)):
        sizes = [one(*dims, p, f) for p in range(3) for f in (0, libmod.CONV_BF16)]
        assert all(0 < v <= whole(*dims) for v in sizes), dims
        assert max(sizes) == whole(*dims), dims
        assert one(*dims, 3, 0) == 0 and one(*dims, -1, 0) == 0
    # a layout workspace of the benchmark layer is the packed filter, not the split partials of the weight gradient
    c2 = (32, 64, 56, 56, 64, 3, 3, 1, 1, 1)
    assert one(*c2, 0, 0) < 1 << 20 and one(*c2, 1, 0) < 1 << 20 and one(*c2, 2, 0) > 8 << 20
    assert one(32, 64, 56, 56, 64, 3, 3, 0, 1, 1, 0, 0) == 0
    assert libmod.lib.raw("xsmi_scratch_bytes")() >= libmod.NOALLOC_SCRATCH_BYTES
