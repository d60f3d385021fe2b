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
