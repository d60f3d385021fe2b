"""xsmi_conv2d_fwd_noalloc (the forward that takes no workspace and allocates nothing) against xsmi_conv2d_fwd,
through the C ABI.  It runs the kernels whose only scratch is the workspace, so with the even-split kernels switched
off (they exchange partial tiles through memory that xsmi_init allocated) the two entry points run the same kernels
and give the same bits; against the default selection the bar is the fp32 path's relative L2 error of 1e-5.  Two
calls in a row share the library's static scratch array; the second is smaller, so stale contents of the first must
not show."""
import ctypes

import numpy as np
import pytest

from xshinnosuke_amd.backend import capi
from util import he_normal, rel_l2

pytestmark = pytest.mark.gpu


def _forward_both(gpu, n, c, h, w, k, r, s, sh, sw, pad, relu, seed):
    rng = np.random.default_rng(seed)
    x = gpu.to_device(rng.standard_normal((n, c, h, w)).astype(np.float32))
    wt = gpu.to_device(he_normal(rng, (k, c, r, s)))
    b = gpu.to_device(rng.standard_normal((k,)).astype(np.float32))
    oh, ow = (h + 2 * pad - r) // sh + 1, (w + 2 * pad - s) // sw + 1
    dims = [n, c, h, w, k, r, s, sh, sw, pad]
    flags = capi.CONV_RELU if relu else 0
    y_ref, m_ref = gpu.empty((n, k, oh, ow)), gpu.empty((n, k, oh, ow), np.uint8)
    # a workspace of the static array's size: the library picks its kernels by the room it is given, and the same
    # kernels give the same bits
    ws = gpu.empty((capi.NOALLOC_SCRATCH_BYTES // 4,))
    y_def = gpu.empty((n, k, oh, ow))
    capi.lib.call("xsmi_conv2d_fwd", x.cptr, wt.cptr, b.cptr, y_def.cptr, m_ref.cptr if relu else None, *dims, flags,
                  ws.cptr, ws.nbytes)
    old = gpu.set_option("tap_sk", 0)
    try:
        capi.lib.call("xsmi_conv2d_fwd", x.cptr, wt.cptr, b.cptr, y_ref.cptr, m_ref.cptr if relu else None, *dims, flags,
                      ws.cptr, ws.nbytes)
    finally:
        gpu.set_option("tap_sk", old)
    y, m = gpu.empty((n, k, oh, ow)), gpu.empty((n, k, oh, ow), np.uint8)
    calls = []
    real = capi.lib.call
    capi.lib.call = lambda name, *a: (calls.append(name), real(name, *a))[1]
    try:
        capi.lib.call("xsmi_conv2d_fwd_noalloc", x.cptr, wt.cptr, b.cptr, y.cptr, m.cptr if relu else None, *dims, flags)
    finally:
        capi.lib.call = real
    assert calls == ["xsmi_conv2d_fwd_noalloc"]              # the binding itself allocated nothing either
    assert rel_l2(y.numpy(), y_def.numpy()) <= 1e-5
    return (y.numpy(), m.numpy() if relu else None), (y_ref.numpy(), m_ref.numpy() if relu else None)


def test_noalloc_forward_matches_the_workspace_forward_on_two_calls_in_a_row(gpu):
    # 1: the benchmark layer's geometry with fewer images (tap-major MFMA kernel, 147 KB of packed filter)
    (y, _), (y_ref, _) = _forward_both(gpu, 4, 64, 56, 56, 64, 3, 3, 1, 1, 1, False, 1)
    assert np.abs(y_ref).max() > 0 and y.tobytes() == y_ref.tobytes()
    # 2: smaller, another kernel (3 input channels: the table-driven one), fused ReLU + mask, stride 2
    (y, m), (y_ref, m_ref) = _forward_both(gpu, 2, 3, 17, 15, 10, 5, 3, 2, 2, 2, True, 2)
    assert np.abs(y_ref).max() > 0 and y.tobytes() == y_ref.tobytes() and m.tobytes() == m_ref.tobytes()
    # 3: and back to a tap-major geometry smaller than the first
    (y, m), (y_ref, m_ref) = _forward_both(gpu, 1, 32, 9, 9, 40, 3, 3, 1, 1, 1, True, 3)
    assert y.tobytes() == y_ref.tobytes() and m.tobytes() == m_ref.tobytes()


def test_noalloc_forward_refuses_what_does_not_fit(gpu):
    x = gpu.zeros((1, 1024, 4, 4)); w = gpu.zeros((1024, 1024, 3, 3)); y = gpu.zeros((1, 1024, 4, 4))
    dims = [1, 1024, 4, 4, 1024, 3, 3, 1, 1, 1]
    assert capi.lib.raw("xsmi_conv2d_workspace_bytes")(*dims) > capi.NOALLOC_SCRATCH_BYTES
    with pytest.raises(ValueError, match="static buffer"):
        capi.lib.call("xsmi_conv2d_fwd_noalloc", x.cptr, w.cptr, None, y.cptr, None, *dims, 0)
    with pytest.raises(ValueError, match="flags"):
        capi.lib.call("xsmi_conv2d_fwd_noalloc", x.cptr, w.cptr, None, y.cptr, None, *dims, capi.CONV_WS_PACKED)
