"""Channels-last bf16 activations (inference chains under bf16 precision).

The channels-last entry points run the same bf16 MFMA kernel as the plain bf16 forward and differ only in where the
activations live (bf16 [N][H+2b][W+2b][C] instead of float32 NCHW), so every check here is exact: the float32 form
of a channels-last result must equal the plain path's result rounded to bf16 (round to nearest even), and a chain
fed with bf16-representable values must reproduce the plain path bit for bit.  The plain bf16 path itself is
checked against the oracle in test_gpu_conv.py; the max-pool is checked against the oracle here.
"""
import numpy as np
import pytest

import oracle            # the CPU checker

pytestmark = pytest.mark.gpu


def bf16_round(a):
    """float32 -> nearest bf16 (ties to even) -> float32."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u >> 16) & 1) + 0x7FFF
    return ((u + r) & 0xFFFF0000).astype(np.uint32).view(np.float32).reshape(np.shape(a))


def _inputs(rng, n, c, h, k, r):
    x = rng.standard_normal((n, c, h, h)).astype(np.float32)
    w = (rng.standard_normal((k, c, r, r)) * np.sqrt(2.0 / (c * r * r))).astype(np.float32)
    b = rng.standard_normal(k).astype(np.float32)
    return x, w, b


@pytest.mark.parametrize("n,c,h,k,r,stride,pad,relu", [
    (2, 64, 12, 64, 3, 1, 1, True),          # 64-row tiles
    (3, 32, 9, 128, 3, 2, 1, False),         # 128-row tiles, stride 2, ragged pixel tile
    (2, 3, 20, 64, 7, 2, 3, True),           # a stem: float32 input only, channels-last output
    (2, 64, 8, 72, 1, 1, 0, False),          # 1x1, K a multiple of 8 but not of 64
    (2, 96, 30, 200, 3, 1, 1, True),         # input staged once for nine taps: three channel groups, two row tiles (one partial)
    (3, 64, 14, 64, 3, 1, 1, False),         # ... on the smallest feature map that takes that kernel, 64-row tiles
    (1, 32, 61, 64, 3, 1, 1, True),          # ... at its widest row (63 bordered pixels) ...
    (1, 32, 62, 64, 3, 1, 1, True),          # ... and one pixel wider: the tap-major kernel serves it
    (3, 3, 37, 32, 7, 2, 3, False),          # first-layer kernel: odd output height (a last item of one row), 32 filters
    (1, 1, 224, 64, 7, 2, 3, True),          # ... one channel, the full 112-column row
    (2, 4, 30, 8, 7, 2, 3, True),            # ... four channels, eight filters
    (1, 3, 300, 16, 3, 1, 1, False),         # rows of 300 pixels: converted back to float32 in two segments
    (1, 32, 256, 8, 1, 1, 0, True),          # ... 256 pixels, one more than a segment holds
])
def test_channels_last_output_is_the_plain_result_rounded_to_bf16(gpu, n, c, h, k, r, stride, pad, relu):
    K = gpu.kernels
    x, w, b = _inputs(np.random.default_rng(n * 100 + c + k + r), n, c, h, k, r)
    dx, dw, db = gpu.to_device(x), gpu.to_device(w), gpu.to_device(b)
    plain = K.conv2d_fwd(dx, dw, db, (stride, stride), pad, relu=relu, bf16=True).numpy()
    y = K.conv2d_fwd(dx, dw, db, (stride, stride), pad, relu=relu, bf16=True, channels_last=True)
    assert y.channels_last() is not None                       # it does live in channels-last form
    got = y.numpy()                                            # converts back
    assert y.channels_last() is None
    np.testing.assert_array_equal(got, bf16_round(plain))
    np.testing.assert_array_equal(y.numpy(), got)              # and the float32 memory now holds it


@pytest.mark.parametrize("stride2,r2,pad2", [(1, 3, 1), (2, 3, 1), (2, 1, 0), (1, 1, 0)])
def test_channels_last_chain_equals_the_plain_path(gpu, stride2, r2, pad2):
    """conv -> conv with the activation never leaving channels-last form; the second conv also covers a border wider
    than its padding (1x1, pad 0 on a border of 1)."""
    K = gpu.kernels
    rng = np.random.default_rng(7 + stride2 * 10 + r2)
    x, w1, b1 = _inputs(rng, 2, 32, 14, 64, 3)
    _, w2, b2 = _inputs(rng, 2, 64, 14, 128, r2)
    dx = gpu.to_device(x)
    mid = K.conv2d_fwd(dx, gpu.to_device(w1), gpu.to_device(b1), (1, 1), 1, relu=True, bf16=True, channels_last=True)
    out = K.conv2d_fwd(mid, gpu.to_device(w2), gpu.to_device(b2), (stride2, stride2), pad2, bf16=True, channels_last=True)
    assert mid.channels_last() is not None and out.channels_last() is not None      # nothing was converted back
    got = out.numpy()
    mid_plain = bf16_round(K.conv2d_fwd(dx, gpu.to_device(w1), gpu.to_device(b1), (1, 1), 1, relu=True, bf16=True).numpy())
    ref = K.conv2d_fwd(gpu.to_device(mid_plain), gpu.to_device(w2), gpu.to_device(b2), (stride2, stride2), pad2, bf16=True).numpy()
    np.testing.assert_array_equal(got, bf16_round(ref))
    np.testing.assert_array_equal(mid.numpy(), mid_plain)


def test_channels_last_add_relu_and_max_pool(gpu):
    K = gpu.kernels
    rng = np.random.default_rng(21)
    x, w1, b1 = _inputs(rng, 3, 32, 13, 64, 3)
    _, w2, b2 = _inputs(rng, 3, 32, 13, 64, 1)
    dx = gpu.to_device(x)
    a = K.conv2d_fwd(dx, gpu.to_device(w1), gpu.to_device(b1), (1, 1), 1, bf16=True, channels_last=True)
    b = K.conv2d_fwd(dx, gpu.to_device(w2), gpu.to_device(b2), (1, 1), 0, bf16=True, channels_last=True)
    s = K.add(a, b, defer=True)
    s = K.relu_fwd(s, out=s)                                   # the held-back add joins the in-place ReLU
    assert s.channels_last() is not None and a.channels_last() is not None
    p, idx = K.maxpool2d_fwd(s, 3, (2, 2), 1, want_idx=False)
    assert idx is None and p.channels_last() is not None
    an, bn = a.numpy(), b.numpy()
    s_ref = bf16_round(np.maximum(an + bn, np.float32(0)))
    np.testing.assert_array_equal(s.numpy(), s_ref)
    np.testing.assert_array_equal(p.numpy(), oracle.max_pool2d_fwd(s_ref, 3, (2, 2), 1)[0])
    # a window without padding on the same tensor, and one whose padding the border does not cover (falls back)
    q, _ = K.maxpool2d_fwd(gpu.to_device(s_ref), 2, (2, 2), 0, want_idx=False)
    np.testing.assert_array_equal(q.numpy(), oracle.max_pool2d_fwd(s_ref, 2, (2, 2), 0)[0])
    s2 = K.conv2d_fwd(dx, gpu.to_device(w1), gpu.to_device(b1), (1, 1), 1, bf16=True, channels_last=True)
    r2, _ = K.maxpool2d_fwd(s2, 5, (2, 2), 2, want_idx=False)
    np.testing.assert_array_equal(r2.numpy(), oracle.max_pool2d_fwd(an, 5, (2, 2), 2)[0])


def test_negative_inputs_meet_the_zero_padding_in_the_channels_last_max_pool(gpu):
    """The reference's padding is zero-valued and takes part in the max (xs/nn/functional.py:445-491): an all-negative
    window at the edge yields 0, inside the image the (negative) maximum."""
    K = gpu.kernels
    rng = np.random.default_rng(5)
    x, w, b = _inputs(rng, 2, 32, 10, 64, 3)
    y = K.conv2d_fwd(gpu.to_device(x), gpu.to_device(w), gpu.to_device(b - 50.0), (1, 1), 1, bf16=True, channels_last=True)
    p, _ = K.maxpool2d_fwd(y, 3, (2, 2), 1, want_idx=False)
    assert p.channels_last() is not None
    yn = y.numpy()
    assert yn.max() < 0
    np.testing.assert_array_equal(p.numpy(), oracle.max_pool2d_fwd(yn, 3, (2, 2), 1)[0])


def test_consumers_that_do_not_read_channels_last_see_float32(gpu):
    """A float32 consumer (here the plain fp32 convolution and a host copy of a view) converts back transparently, and
    overwriting the array drops the channels-last form."""
    K = gpu.kernels
    rng = np.random.default_rng(9)
    x, w, b = _inputs(rng, 2, 32, 8, 32, 3)
    y = K.conv2d_fwd(gpu.to_device(x), gpu.to_device(w), gpu.to_device(b), (1, 1), 1, bf16=True, channels_last=True)
    expect = bf16_round(K.conv2d_fwd(gpu.to_device(x), gpu.to_device(w), gpu.to_device(b), (1, 1), 1, bf16=True).numpy())
    flat = y.reshape(2, -1)                                    # a view of the same allocation
    np.testing.assert_array_equal(flat.numpy(), expect.reshape(2, -1))
    y2 = K.conv2d_fwd(gpu.to_device(x), gpu.to_device(w), gpu.to_device(b), (1, 1), 1, bf16=True, channels_last=True)
    z = K.conv2d_fwd(y2, gpu.to_device(w), None, (1, 1), 1)     # fp32 kernels read y2 through its float32 form
    z_ref = K.conv2d_fwd(gpu.to_device(expect), gpu.to_device(w), None, (1, 1), 1)
    np.testing.assert_array_equal(z.numpy(), z_ref.numpy())
    y3 = K.conv2d_fwd(gpu.to_device(x), gpu.to_device(w), gpu.to_device(b), (1, 1), 1, bf16=True, channels_last=True)
    y3.set(np.ones(y3.shape, np.float32))
    assert y3.channels_last() is None
    np.testing.assert_array_equal(y3.numpy(), np.ones(y3.shape, np.float32))


def test_channels_last_entry_points_refuse_what_they_cannot_do(gpu):
    from xshinnosuke_amd.backend.capi import lib
    x = gpu.zeros((1, 16, 6, 6)); w = gpu.zeros((8, 16, 3, 3)); y = gpu.zeros((1, 8, 6, 6))
    ws = gpu.empty((1 << 20,), np.uint8)
    buf = gpu.zeros((1, 8, 8, 16), np.uint16)
    dims = (1, 16, 6, 6, 8, 3, 3, 1, 1, 1)
    with pytest.raises(ValueError):                              # a channels-last input needs C % 32 == 0
        lib.call("xsmi_conv2d_fwd_cl", None, buf.cptr, 1, w.cptr, None, y.cptr, None, 0, *dims, 0, ws.cptr, ws.nbytes)
    with pytest.raises(ValueError):                              # both forms of the input at once
        lib.call("xsmi_conv2d_fwd_cl", x.cptr, buf.cptr, 1, w.cptr, None, y.cptr, None, 0, *dims, 0, ws.cptr, ws.nbytes)
    with pytest.raises(ValueError):                              # border narrower than the padding
        lib.call("xsmi_cl_maxpool2d", buf.cptr, 0, buf.cptr, 0, 1, 16, 6, 6, 3, 2, 2, 1)
    with pytest.raises(ValueError):
        lib.call("xsmi_cl_add", buf.cptr, buf.cptr, buf.cptr, 12, 1)       # not a multiple of 8
