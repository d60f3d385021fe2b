"""Conv parity on the GPU through the C ABI.

Tolerance (fp32 MFMA path): relative L2 error <= 1e-5 against the oracle, which
computes in float64 and rounds once to float32 like the reference.
"""
import os

import numpy as np
import pytest

import oracle
from util import rel_l2, he_normal, round_bf16

pytestmark = pytest.mark.gpu
TOL = 1e-5

CASES = [  # n c h w k r s sh sw pad
    (1, 1, 4, 4, 3, 3, 3, 1, 1, 0),        # tests/gradient_check/xs_pytorch/cnn.py shapes
    (2, 3, 7, 6, 4, 3, 3, 1, 1, 1),
    (1, 3, 5, 5, 1, 3, 3, 1, 1, 0),        # tests/gradient_check/check_cnn.py shapes
    (4, 1, 28, 28, 8, 2, 2, 1, 1, 0),      # README net conv
    (2, 64, 56, 56, 64, 3, 3, 1, 1, 1),    # the benchmark conv geometry, fewer images
    (2, 3, 32, 32, 64, 7, 7, 2, 2, 3),     # ResNet stem geometry (small image)
    (2, 64, 28, 28, 128, 3, 3, 2, 2, 1),   # layer2.0 conv_a
    (2, 64, 28, 28, 128, 1, 1, 2, 2, 0),   # 1x1 / 2 shortcut
    (3, 128, 14, 14, 128, 3, 3, 1, 1, 1),
    (2, 256, 7, 7, 512, 3, 3, 2, 2, 1),    # small-M layer
    (1, 5, 9, 11, 70, 3, 2, 1, 2, 2),      # ragged: rows not a multiple of 64, asymmetric filter/stride
    (2, 7, 13, 12, 9, 5, 5, 3, 2, 2),      # stride 3x2, leftover input rows get zero gradient
    (1, 2, 6, 6, 3, 3, 3, 1, 1, 2),        # pad > (R-1)/2
    (5, 33, 10, 10, 65, 1, 1, 1, 1, 0),    # 1x1 == GEMM, odd sizes
    (1, 1, 3, 3, 1, 3, 3, 1, 1, 0),        # single output pixel
    (3, 1, 20, 32, 64, 5, 5, 1, 2, 2),     # few-channel first layers (horizontal stride 2, output width % 8 == 0):
    (2, 3, 17, 32, 128, 3, 3, 2, 2, 1),    #   one channel with vertical stride 1; two row tiles of filters;
    (2, 4, 12, 30, 64, 3, 3, 2, 2, 2),     #   four channels, padding wider than the filter's reach
]


def _oracle(x, w, b, stride, pad, dy):
    y, col = oracle.conv2d_fwd(x, w, b, stride, pad)
    dx, dw, db = oracle.conv2d_bwd(dy, x.shape, w, col, stride, pad,
                                   np.zeros_like(x), np.zeros_like(w), np.zeros((w.shape[0],), dtype=np.float32))
    return y, dx, dw, db


@pytest.mark.parametrize("n,c,h,w,k,r,s,sh,sw,pad", CASES)
def test_conv_fwd_bwd_parity(gpu, n, c, h, w, k, r, s, sh, sw, pad):
    K = gpu.kernels
    rng = np.random.default_rng(1000 + c * k + h)
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    wt = he_normal(rng, (k, c, r, s))
    b = rng.standard_normal((k,)).astype(np.float32)
    oh, ow = K.conv_out_hw(h, w, r, s, (sh, sw), pad)
    dy = rng.standard_normal((n, k, oh, ow)).astype(np.float32)
    y_ref, dx_ref, dw_ref, db_ref = _oracle(x, wt, b, (sh, sw), pad, dy)

    dx_, dw_, db_, ddy = gpu.to_device(x), gpu.to_device(wt), gpu.to_device(b), gpu.to_device(dy)
    y = K.conv2d_fwd(dx_, dw_, db_, (sh, sw), pad).numpy()
    assert y.shape == y_ref.shape
    assert rel_l2(y, y_ref) <= TOL
    gx = K.conv2d_bwd_data(ddy, dw_, x.shape, (sh, sw), pad).numpy()
    assert rel_l2(gx, dx_ref) <= TOL
    gw, gb = K.conv2d_bwd_weight(ddy, dx_, wt.shape, (sh, sw), pad, want_db=True)
    assert rel_l2(gw.numpy(), dw_ref) <= TOL
    assert rel_l2(gb.numpy(), db_ref) <= TOL


@pytest.mark.parametrize("n,c,h,w,k", [(2, 64, 28, 28, 128), (3, 32, 8, 12, 40), (2, 64, 27, 28, 64), (1, 96, 6, 6, 32)])
def test_shortcut_bwd_data_overwrites_every_element(gpu, n, c, h, w, k):
    """1 x 1 / 2 backward-data into a tensor that holds other values: the three residue classes no tap reaches must
    come out as exact zeros (even sizes: written by the kernel's own epilogue; odd sizes: by a fill), whole and ragged
    row tiles alike."""
    K = gpu.kernels
    rng = np.random.default_rng(c + h)
    wt = he_normal(rng, (k, c, 1, 1))
    oh, ow = K.conv_out_hw(h, w, 1, 1, (2, 2), 0)
    dy = rng.standard_normal((n, k, oh, ow)).astype(np.float32)
    ref = np.zeros((n, c, h, w), np.float32)
    ref[:, :, ::2, ::2] = np.einsum("nkyx,kc->ncyx", dy.astype(np.float64), wt[:, :, 0, 0].astype(np.float64))
    dx = gpu.to_device(np.full((n, c, h, w), 7.0, np.float32))
    got = K.conv2d_bwd_data(gpu.to_device(dy), gpu.to_device(wt), (n, c, h, w), (2, 2), 0, dx=dx).numpy()
    lattice = np.zeros((h, w), bool); lattice[::2, ::2] = True
    assert np.all(got[:, :, ~lattice] == 0.0)
    assert rel_l2(got, ref) <= TOL
    twice = K.conv2d_bwd_data(gpu.to_device(dy), gpu.to_device(wt), (n, c, h, w), (2, 2), 0, dx=dx, accumulate=True).numpy()
    assert np.all(twice[:, :, ~lattice] == 0.0)
    assert rel_l2(twice, 2 * ref) <= TOL


def test_conv_accumulates_into_existing_gradients(gpu):
    K = gpu.kernels
    rng = np.random.default_rng(7)
    x = rng.standard_normal((2, 6, 9, 9)).astype(np.float32); wt = he_normal(rng, (10, 6, 3, 3))
    dy = rng.standard_normal((2, 10, 5, 5)).astype(np.float32)
    _, col = oracle.conv2d_fwd(x, wt, None, (2, 2), 1)
    dx0 = rng.standard_normal(x.shape).astype(np.float32); dw0 = rng.standard_normal(wt.shape).astype(np.float32)
    db0 = rng.standard_normal((10,)).astype(np.float32)
    dx_ref, dw_ref, db_ref = oracle.conv2d_bwd(dy, x.shape, wt, col, (2, 2), 1, dx0.copy(), dw0.copy(), db0.copy())
    gx, gw, gb = gpu.to_device(dx0), gpu.to_device(dw0), gpu.to_device(db0)
    ddy = gpu.to_device(dy)
    K.conv2d_bwd_data(ddy, gpu.to_device(wt), x.shape, (2, 2), 1, dx=gx, accumulate=True)
    K.conv2d_bwd_weight(ddy, gpu.to_device(x), wt.shape, (2, 2), 1, dw=gw, db=gb, accumulate=True)
    assert rel_l2(gx.numpy(), dx_ref) <= TOL
    assert rel_l2(gw.numpy(), dw_ref) <= TOL
    assert rel_l2(gb.numpy(), db_ref) <= TOL


def test_conv_fused_bias_relu_and_mask(gpu):
    K = gpu.kernels
    rng = np.random.default_rng(8)
    x = rng.standard_normal((3, 4, 12, 12)).astype(np.float32); wt = he_normal(rng, (6, 4, 3, 3))
    b = rng.standard_normal((6,)).astype(np.float32)
    pre_ref, _ = oracle.conv2d_fwd(x, wt, b, (1, 1), 1)
    dx_, dw_, db_ = gpu.to_device(x), gpu.to_device(wt), gpu.to_device(b)
    pre = K.conv2d_fwd(dx_, dw_, db_, (1, 1), 1).numpy()
    mask = gpu.empty(pre.shape, np.uint8)
    act = K.conv2d_fwd(dx_, dw_, db_, (1, 1), 1, relu=True, neg_mask=mask).numpy()
    np.testing.assert_array_equal(act, oracle.relu_fwd(pre))           # same kernel arithmetic, then max(0, .)
    np.testing.assert_array_equal(mask.numpy(), (pre < 0).astype(np.uint8))
    assert rel_l2(act, oracle.relu_fwd(pre_ref)) <= TOL
    dy = rng.standard_normal(pre.shape).astype(np.float32)
    g = K.relu_mask_bwd(gpu.to_device(dy), mask).numpy()
    np.testing.assert_array_equal(g, oracle.relu_bwd(dy, pre))


BF16_CASES = [  # shapes whose reduction channels are a multiple of 32 take the bf16 MFMA kernel
    (2, 64, 56, 56, 64, 3, 3, 1, 1, 1),
    (2, 64, 28, 28, 128, 3, 3, 2, 2, 1),
    (2, 64, 28, 28, 128, 1, 1, 2, 2, 0),
    (3, 128, 14, 14, 130, 3, 3, 1, 1, 1),
    (2, 3, 32, 32, 64, 7, 7, 2, 2, 3),     # stem: channels padded to one octet in the channels-last forward
]


@pytest.mark.parametrize("n,c,h,w,k,r,s,sh,sw,pad", BF16_CASES)
def test_conv_bf16_opt_in(gpu, n, c, h, w, k, r, s, sh, sw, pad):
    """bf16 opt-in: tolerance rel-L2 <= 1e-2 against the fp32-rounded float64 oracle; against the oracle fed
    with operands rounded to bf16 (round to nearest even) only the fp32 accumulation differs: <= 1e-5."""
    K = gpu.kernels
    rng = np.random.default_rng(77 + c + k)
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    wt = he_normal(rng, (k, c, r, s))
    b = rng.standard_normal((k,)).astype(np.float32)
    oh, ow = K.conv_out_hw(h, w, r, s, (sh, sw), pad)
    dy = rng.standard_normal((n, k, oh, ow)).astype(np.float32)
    y_ref, dx_ref, _, _ = _oracle(x, wt, b, (sh, sw), pad, dy)
    dx_, dw_, db_, ddy = gpu.to_device(x), gpu.to_device(wt), gpu.to_device(b), gpu.to_device(dy)
    y = K.conv2d_fwd(dx_, dw_, db_, (sh, sw), pad, bf16=True).numpy()
    gx = K.conv2d_bwd_data(ddy, dw_, x.shape, (sh, sw), pad, bf16=True).numpy()
    assert rel_l2(y, y_ref) <= 1e-2
    assert rel_l2(gx, dx_ref) <= 1e-2
    if c % 32 == 0 or c <= 8:
        y_r, _ = oracle.conv2d_fwd(round_bf16(x), round_bf16(wt), b, (sh, sw), pad)
        assert rel_l2(y, y_r) <= TOL
        assert rel_l2(y, y_ref) > 1e-4            # the bf16 kernel really ran
    if k % 32 == 0:
        _, col = oracle.conv2d_fwd(x, round_bf16(wt), None, (sh, sw), pad)
        dx_r, _, _ = oracle.conv2d_bwd(round_bf16(dy), x.shape, round_bf16(wt), col, (sh, sw), pad, np.zeros_like(x),
                                       np.zeros_like(wt), np.zeros((k,), dtype=np.float32))
        assert rel_l2(gx, dx_r) <= TOL
    # the weight gradient accepts the flag and stays on the fp32 path
    gw, _ = K.conv2d_bwd_weight(ddy, dx_, wt.shape, (sh, sw), pad, want_db=True, bf16=True)
    gw32, _ = K.conv2d_bwd_weight(ddy, dx_, wt.shape, (sh, sw), pad, want_db=True)
    np.testing.assert_array_equal(gw.numpy(), gw32.numpy())


BF16_FWD_CASES = [  # n, c, h, w, k, r, s, sh, sw, pad: tile tails in rows and pixels, odd chunk counts, both tile shapes
    (1, 32, 5, 7, 8, 1, 1, 1, 1, 0),
    (3, 96, 9, 11, 70, 3, 3, 1, 1, 1),
    (2, 32, 13, 13, 200, 5, 5, 2, 2, 2),
    (5, 64, 17, 15, 64, 3, 3, 1, 1, 0),
    (2, 128, 30, 30, 128, 3, 3, 1, 1, 1),
    (4, 1, 28, 28, 8, 2, 2, 1, 1, 0),
    (2, 8, 20, 18, 130, 3, 5, 1, 2, 2),
    (1, 3, 224, 224, 64, 7, 7, 2, 2, 3),
    (2, 512, 7, 7, 512, 3, 3, 1, 1, 1),
]


@pytest.mark.parametrize("n,c,h,w,k,r,s,sh,sw,pad", BF16_FWD_CASES)
def test_conv_bf16_forward_channels_last(gpu, n, c, h, w, k, r, s, sh, sw, pad):
    """bf16 forward through the channels-last copy, with the fused bias + ReLU epilogue and its sign mask:
    against the oracle on operands rounded to bf16 only the fp32 accumulation order differs (<= 1e-5)."""
    K = gpu.kernels
    rng = np.random.default_rng(1000 + 7 * c + k)
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    wt = he_normal(rng, (k, c, r, s))
    b = rng.standard_normal((k,)).astype(np.float32)
    pre_ref, _ = oracle.conv2d_fwd(round_bf16(x), round_bf16(wt), b, (sh, sw), pad)
    dx_, dw_, db_ = gpu.to_device(x), gpu.to_device(wt), gpu.to_device(b)
    y = K.conv2d_fwd(dx_, dw_, db_, (sh, sw), pad, bf16=True).numpy()
    assert y.shape == pre_ref.shape
    assert rel_l2(y, pre_ref) <= TOL
    mask = gpu.empty(pre_ref.shape, np.uint8)
    act = K.conv2d_fwd(dx_, dw_, db_, (sh, sw), pad, relu=True, neg_mask=mask, bf16=True).numpy()
    np.testing.assert_array_equal(act, np.maximum(y, 0.0))
    np.testing.assert_array_equal(mask.numpy(), (y < 0).astype(np.uint8))
    # the filter may stay packed between calls; without a bias the epilogue adds nothing
    y0 = K.conv2d_fwd(dx_, dw_, None, (sh, sw), pad, bf16=True).numpy()
    y1 = K.conv2d_fwd(dx_, dw_, None, (sh, sw), pad, bf16=True, packed=True).numpy()
    np.testing.assert_array_equal(y0, y1)
    assert rel_l2(y0 + b.reshape(1, -1, 1, 1), pre_ref) <= TOL


@pytest.mark.parametrize("n,c,h,w,k,r,s,sh,sw,pad", [CASES[2], CASES[4], CASES[6], CASES[9], CASES[11]])
@pytest.mark.parametrize("accumulate", [False, True])
@pytest.mark.parametrize("async_dw", [False, True])
def test_conv_both_gradients_in_one_call(gpu, n, c, h, w, k, r, s, sh, sw, pad, accumulate, async_dw):
    """xsmi_conv2d_bwd runs the two backward kernels on two streams: same bits as the two calls one after the
    other, also when adding into gradients that are already there, and twice in a row (the second call's kernels
    must wait for the first call's).  With async_dw the weight gradient is still on the second stream when the call
    returns; reading it back joins first."""
    from xshinnosuke_amd.backend import capi
    K = gpu.kernels
    rng = np.random.default_rng(77 + c + k)
    x = gpu.to_device(rng.standard_normal((n, c, h, w)).astype(np.float32))
    wt = gpu.to_device(he_normal(rng, (k, c, r, s)))
    oh, ow = K.conv_out_hw(h, w, r, s, (sh, sw), pad)
    dys = [gpu.to_device(rng.standard_normal((n, k, oh, ow)).astype(np.float32)) for _ in range(2)]
    init = [rng.standard_normal(shape).astype(np.float32) for shape in ((n, c, h, w), (k, c, r, s), (k,))]
    a = [gpu.to_device(v) for v in init]
    b = [gpu.to_device(v) for v in init]
    for dy in dys:
        K.conv2d_bwd_weight(dy, x, wt.shape, (sh, sw), pad, dw=a[1], db=a[2], accumulate=accumulate)
        K.conv2d_bwd_data(dy, wt, x.shape, (sh, sw), pad, dx=a[0], accumulate=accumulate)
    for dy in dys:
        K.conv2d_bwd(dy, x, wt, b[0], b[1], b[2], (sh, sw), pad, accumulate=accumulate, async_dw=async_dw)
        assert capi.side_pending() == async_dw
    for u, v in zip(a, b):
        assert np.array_equal(u.numpy(), v.numpy())
    assert not capi.side_pending()


def test_conv_async_weight_gradient_is_joined_before_use(gpu):
    """Whatever touches the weight gradient after an asynchronous xsmi_conv2d_bwd (an optimizer update, the plain
    weight-gradient entry point adding into the same buffer) sees it complete; the passes of a backward sweep that
    cannot touch it do not wait."""
    from xshinnosuke_amd.backend import capi
    K = gpu.kernels
    rng = np.random.default_rng(5)
    n, c, h, k = 8, 64, 28, 64
    x = gpu.to_device(rng.standard_normal((n, c, h, h)).astype(np.float32))
    wt = gpu.to_device(he_normal(rng, (k, c, 3, 3)))
    dy = gpu.to_device(rng.standard_normal((n, k, h, h)).astype(np.float32))
    ref_dw, _ = K.conv2d_bwd_weight(dy, x, wt.shape, (1, 1), 1)
    ref = ref_dw.numpy()
    twice = gpu.to_device(ref)
    K.conv2d_bwd_weight(dy, x, wt.shape, (1, 1), 1, dw=twice, accumulate=True)
    for use in ("axpy", "bwd_weight", "sync"):
        dx, dw = gpu.empty(x.shape), gpu.empty(wt.shape)
        other = gpu.empty(x.shape)
        mask = gpu.to_device(np.zeros(x.shape, np.uint8))
        K.conv2d_bwd(dy, x, wt, dx, dw, None, (1, 1), 1, async_dw=True)
        K.relu_mask_bwd(dx, mask, dx=other)                  # a pass of the sweep: does not join
        assert capi.side_pending()
        if use == "axpy":
            p = gpu.to_device(np.zeros(wt.shape, np.float32))
            K.axpy(p, dw, 1.0)
            assert not capi.side_pending()
            np.testing.assert_array_equal(p.numpy(), ref)
        elif use == "bwd_weight":
            K.conv2d_bwd_weight(dy, x, wt.shape, (1, 1), 1, dw=dw, accumulate=True)
            assert not capi.side_pending()
            np.testing.assert_array_equal(dw.numpy(), twice.numpy())
        else:
            gpu.synchronize()
            assert not capi.side_pending()
            np.testing.assert_array_equal(dw.numpy(), ref)


def test_conv_packed_workspace_flag(gpu):
    """XSMI_CONV_WS_PACKED: a repeated forward / backward-data call may skip laying the filter out again."""
    K = gpu.kernels
    rng = np.random.default_rng(21)
    for (n, c, h, w, k, st) in ((2, 64, 20, 20, 64, 1), (2, 64, 20, 20, 128, 2), (1, 3, 9, 9, 5, 1)):
        x = rng.standard_normal((n, c, h, w)).astype(np.float32)
        wt = he_normal(rng, (k, c, 3, 3))
        dx_, dw_ = gpu.to_device(x), gpu.to_device(wt)
        y0 = K.conv2d_fwd(dx_, dw_, None, (st, st), 1).numpy()
        y1 = K.conv2d_fwd(dx_, dw_, None, (st, st), 1, packed=True).numpy()
        np.testing.assert_array_equal(y0, y1)
        dy = gpu.to_device(rng.standard_normal(y0.shape).astype(np.float32))
        g0 = K.conv2d_bwd_data(dy, dw_, x.shape, (st, st), 1).numpy()
        g1 = K.conv2d_bwd_data(dy, dw_, x.shape, (st, st), 1, packed=True).numpy()
        np.testing.assert_array_equal(g0, g1)


def test_conv_special_kernels_exact(gpu):
    """Closed forms that need no rounding: delta filter == shift, ones filter on small integers == box sum."""
    K = gpu.kernels
    rng = np.random.default_rng(9)
    x = rng.integers(-8, 9, size=(2, 1, 10, 12)).astype(np.float32)
    wd = np.zeros((1, 1, 3, 3), dtype=np.float32); wd[0, 0, 0, 2] = 1.0
    y = K.conv2d_fwd(gpu.to_device(x), gpu.to_device(wd), None, (1, 1), 1).numpy()
    ref = np.zeros_like(x); ref[:, :, 1:, :-1] = x[:, :, :-1, 1:]
    np.testing.assert_array_equal(y, ref)
    wo = np.ones((1, 1, 2, 2), dtype=np.float32)
    y = K.conv2d_fwd(gpu.to_device(x), gpu.to_device(wo), None, (1, 1), 0).numpy()
    np.testing.assert_array_equal(y, x[:, :, :-1, :-1] + x[:, :, 1:, :-1] + x[:, :, :-1, 1:] + x[:, :, 1:, 1:])


def test_conv_golden_fixture(gpu):
    K = gpu.kernels
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "conv_pool_small.npz"))
    stride = tuple(int(v) for v in g["conv_stride"]); pad = int(g["conv_pad"])
    x, w, b, dy = (gpu.to_device(g[k]) for k in ("conv_x", "conv_w", "conv_b", "conv_dy"))
    # dyadic inputs: every partial sum is exactly representable, so the match is exact
    np.testing.assert_array_equal(K.conv2d_fwd(x, w, b.reshape(-1), stride, pad).numpy(), g["conv_y"])
    np.testing.assert_array_equal(K.conv2d_bwd_data(dy, w, x.shape, stride, pad).numpy(), g["conv_dx"])
    gw, gb = K.conv2d_bwd_weight(dy, x, w.shape, stride, pad, want_db=True)
    np.testing.assert_array_equal(gw.numpy(), g["conv_dw"])
    np.testing.assert_array_equal(gb.numpy().reshape(1, -1), g["conv_db"])


def test_conv_full_size_adjoint_and_slice(gpu):
    """The benchmark conv configuration at full size (N=32, 64->64, 56x56, 3x3/1/1): bilinear identities in float64 on
    the device results plus oracle parity on a slice of images."""
    K = gpu.kernels
    x = np.random.default_rng(1).standard_normal((32, 64, 56, 56), dtype=np.float32)
    wt = he_normal(np.random.default_rng(2), (64, 64, 3, 3))
    dy = np.random.default_rng(3).standard_normal((32, 64, 56, 56), dtype=np.float32)
    dx_, dw_, ddy = gpu.to_device(x), gpu.to_device(wt), gpu.to_device(dy)
    y = K.conv2d_fwd(dx_, dw_, None, (1, 1), 1).numpy()
    gx = K.conv2d_bwd_data(ddy, dw_, x.shape, (1, 1), 1).numpy()
    gw, gb = K.conv2d_bwd_weight(ddy, dx_, wt.shape, (1, 1), 1, want_db=True)
    gw, gb = gw.numpy(), gb.numpy()
    f = np.float64
    lhs = np.sum(dy.astype(f) * y.astype(f))
    assert abs(lhs - np.sum(gx.astype(f) * x.astype(f))) <= 2e-5 * abs(lhs) + 1e-2 * np.sqrt(x.size) * 1e-5
    assert abs(lhs - np.sum(gw.astype(f) * wt.astype(f))) <= 2e-5 * abs(lhs) + 1e-2 * np.sqrt(x.size) * 1e-5
    assert rel_l2(gb, dy.astype(f).sum(axis=(0, 2, 3))) <= TOL
    y_ref, col = oracle.conv2d_fwd(x[:2], wt, None, (1, 1), 1)
    assert rel_l2(y[:2], y_ref) <= TOL
    dx_ref, _, _ = oracle.conv2d_bwd(dy[:2], x[:2].shape, wt, col, (1, 1), 1, np.zeros_like(x[:2]), None, None)
    assert rel_l2(gx[:2], dx_ref) <= TOL
    # dW over the full batch in float64 (einsum over taps), the reference's dot(grad, col) without the 462 MB matrix
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1))).astype(f)
    dw_ref = np.empty((64, 64, 3, 3))
    dyf = dy.astype(f).transpose(1, 0, 2, 3).reshape(64, -1)
    for r in range(3):
        for s in range(3):
            win = xp[:, :, r:r + 56, s:s + 56].transpose(1, 0, 2, 3).reshape(64, -1)
            dw_ref[:, :, r, s] = dyf @ win.T
    assert rel_l2(gw, dw_ref) <= TOL


@pytest.mark.parametrize("c,hw,k,r,st,pad", [(128, 28, 128, 3, 1, 1), (3, 224, 64, 7, 2, 3)])
def test_conv_bf16_full_size_batch_slices(gpu, c, hw, k, r, st, pad):
    """bf16 forward at the inference batch (N=256; a residual-stage layer and the stem): every image is
    convolved independently and in one reduction order, so images cut from the big batch equal the same images
    run as a small batch bit for bit, and the small batch meets the oracle on bf16-rounded operands."""
    K = gpu.kernels
    n = 256
    rng = np.random.default_rng(40 + c)
    x = rng.standard_normal((n, c, hw, hw), dtype=np.float32)
    wt = he_normal(rng, (k, c, r, r))
    b = rng.standard_normal((k,)).astype(np.float32)
    dw_, db_ = gpu.to_device(wt), gpu.to_device(b)
    y = K.conv2d_fwd(gpu.to_device(x), dw_, db_, (st, st), pad, relu=True, bf16=True).numpy()
    for sl in (slice(0, 2), slice(101, 104), slice(254, 256)):
        part = K.conv2d_fwd(gpu.to_device(x[sl]), dw_, db_, (st, st), pad, relu=True, bf16=True).numpy()
        np.testing.assert_array_equal(y[sl], part)
    ref, _ = oracle.conv2d_fwd(round_bf16(x[254:]), round_bf16(wt), b, (st, st), pad)
    assert rel_l2(y[254:], np.maximum(ref, 0.0)) <= TOL


def test_conv_rejects_bad_arguments(gpu):
    K = gpu.kernels
    x = gpu.zeros((1, 3, 4, 4)); w = gpu.zeros((2, 4, 3, 3))
    with pytest.raises(ValueError):
        K.conv2d_fwd(x, w)                       # channel mismatch
    w = gpu.zeros((2, 3, 5, 5))
    with pytest.raises(ValueError):
        K.conv2d_fwd(x, w)                       # filter larger than the input
    with pytest.raises(ValueError):
        K.conv2d_fwd(x, gpu.zeros((2, 3, 3, 3)), stride=(0, 1))


def test_conv_combined_backward_rejects_bad_arguments(gpu):
    """The C ABI refuses what it cannot run safely: unknown flags, a missing or too small workspace, two workspaces
    that overlap; the wrappers refuse mismatched buffers before anything is enqueued."""
    import ctypes
    from xshinnosuke_amd.backend import capi
    K = gpu.kernels
    x = gpu.zeros((2, 64, 8, 8)); w = gpu.zeros((64, 64, 3, 3)); dy = gpu.zeros((2, 64, 8, 8))
    dx = gpu.zeros(x.shape); dw = gpu.zeros(w.shape)
    dims = [2, 64, 8, 8, 64, 3, 3, 1, 1, 1]
    need = capi.lib.raw("xsmi_conv2d_workspace_bytes")(*dims)
    ws = gpu.empty((2 * need // 4 + 64,))
    base = ws.cptr.value
    a, b = ctypes.c_void_p(base), ctypes.c_void_p(base + (need + 255) // 256 * 256)
    args = [dy.cptr, x.cptr, w.cptr, dx.cptr, dw.cptr, None] + dims + [0.0, 0.0]
    capi.lib.call("xsmi_conv2d_bwd", *args, 0, a, need, b, need)                 # the well-formed call
    with pytest.raises(ValueError, match="unknown flags"):
        capi.lib.call("xsmi_conv2d_bwd", *args, 0x40, a, need, b, need)
    with pytest.raises(ValueError, match="workspace"):
        capi.lib.call("xsmi_conv2d_bwd", *args, 0, a, need, None, 0)
    with pytest.raises(ValueError, match="workspace"):
        capi.lib.call("xsmi_conv2d_bwd", *args, 0, a, 16, b, need)
    with pytest.raises(ValueError, match="overlap"):
        capi.lib.call("xsmi_conv2d_bwd", *args, 0, a, need, ctypes.c_void_p(base + 256), need)
    with pytest.raises(ValueError, match="beta"):
        capi.lib.call("xsmi_conv2d_bwd", *(args[:-2] + [0.5, 0.0]), 0, a, need, b, need)
    with pytest.raises(ValueError):
        K.conv2d_bwd(dy, x, w, gpu.zeros((2, 64, 8, 9)), dw)                      # dx of another shape
    with pytest.raises(ValueError):
        K.conv2d_bwd(gpu.zeros((2, 64, 7, 8)), x, w, dx, dw)                      # dy of another shape
    with pytest.raises(ValueError):
        K.relu_mask_bwd2(dy, gpu.zeros(dy.shape, np.uint8), dx, dx)               # one buffer given twice
    gpu.synchronize()
    assert not capi.side_pending()


@pytest.mark.parametrize("n,c,h,w,k,r,s,sh,sw,pad", [CASES[4], CASES[5], CASES[6], CASES[7], CASES[9], CASES[10]])
def test_each_pass_runs_in_a_workspace_of_its_own_size(gpu, n, c, h, w, k, r, s, sh, sw, pad):
    """xsmi_conv2d_pass_workspace_bytes is enough for its pass and selects the same kernel as the full-size workspace:
    the three passes through the C ABI with exactly that many bytes give the wrappers' bits."""
    import ctypes
    from xshinnosuke_amd.backend import capi
    K = gpu.kernels
    rng = np.random.default_rng(77 + c + k)
    x = gpu.to_device(rng.standard_normal((n, c, h, w)).astype(np.float32))
    wt = gpu.to_device(he_normal(rng, (k, c, r, s)))
    oh, ow = K.conv_out_hw(h, w, r, s, (sh, sw), pad)
    dy = gpu.to_device(rng.standard_normal((n, k, oh, ow)).astype(np.float32))
    dims = [n, c, h, w, k, r, s, sh, sw, pad]
    y_ref = K.conv2d_fwd(x, wt, None, (sh, sw), pad).numpy()
    dx_ref = K.conv2d_bwd_data(dy, wt, x.shape, (sh, sw), pad).numpy()
    dw_ref = K.conv2d_bwd_weight(dy, x, wt.shape, (sh, sw), pad)[0].numpy()
    size = [capi.lib.raw("xsmi_conv2d_pass_workspace_bytes")(*dims, p, 0) for p in range(3)]
    assert all(v > 0 for v in size)
    y = gpu.empty(y_ref.shape); dx = gpu.empty(dx_ref.shape); dw = gpu.empty(dw_ref.shape)
    ws = [gpu.empty(((v + 3) // 4,)) for v in size]
    capi.lib.call("xsmi_conv2d_fwd", x.cptr, wt.cptr, None, y.cptr, None, *dims, 0, ws[0].cptr, size[0])
    capi.lib.call("xsmi_conv2d_bwd_data", dy.cptr, wt.cptr, dx.cptr, *dims, 0.0, 0, ws[1].cptr, size[1])
    capi.lib.call("xsmi_conv2d_bwd_weight", dy.cptr, x.cptr, dw.cptr, None, *dims, 0.0, 0, ws[2].cptr, size[2])
    assert y.numpy().tobytes() == y_ref.tobytes()
    assert dx.numpy().tobytes() == dx_ref.tobytes()
    assert dw.numpy().tobytes() == dw_ref.tobytes()
    with pytest.raises(ValueError, match="workspace"):
        capi.lib.call("xsmi_conv2d_fwd", x.cptr, wt.cptr, None, y.cptr, None, *dims, 0, ws[0].cptr, 16)
