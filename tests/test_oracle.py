"""Pins the CPU oracle (oracle/xs_oracle.py) without running the reference.

The reference's own tests hold no stored expected values for conv / max-pool
(they print distances to PyTorch), so the oracle is pinned by
  * brute-force loops written from the index formulas (oracle/brute.py),
  * torch CPU on the shapes and seeds of the reference's scripts
    (tests/gradient_check/xs_pytorch/cnn.py:4-8, pooling.py:4-5),
  * adjoint identities, central differences (technique of
    xs/utils/toolkit.py:160-194), special kernels with closed forms,
  * the committed fixtures under tests/golden/ (made by the brute-force code).
"""
import os

import numpy as np
import pytest

import oracle
from util import rel_l2, with_ties, idx_ref_to_nchw

CASES = [  # n c h w k r s sh sw pad
    (2, 3, 7, 6, 4, 3, 3, 1, 1, 1),
    (1, 2, 8, 9, 3, 3, 2, 2, 2, 1),
    (2, 1, 5, 5, 2, 1, 1, 2, 2, 0),
    (1, 3, 9, 9, 2, 7, 7, 2, 2, 3),
    (1, 2, 6, 7, 3, 2, 2, 1, 1, 0),
    (1, 2, 7, 8, 2, 3, 3, 3, 2, 2),
]


@pytest.mark.parametrize("n,c,h,w,k,r,s,sh,sw,pad", CASES)
def test_conv_forward_matches_brute_force(n, c, h, w, k, r, s, sh, sw, pad):
    rng = np.random.default_rng(11)
    x = rng.standard_normal((n, c, h, w))
    wt = rng.standard_normal((k, c, r, s))
    b = rng.standard_normal((1, k))
    y, _ = oracle.conv2d_fwd(x, wt, b, (sh, sw), pad)
    yb = oracle.conv2d_fwd_brute(x, wt, b, (sh, sw), pad)
    assert y.shape == yb.shape
    np.testing.assert_allclose(y, yb, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("n,c,h,w,k,r,s,sh,sw,pad", CASES)
def test_conv_backward_matches_brute_force(n, c, h, w, k, r, s, sh, sw, pad):
    rng = np.random.default_rng(12)
    x = rng.standard_normal((n, c, h, w))
    wt = rng.standard_normal((k, c, r, s))
    y, col = oracle.conv2d_fwd(x, wt, None, (sh, sw), pad)
    dy = rng.standard_normal(y.shape)
    dx, dw, db = oracle.conv2d_bwd(dy, x.shape, wt, col, (sh, sw), pad,
                                   np.zeros_like(x), np.zeros_like(wt), np.zeros((1, k)))
    dxb, dwb, dbb = oracle.conv2d_bwd_brute(dy, x, wt, (sh, sw), pad)
    np.testing.assert_allclose(dx, dxb, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dw, dwb, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(db.ravel(), dbb, rtol=1e-12, atol=1e-12)


def test_conv_backward_accumulates():
    rng = np.random.default_rng(13)
    x = rng.standard_normal((2, 3, 6, 6)); wt = rng.standard_normal((4, 3, 3, 3))
    y, col = oracle.conv2d_fwd(x, wt, None, (1, 1), 1)
    dy = rng.standard_normal(y.shape)
    dx = np.zeros_like(x); dw = np.zeros_like(wt); db = np.zeros((4,))
    oracle.conv2d_bwd(dy, x.shape, wt, col, (1, 1), 1, dx, dw, db)
    once = (dx.copy(), dw.copy(), db.copy())
    oracle.conv2d_bwd(dy, x.shape, wt, col, (1, 1), 1, dx, dw, db)
    for a, b in zip((dx, dw, db), once):
        np.testing.assert_allclose(a, 2 * b, rtol=1e-13)


def test_conv_matches_torch_on_reference_script_shapes():
    torch = pytest.importorskip("torch")
    np.random.seed(0)   # seeds and shapes of tests/gradient_check/xs_pytorch/cnn.py:4-8
    n_x = np.random.randn(1, 1, 4, 4).astype(np.float32)
    _ = np.random.randn(1).astype(np.float32)
    n_w = np.random.randn(3, 1, 3, 3).astype(np.float32)
    n_b = np.random.randn(3).astype(np.float32)
    tx = torch.tensor(n_x, requires_grad=True); tw = torch.tensor(n_w, requires_grad=True)
    tb = torch.tensor(n_b, requires_grad=True)
    ty = torch.nn.functional.conv2d(tx, tw, tb)
    g = torch.arange(ty.numel(), dtype=torch.float32).reshape(ty.shape) / 7 - 1
    ty.backward(g)
    y, col = oracle.conv2d_fwd(n_x, n_w, n_b, (1, 1), 0)
    assert y.dtype == np.float32
    dx, dw, db = oracle.conv2d_bwd(g.numpy(), n_x.shape, n_w, col, (1, 1), 0,
                                   np.zeros_like(n_x), np.zeros_like(n_w), np.zeros_like(n_b))
    assert rel_l2(y, ty.detach().numpy()) < 1e-6
    assert rel_l2(dx, tx.grad.numpy()) < 1e-6
    assert rel_l2(dw, tw.grad.numpy()) < 1e-6
    assert rel_l2(db, tb.grad.numpy()) < 1e-6


@pytest.mark.parametrize("stride,pad,r", [((1, 1), 1, 3), ((2, 2), 1, 3), ((2, 2), 3, 7), ((2, 2), 0, 1)])
def test_conv_matches_torch_strided(stride, pad, r):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 4, 13, 12)).astype(np.float32)
    wt = rng.standard_normal((5, 4, r, r)).astype(np.float32)
    tx = torch.tensor(x, requires_grad=True); tw = torch.tensor(wt, requires_grad=True)
    ty = torch.nn.functional.conv2d(tx, tw, None, stride=stride, padding=pad)
    g = torch.tensor(rng.standard_normal(tuple(ty.shape)).astype(np.float32))
    ty.backward(g)
    y, col = oracle.conv2d_fwd(x, wt, None, stride, pad)
    dx, dw, _ = oracle.conv2d_bwd(g.numpy(), x.shape, wt, col, stride, pad, np.zeros_like(x), np.zeros_like(wt), None)
    assert rel_l2(y, ty.detach().numpy()) < 2e-6
    assert rel_l2(dx, tx.grad.numpy()) < 2e-6
    assert rel_l2(dw, tw.grad.numpy()) < 2e-6


def test_conv_adjoint_identities():
    rng = np.random.default_rng(21)
    x = rng.standard_normal((2, 3, 9, 8)); wt = rng.standard_normal((4, 3, 3, 3))
    for stride, pad in [((1, 1), 1), ((2, 2), 1), ((2, 1), 0)]:
        y, col = oracle.conv2d_fwd(x, wt, None, stride, pad)
        dy = rng.standard_normal(y.shape)
        dx, dw, db = oracle.conv2d_bwd(dy, x.shape, wt, col, stride, pad,
                                       np.zeros_like(x), np.zeros_like(wt), np.zeros(4))
        lhs = np.sum(dy * y)
        assert abs(lhs - np.sum(dx * x)) < 1e-9 * abs(lhs) + 1e-9     # <dY, conv(X,W)> = <dX, X>
        assert abs(lhs - np.sum(dw * wt)) < 1e-9 * abs(lhs) + 1e-9    #                 = <dW, W>
        np.testing.assert_allclose(db, dy.sum(axis=(0, 2, 3)), rtol=1e-12)


def test_conv_central_differences():
    rng = np.random.default_rng(22)
    x = rng.standard_normal((1, 3, 5, 5)); wt = rng.standard_normal((1, 3, 3, 3)); b = rng.standard_normal((1, 1))
    stride, pad, eps = (1, 1), 0, 1e-4   # shapes of tests/gradient_check/check_cnn.py:8-42

    def loss(xx, ww, bb):
        y, _ = oracle.conv2d_fwd(xx, ww, bb, stride, pad)
        return 0.5 * np.sum(y * y)

    y, col = oracle.conv2d_fwd(x, wt, b, stride, pad)
    dx, dw, db = oracle.conv2d_bwd(y, x.shape, wt, col, stride, pad, np.zeros_like(x), np.zeros_like(wt), np.zeros((1, 1)))
    for arr, grad, which in ((x, dx, 0), (wt, dw, 1), (b, db, 2)):
        num = np.zeros_like(arr)
        it = np.nditer(arr, flags=["multi_index"])
        for _ in it:
            i = it.multi_index
            old = arr[i]
            arr[i] = old + eps; lp = loss(x, wt, b)
            arr[i] = old - eps; lm = loss(x, wt, b)
            arr[i] = old
            num[i] = (lp - lm) / (2 * eps)
        assert rel_l2(grad, num) < 1e-6, which


def test_conv_special_kernels():
    rng = np.random.default_rng(23)
    x = rng.standard_normal((2, 3, 6, 7))
    # 1x1 filter == channel-mixing GEMM
    w1 = rng.standard_normal((4, 3, 1, 1))
    y, _ = oracle.conv2d_fwd(x, w1, None, (1, 1), 0)
    np.testing.assert_allclose(y, np.einsum("kc,nchw->nkhw", w1[:, :, 0, 0], x), rtol=1e-12, atol=1e-12)
    # delta at tap (0, 2) of a 3x3 filter with pad 1 == shift: y[h,w] = x[h-1, w+1]  (no kernel flip)
    wd = np.zeros((1, 1, 3, 3)); wd[0, 0, 0, 2] = 1.0
    y, _ = oracle.conv2d_fwd(x[:, :1], wd, None, (1, 1), 1)
    ref = np.zeros_like(x[:, :1]); ref[:, :, 1:, :-1] = x[:, :1, :-1, 1:]
    np.testing.assert_allclose(y, ref, atol=0)
    # all-ones 2x2 filter == box sum
    wo = np.ones((1, 1, 2, 2))
    y, _ = oracle.conv2d_fwd(x[:, :1], wo, None, (1, 1), 0)
    xs = x[:, :1]
    np.testing.assert_allclose(y, xs[:, :, :-1, :-1] + xs[:, :, 1:, :-1] + xs[:, :, :-1, 1:] + xs[:, :, 1:, 1:], rtol=1e-12)


def test_conv_output_dtype_and_single_rounding():
    rng = np.random.default_rng(24)
    x = rng.standard_normal((1, 8, 6, 6)).astype(np.float32)
    wt = rng.standard_normal((2, 8, 3, 3)).astype(np.float32)
    y, col = oracle.conv2d_fwd(x, wt, None, (1, 1), 1)
    assert y.dtype == np.float32 and col.dtype == np.float64
    y64 = oracle.conv2d_fwd_brute(x, wt, None, (1, 1), 1)
    np.testing.assert_array_equal(y, y64.astype(np.float32))     # fp64 sum rounded once


def test_im2col_col2im_are_adjoint():
    rng = np.random.default_rng(25)
    for (h, w, r, s, sh, sw, pad) in [(7, 6, 3, 3, 1, 1, 1), (8, 9, 3, 2, 2, 2, 1), (9, 9, 7, 7, 2, 2, 3)]:
        x = rng.standard_normal((2, 3, h, w))
        oh = oracle.out_size(h, r, sh, pad); ow = oracle.out_size(w, s, sw, pad)
        xp = np.pad(x, ((0, 0), (0, 0), (pad, pad), (pad, pad)))
        col = oracle.im2col(xp, oh, ow, r, s, (sh, sw))
        c = rng.standard_normal(col.shape)
        back = oracle.col2im(x.shape, pad, r, s, (sh, sw), c)
        assert abs(np.sum(col * c) - np.sum(x * back)) < 1e-9
        # explicit index formula for one entry
        n, o_h, o_w, ch, ky, kx = 1, oh - 1, ow // 2, 2, r - 1, 0
        assert col[(n * oh + o_h) * ow + o_w, (ch * r + ky) * s + kx] == xp[n, ch, o_h * sh + ky, o_w * sw + kx]


POOL_CASES = [  # n c h w k sh sw pad
    (2, 3, 7, 7, 3, 2, 2, 1),
    (1, 2, 8, 8, 2, 2, 2, 0),
    (1, 2, 9, 7, 3, 1, 1, 1),
    (2, 1, 5, 5, 3, 2, 2, 0),
    (1, 3, 6, 6, 2, 1, 2, 1),
    (1, 1, 9, 9, 3, 3, 3, 2),
]


@pytest.mark.parametrize("n,c,h,w,k,sh,sw,pad", POOL_CASES)
def test_pool_matches_brute_force_with_ties(n, c, h, w, k, sh, sw, pad):
    rng = np.random.default_rng(31)
    x = with_ties(rng, rng.standard_normal((n, c, h, w)).astype(np.float32), 0.3)
    x[0, 0, 0, :] = -np.abs(x[0, 0, 0, :])        # a negative border row: the zero pad cell must win there
    y, am = oracle.max_pool2d_fwd(x, k, (sh, sw), pad)
    yb, ib = oracle.max_pool2d_fwd_brute(x, k, (sh, sw), pad)
    assert y.dtype == np.float32
    np.testing.assert_array_equal(y, yb.astype(np.float32))
    np.testing.assert_array_equal(idx_ref_to_nchw(am, n, c, *y.shape[2:]), ib)
    dy = rng.standard_normal(y.shape).astype(np.float32)
    dx = oracle.max_pool2d_bwd(dy, am, x.shape, k, (sh, sw), pad, np.zeros_like(x))
    dxb = oracle.max_pool2d_bwd_brute(dy, ib, x.shape, k, (sh, sw), pad)
    np.testing.assert_array_equal(dx, dxb.astype(np.float32))


def test_pool_zero_border_participates_and_drops_gradient():
    x = -np.ones((1, 1, 4, 4), dtype=np.float32)
    y, am = oracle.max_pool2d_fwd(x, 3, 2, 1)
    # every window that touches the border sees a 0 > -1; window (1,1) covers rows/cols 1..3 only
    assert y[0, 0, 0, 0] == 0 and y[0, 0, 0, 1] == 0 and y[0, 0, 1, 0] == 0 and y[0, 0, 1, 1] == -1
    dx = oracle.max_pool2d_bwd(np.ones_like(y), am, x.shape, 3, (2, 2), 1, np.zeros_like(x))
    assert dx.sum() == 1.0          # only the interior window routes its gradient to a real cell


def test_pool_matches_torch_without_padding():
    torch = pytest.importorskip("torch")
    np.random.seed(0)   # tests/gradient_check/xs_pytorch/pooling.py:4-5, 18, 43
    n_x = np.random.randn(1, 3, 5, 5).astype(np.float32)
    tx = torch.tensor(n_x, requires_grad=True)
    ty = torch.nn.functional.max_pool2d(tx, 3, 2)
    g = torch.arange(ty.numel(), dtype=torch.float32).reshape(ty.shape) + 1
    ty.backward(g)
    y, am = oracle.max_pool2d_fwd(n_x, 3, 2, 0)
    dx = oracle.max_pool2d_bwd(g.numpy(), am, n_x.shape, 3, (2, 2), 0, np.zeros_like(n_x))
    np.testing.assert_array_equal(y, ty.detach().numpy())
    np.testing.assert_array_equal(dx, tx.grad.numpy())


def test_pool_mean_loss_invariant():
    # demos/examples/autograd.ipynb cells 14-16: 2x2/2 pool followed by mean() puts 1/(OH*OW) at each maximum
    rng = np.random.default_rng(33)
    x = rng.standard_normal((1, 1, 4, 4)).astype(np.float32)
    y, am = oracle.max_pool2d_fwd(x, 2, None, 0)
    dy = np.full(y.shape, 1.0 / y.size, dtype=np.float32)
    dx = oracle.max_pool2d_bwd(dy, am, x.shape, 2, (2, 2), 0, np.zeros_like(x))
    assert np.count_nonzero(dx) == 4 and np.all(dx[dx != 0] == 0.25)
    blocks = x.reshape(1, 1, 2, 2, 2, 2).transpose(0, 1, 2, 4, 3, 5).reshape(2, 2, 4)
    np.testing.assert_array_equal(y[0, 0], blocks.max(axis=2))


def test_pool_invariants_large():
    rng = np.random.default_rng(34)
    x = with_ties(rng, rng.standard_normal((2, 4, 32, 32)).astype(np.float32))
    y, am = oracle.max_pool2d_fwd(x, 3, 2, 1)
    assert am.min() >= 0 and am.max() < 9
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    idx = idx_ref_to_nchw(am, 2, 4, 16, 16)
    r, s = np.divmod(idx, 3)
    oh, ow = np.meshgrid(np.arange(16), np.arange(16), indexing="ij")
    picked = xp[np.arange(2)[:, None, None, None], np.arange(4)[None, :, None, None], 2 * oh + r, 2 * ow + s]
    np.testing.assert_array_equal(picked, y)
    assert np.all(y[:, :, 0, :] >= 0) and np.all(y[:, :, :, 0] >= 0)   # a pad cell is in those windows
    dy = rng.standard_normal(y.shape).astype(np.float32)
    dx = oracle.max_pool2d_bwd(dy, am, x.shape, 3, (2, 2), 1, np.zeros(x.shape, dtype=np.float64))
    on_pad = (2 * oh + r == 0) | (2 * ow + s == 0)
    assert abs(dx.sum() - dy[~on_pad].astype(np.float64).sum()) < 1e-9


def test_relu_mask_is_strict():
    pre = np.array([-1.0, -0.0, 0.0, 2.0], dtype=np.float32)
    np.testing.assert_array_equal(oracle.relu_fwd(pre), [0, 0, 0, 2])
    np.testing.assert_array_equal(oracle.relu_bwd(np.ones(4, dtype=np.float32), pre), [0, 1, 1, 1])


def test_golden_fixtures():
    path = os.path.join(os.path.dirname(__file__), "golden", "conv_pool_small.npz")
    g = np.load(path)
    stride = tuple(int(v) for v in g["conv_stride"]); pad = int(g["conv_pad"])
    y, col = oracle.conv2d_fwd(g["conv_x"], g["conv_w"], g["conv_b"], stride, pad)
    np.testing.assert_array_equal(y, g["conv_y"])
    dx, dw, db = oracle.conv2d_bwd(g["conv_dy"], g["conv_x"].shape, g["conv_w"], col, stride, pad,
                                   np.zeros_like(g["conv_x"]), np.zeros_like(g["conv_w"]), np.zeros_like(g["conv_b"]))
    np.testing.assert_array_equal(dx, g["conv_dx"]); np.testing.assert_array_equal(dw, g["conv_dw"])
    np.testing.assert_array_equal(db, g["conv_db"])
    k, ps, pp = int(g["pool_k"]), tuple(int(v) for v in g["pool_stride"]), int(g["pool_pad"])
    py, am = oracle.max_pool2d_fwd(g["pool_x"], k, ps, pp)
    np.testing.assert_array_equal(py, g["pool_y"])
    np.testing.assert_array_equal(idx_ref_to_nchw(am, *py.shape), g["pool_idx"])
    pdx = oracle.max_pool2d_bwd(g["pool_dy"], am, g["pool_x"].shape, k, ps, pp, np.zeros_like(g["pool_x"]))
    np.testing.assert_array_equal(pdx, g["pool_dx"])
