"""Device kernels next to the conv / pool path (batch norm, element-wise, reductions, dense GEMM, loss, SGD)
against plain NumPy float64 formulas of the reference's expressions.  Tolerances are for float32 kernels."""
import numpy as np
import pytest

from util import rel_l2

pytestmark = pytest.mark.gpu


# per channel up to 8192 elements: one kernel does both passes; beyond: partial sums + apply (float4 or scalar form)
@pytest.mark.parametrize("shape", [(4, 8, 6, 6), (32, 64, 14, 14), (5, 3, 7, 7), (2, 130, 9, 5), (64, 16),
                                   (8, 16, 40, 40), (6, 5, 37, 41), (32, 8, 16, 16), (33, 4, 16, 16),
                                   # single-kernel form: 2048 elements per channel (256 threads) and one more (1024),
                                   # its upper limit 8192 and one more (two-kernel form), planes wider than a workgroup
                                   (8, 3, 16, 16), (3, 5, 683), (2, 3, 64, 64), (1, 2, 8193), (3, 7, 20, 15), (256, 5)])
def test_batch_norm_forward_backward_and_moving_statistics(gpu, shape):
    """xs/nn/functional.py:676-707 and xs/nn/grad_fn.py:379-411."""
    K = gpu.kernels
    rng = np.random.default_rng(sum(shape))
    c = shape[1]
    x = (rng.standard_normal(shape) * 2 + 0.5).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, c).astype(np.float32); beta = rng.standard_normal(c).astype(np.float32)
    mm0 = rng.standard_normal(c).astype(np.float32); mv0 = rng.uniform(0.5, 2.0, c).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    axes = tuple(i for i in range(len(shape)) if i != 1)
    b = [1, -1] + [1] * (len(shape) - 2)
    x64 = x.astype(np.float64)
    mean = x64.mean(axis=axes); var = x64.var(axis=axes); eps = 1e-5
    sq = np.sqrt(var + eps)
    xhat = (x64 - mean.reshape(b)) / sq.reshape(b)
    y_ref = gamma.reshape(b) * xhat + beta.reshape(b)
    mm, mv = gpu.to_device(mm0), gpu.to_device(mv0)
    y, xh, sqv, mean_d, var_d = K.bn_fwd(gpu.to_device(x), gpu.to_device(gamma), gpu.to_device(beta), eps,
                                          moving=(mm, mv), momentum=0.9)
    assert rel_l2(y.numpy(), y_ref) <= 1e-5 and rel_l2(xh.numpy(), xhat) <= 1e-5
    np.testing.assert_allclose(mean_d.numpy(), mean, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(var_d.numpy(), var, rtol=1e-5)
    np.testing.assert_allclose(mm.numpy(), 0.9 * mm0 + 0.1 * mean, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(mv.numpy(), 0.9 * mv0 + 0.1 * var, rtol=1e-5)
    m = x.size // c
    dxh = dy.astype(np.float64) * gamma.reshape(b)
    dx_ref = (dxh * m - dxh.sum(axis=axes).reshape(b) - xhat * (dxh * xhat).sum(axis=axes).reshape(b)) / (m * sq.reshape(b))
    dx, dg, db = K.bn_bwd(gpu.to_device(dy), xh, sqv, gpu.to_device(gamma))
    assert rel_l2(dx.numpy(), dx_ref) <= 2e-5
    np.testing.assert_allclose(dg.numpy(), (dy * xhat).sum(axis=axes), rtol=2e-5, atol=1e-4)
    np.testing.assert_allclose(db.numpy(), dy.astype(np.float64).sum(axis=axes), rtol=2e-5, atol=1e-4)
    # fused ReLU: clipped output, strict mask, and a backward that ignores the clipped gradient entries
    mask = gpu.empty(shape, np.uint8)
    yr, xh2, sqv2, _, _ = K.bn_fwd(gpu.to_device(x), gpu.to_device(gamma), gpu.to_device(beta), eps, neg_mask=mask)
    np.testing.assert_array_equal(yr.numpy(), np.maximum(y.numpy(), 0))
    np.testing.assert_array_equal(mask.numpy(), (y.numpy() < 0).astype(np.uint8))
    dym = np.where(y.numpy() < 0, np.float32(0), dy)
    dx2, dg2, db2 = K.bn_bwd(gpu.to_device(dy), xh2, sqv2, gpu.to_device(gamma), neg_mask=mask)
    dx3, dg3, db3 = K.bn_bwd(gpu.to_device(dym), xh2, sqv2, gpu.to_device(gamma))
    np.testing.assert_array_equal(dx2.numpy(), dx3.numpy())
    np.testing.assert_array_equal(dg2.numpy(), dg3.numpy())
    np.testing.assert_array_equal(db2.numpy(), db3.numpy())
    # without the stored normalised input: the backward forms it again from x and the batch mean, same bits
    xd = gpu.to_device(x)
    y4, xh4, sqv4, mean4, _ = K.bn_fwd(xd, gpu.to_device(gamma), gpu.to_device(beta), eps, neg_mask=mask, want_xhat=False)
    assert xh4 is None
    np.testing.assert_array_equal(y4.numpy(), yr.numpy())
    dx4, dg4, db4 = K.bn_bwd(gpu.to_device(dy), xd, sqv4, gpu.to_device(gamma), neg_mask=mask, mean=mean4)
    np.testing.assert_array_equal(dx4.numpy(), dx2.numpy())
    np.testing.assert_array_equal(dg4.numpy(), dg2.numpy())
    np.testing.assert_array_equal(db4.numpy(), db2.numpy())
    # inference form with the given statistics (xs/nn/functional.py:708-725)
    yi = K.bn_infer(gpu.to_device(x), gpu.to_device(gamma), gpu.to_device(beta), gpu.to_device(mm0), gpu.to_device(mv0), eps)
    yi_ref = gamma.reshape(b) * (x64 - mm0.reshape(b)) / np.sqrt(mv0.reshape(b) + eps) + beta.reshape(b)
    assert rel_l2(yi.numpy(), yi_ref) <= 1e-5
    yir = K.bn_infer(gpu.to_device(x), gpu.to_device(gamma), gpu.to_device(beta), gpu.to_device(mm0), gpu.to_device(mv0), eps,
                     relu=True)
    np.testing.assert_array_equal(yir.numpy(), np.maximum(yi.numpy(), 0))


@pytest.mark.parametrize("shape", [(4, 8, 56, 56), (2, 3, 112, 112), (33, 5, 16, 20), (2, 4, 8, 12)])
def test_batch_norm_relu_max_pool_as_one_pass(gpu, shape):
    """The head of a ResNet: a held-back normalisation with its own ReLU followed by the 3x3 / stride 2 / pad 1 max-pool
    of its result runs as one normalisation whose second pass pools.  Pooled values, window indices, sign mask and
    statistics equal those of the separate passes bit for bit (same operations on the same values; the last shape is
    small enough for the separate normalisation to take its single-kernel form, whose sums are added in another order:
    compared to float32 accuracy there); the normalisation's own result is not stored and says so when read."""
    K = gpu.kernels
    rng = np.random.default_rng(sum(shape) + 2)
    n, c, h, w = shape
    x = (rng.standard_normal(shape) * 2 + 0.5).astype(np.float32)
    x[0, 0, :2, :4] = x[0, 0, 0, 0]                  # ties inside a window: the first maximum in window order wins
    gamma = rng.uniform(0.5, 1.5, c).astype(np.float32); beta = rng.standard_normal(c).astype(np.float32)
    mm0 = rng.standard_normal(c).astype(np.float32); mv0 = rng.uniform(0.5, 2.0, c).astype(np.float32)
    eps = 1e-5
    xd, gd, bd = gpu.to_device(x), gpu.to_device(gamma), gpu.to_device(beta)
    mm, mv = gpu.to_device(mm0), gpu.to_device(mv0)
    mask = gpu.empty(shape, np.uint8)
    y, _, sq, mean, var = K.bn_fwd(xd, gd, bd, eps, moving=(mm, mv), momentum=0.9, neg_mask=mask, want_xhat=False)
    p, i = K.maxpool2d_fwd(y, 3, (2, 2), 1)
    ref = [a.numpy() for a in (p, i, mask, sq, mean, var, mm, mv)]
    mm, mv = gpu.to_device(mm0), gpu.to_device(mv0)
    mask2 = gpu.empty(shape, np.uint8)
    y2, _, sq2, mean2, var2 = K.bn_fwd(xd, gd, bd, eps, moving=(mm, mv), momentum=0.9, neg_mask=mask2, want_xhat=False,
                                       defer=True)
    p2, i2 = K.maxpool2d_fwd(y2, 3, (2, 2), 1)
    got = [a.numpy() for a in (p2, i2, mask2, sq2, mean2, var2, mm, mv)]
    exact = n * h * w > 8192
    for g, e in zip(got, ref):
        if exact or g.dtype == np.uint8:
            np.testing.assert_array_equal(g, e)
        else:
            np.testing.assert_allclose(g, e, rtol=2e-6, atol=1e-6)
    with pytest.raises(gpu.XsmiError, match="not stored"):
        y2.numpy()
    # any other pool geometry, and any other call in between: the separate passes
    y3, _, _, _, _ = K.bn_fwd(xd, gd, bd, eps, neg_mask=mask2, want_xhat=False, defer=True)
    p3, _ = K.maxpool2d_fwd(y3, 2, (2, 2), 0)
    np.testing.assert_array_equal(y3.numpy(), y.numpy())
    np.testing.assert_array_equal(p3.numpy(), K.maxpool2d_fwd(y, 2, (2, 2), 0)[0].numpy())
    y4, _, _, _, _ = K.bn_fwd(xd, gd, bd, eps, neg_mask=mask2, want_xhat=False, defer=True)
    np.testing.assert_array_equal(y4.numpy(), y.numpy())
    np.testing.assert_array_equal(K.maxpool2d_fwd(y4, 3, (2, 2), 1)[0].numpy(), ref[0])


@pytest.mark.parametrize("shape", [(4, 8, 56, 56), (2, 3, 112, 112), (33, 5, 16, 20), (2, 4, 8, 12)])
def test_max_pool_gradient_inside_the_batch_norm_backward(gpu, shape):
    """The backward of the same chain: a held-back 3x3 / stride 2 / pad 1 max-pool gradient followed by the backward of
    the normalisation that fed the pool runs as that backward's two passes, which form the routed gradient themselves.
    The routed values are the pool kernel's own; the channel sums are added in another order, so dx, dgamma and dbeta
    agree with the separate passes to float32 rounding; the pool's gradient tensor is not stored and says so."""
    K = gpu.kernels
    rng = np.random.default_rng(sum(shape) + 3)
    n, c, h, w = shape
    x = (rng.standard_normal(shape) * 2 + 0.5).astype(np.float32)
    x[0, 0, :2, :4] = x[0, 0, 0, 0]
    gamma = rng.uniform(0.5, 1.5, c).astype(np.float32); beta = rng.standard_normal(c).astype(np.float32)
    xd, gd, bd = gpu.to_device(x), gpu.to_device(gamma), gpu.to_device(beta)
    mask = gpu.empty(shape, np.uint8)
    y, _, sq, mean, _ = K.bn_fwd(xd, gd, bd, 1e-5, neg_mask=mask, want_xhat=False)
    p, idx = K.maxpool2d_fwd(y, 3, (2, 2), 1)
    dp = gpu.to_device(rng.standard_normal(p.shape).astype(np.float32))
    g_sep = K.maxpool2d_bwd(dp, idx, shape, 3, (2, 2), 1)
    g_np = g_sep.numpy()                              # a read in between: the pool gradient is launched by itself
    dx_s, dg_s, db_s = K.bn_bwd(g_sep, xd, sq, gd, neg_mask=mask, mean=mean)
    g_fused = K.maxpool2d_bwd(dp, idx, shape, 3, (2, 2), 1)
    dx_f, dg_f, db_f = K.bn_bwd(g_fused, xd, sq, gd, neg_mask=mask, mean=mean)
    assert rel_l2(dx_f.numpy(), dx_s.numpy()) <= 1e-6
    np.testing.assert_allclose(dg_f.numpy(), dg_s.numpy(), rtol=2e-6, atol=1e-5)
    np.testing.assert_allclose(db_f.numpy(), db_s.numpy(), rtol=2e-6, atol=1e-5)
    with pytest.raises(gpu.XsmiError, match="not stored"):
        g_fused.numpy()
    # against float64 formulas on the routed gradient
    m = x.size // c
    b = [1, -1, 1, 1]
    d = np.where(mask.numpy() != 0, 0.0, g_np.astype(np.float64))
    xh = (x.astype(np.float64) - mean.numpy().astype(np.float64).reshape(b)) / sq.numpy().astype(np.float64).reshape(b)
    dxh = d * gamma.reshape(b)
    ref = (dxh * m - dxh.sum(axis=(0, 2, 3)).reshape(b) - xh * (dxh * xh).sum(axis=(0, 2, 3)).reshape(b)) / (m * sq.numpy().reshape(b))
    assert rel_l2(dx_f.numpy(), ref) <= 2e-5
    # the normalisation without the batch mean (stored normalised input) and a pool gradient that accumulates: separate
    g2 = K.maxpool2d_bwd(dp, idx, shape, 3, (2, 2), 1)
    xh32 = gpu.to_device(xh.astype(np.float32))
    dx2, _, _ = K.bn_bwd(g2, xh32, sq, gd, neg_mask=mask)
    np.testing.assert_array_equal(g2.numpy(), g_np)
    assert rel_l2(dx2.numpy(), ref) <= 2e-5


# two-kernel float4 form, two-kernel scalar form (planes not a multiple of four), single-kernel forms (256 / 1024 threads)
@pytest.mark.parametrize("shape", [(8, 16, 40, 40), (6, 5, 37, 41), (32, 64, 14, 14), (4, 8, 6, 6), (64, 16)])
def test_batch_norm_add_relu_as_one_pass(gpu, shape):
    """The end of a residual block: a held-back normalisation, the held-back add of its result and a shortcut, and the
    in-place ReLU of the sum run as one normalisation whose second pass adds and clips.  Same float operations as
    the three passes, hence the same bits; the normalisation's own result is never stored and says so when read; any
    other call in between makes the plain passes run."""
    K = gpu.kernels
    rng = np.random.default_rng(sum(shape) + 1)
    c = shape[1]
    x = (rng.standard_normal(shape) * 2 + 0.5).astype(np.float32)
    r = rng.standard_normal(shape).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, c).astype(np.float32); beta = rng.standard_normal(c).astype(np.float32)
    mm0 = rng.standard_normal(c).astype(np.float32); mv0 = rng.uniform(0.5, 2.0, c).astype(np.float32)
    eps = 1e-5
    xd, rd, gd, bd = gpu.to_device(x), gpu.to_device(r), gpu.to_device(gamma), gpu.to_device(beta)

    def three_passes():
        mm, mv = gpu.to_device(mm0), gpu.to_device(mv0)
        y, _, sq, mean, var = K.bn_fwd(xd, gd, bd, eps, moving=(mm, mv), momentum=0.9, want_xhat=False)
        s = K.add(y, rd)
        out, mask = K.relu_fwd_mask(s, s)
        return [a.numpy() for a in (out, mask, sq, mean, var, mm, mv)], y.numpy()

    ref, y_plain = three_passes()
    assert (ref[0] > 0).any() and (ref[1] == 1).any()
    for first in (True, False):                      # the normalisation's result as the add's first or second operand
        mm, mv = gpu.to_device(mm0), gpu.to_device(mv0)
        y, _, sq, mean, var = K.bn_fwd(xd, gd, bd, eps, moving=(mm, mv), momentum=0.9, want_xhat=False, defer=True)
        s = K.add(y, rd, defer=True) if first else K.add(rd, y, defer=True)
        out, mask = K.relu_fwd_mask(s, s)
        assert out is s
        got = [a.numpy() for a in (out, mask, sq, mean, var, mm, mv)]
        for g, e in zip(got, ref):
            np.testing.assert_array_equal(g, e)
        with pytest.raises(gpu.XsmiError, match="not stored"):
            y.numpy()
        # the same array as the output of the next normalisation is simply written again
        y2, _, _, _, _ = K.bn_fwd(xd, gd, bd, eps, y=y, want_xhat=False)
        assert y2 is y
        np.testing.assert_array_equal(y.numpy(), y_plain)
    # a read of the normalisation's result before the add, and a read of the sum before the ReLU: plain passes
    y, _, sq, mean, var = K.bn_fwd(xd, gd, bd, eps, want_xhat=False, defer=True)
    np.testing.assert_array_equal(y.numpy(), y_plain)
    s = K.add(y, rd, defer=True)
    np.testing.assert_array_equal(K.relu_fwd_mask(s, s)[0].numpy(), ref[0])
    y, _, sq, mean, var = K.bn_fwd(xd, gd, bd, eps, want_xhat=False, defer=True)
    s = K.add(y, rd, defer=True)
    np.testing.assert_array_equal(s.numpy(), y_plain + r)
    np.testing.assert_array_equal(y.numpy(), y_plain)
    np.testing.assert_array_equal(K.relu_fwd_mask(s, s)[0].numpy(), ref[0])
    np.testing.assert_array_equal(sq.numpy(), ref[2])



def test_multi_tensor_axpy_is_one_sgd_step(gpu):
    """xs/optim/sgd.py:4-9 over many parameters of ragged sizes, more than one launch group."""
    K = gpu.kernels
    rng = np.random.default_rng(2)
    sizes = [1, 3, 1023, 1024, 1025, 4097, 64 * 64 * 9] + [int(v) for v in rng.integers(1, 5000, size=60)]
    ps = [rng.standard_normal(n).astype(np.float32) for n in sizes]
    gs = [rng.standard_normal(n).astype(np.float32) for n in sizes]
    dp, dg = [gpu.to_device(p) for p in ps], [gpu.to_device(g) for g in gs]
    K.axpy_multi(dp, dg, -0.05)
    for p, g, d in zip(ps, gs, dp):
        # the kernel may fuse the multiply-add (one rounding instead of two)
        np.testing.assert_allclose(d.numpy(), p.astype(np.float64) - 0.05 * g.astype(np.float64), rtol=1e-6, atol=1e-7)
    K.axpy_multi([], [], 1.0)                       # nothing to do is fine
    with pytest.raises(ValueError):
        K.axpy_multi([dp[0]], [dg[1]], 1.0)


def test_dense_gemm_all_transposes(gpu):
    """addmm forward and the two gradient products (xs/nn/functional.py:99-120, xs/nn/grad_fn.py:86-99)."""
    K = gpu.kernels
    rng = np.random.default_rng(3)
    for (m, k, n) in ((32, 512, 1000), (7, 130, 33), (256, 64, 10), (1, 1, 1), (5, 1001, 3)):
        a = rng.standard_normal((m, k)).astype(np.float32); b = rng.standard_normal((k, n)).astype(np.float32)
        bias = rng.standard_normal(n).astype(np.float32); g = rng.standard_normal((m, n)).astype(np.float32)
        da, db_, dg = gpu.to_device(a), gpu.to_device(b), gpu.to_device(g)
        assert rel_l2(K.gemm(da, db_, bias=gpu.to_device(bias)).numpy(), a.astype(np.float64) @ b + bias) <= 1e-5
        assert rel_l2(K.gemm(dg, db_, trans_b=True).numpy(), g.astype(np.float64) @ b.T) <= 1e-5
        assert rel_l2(K.gemm(da, dg, trans_a=True).numpy(), a.T.astype(np.float64) @ g) <= 1e-5


@pytest.mark.parametrize("m,n", [(37, 100), (32, 1000), (3, 2500)])
def test_softmax_cross_entropy(gpu, m, n):
    """xs/nn/functional.py:984-1010 and xs/nn/grad_fn.py:604-620; rows longer than what a workgroup keeps in
    registers (2048 classes) take the second form of the loops."""
    K = gpu.kernels
    rng = np.random.default_rng(4 + n)
    logits = (rng.standard_normal((m, n)) * 3).astype(np.float32); labels = rng.integers(0, n, size=m)
    z = logits.astype(np.float64); z -= z.max(axis=1, keepdims=True)
    sm = np.exp(z); sm /= sm.sum(axis=1, keepdims=True)
    for reduction in ("mean", "sum"):
        dl = gpu.to_device(labels.astype(np.int64), np.int64)
        loss, smd = K.softmax_ce_fwd(gpu.to_device(logits), dl, reduction)
        assert rel_l2(smd.numpy(), sm) <= 1e-6
        ref = -np.log(sm[np.arange(m), labels])
        ref = ref.mean() if reduction == "mean" else ref.sum()
        assert abs(float(np.asarray(loss.numpy()).reshape(-1)[0]) - ref) <= 1e-5 * abs(ref)
        g = K.softmax_ce_bwd(smd, dl, reduction, 1.0).numpy()
        gref = sm.copy(); gref[np.arange(m), labels] -= 1.0
        if reduction == "mean":
            gref /= m
        assert rel_l2(g, gref) <= 1e-5
        up = gpu.to_device(np.array([0.5], np.float32))          # the loss's own gradient read on the device
        g2 = K.softmax_ce_bwd(smd, dl, reduction, up).numpy()
        assert rel_l2(g2, 0.5 * gref) <= 1e-5


def test_held_back_add_joins_the_in_place_relu(gpu):
    """kernels.add(defer=True) launches nothing until the next library call: an in-place ReLU of the result runs
    as one add+ReLU pass, anything else (a read, a write to an operand, another add) sees the plain sum."""
    from xshinnosuke_amd.backend import capi
    K = gpu.kernels
    rng = np.random.default_rng(12)
    a = rng.standard_normal((3, 5, 7, 9)).astype(np.float32)
    b = rng.standard_normal((3, 5, 7, 9)).astype(np.float32)
    da, db = gpu.to_device(a), gpu.to_device(b)
    c = K.add(da, db, defer=True)
    assert capi._deferred and capi._deferred[0][-1] is c
    r = K.relu_fwd(c, out=c)
    assert r is c and not capi._deferred
    np.testing.assert_array_equal(c.numpy(), np.maximum(a + b, 0.0))
    c = K.add(da, db, defer=True)
    np.testing.assert_array_equal(c.numpy(), a + b)                 # a read enqueues the add first
    c = K.add(da, db, defer=True)
    da.fill_zero()                                                   # so does a write to an operand
    np.testing.assert_array_equal(c.numpy(), a + b)
    np.testing.assert_array_equal(da.numpy(), np.zeros_like(a))
    da.set(a)
    c1 = K.add(da, db, defer=True)
    c2 = K.add(c1, db, defer=True)                                   # and another held-back add
    other = gpu.to_device(a)
    K.relu_fwd(other, out=other)                                     # an in-place ReLU of something else
    assert not capi._deferred
    np.testing.assert_array_equal(c2.numpy(), (a + b) + b)
    np.testing.assert_array_equal(other.numpy(), np.maximum(a, 0.0))
    # through the tensor API: no_grad residual add + in-place ReLU layer
    import xshinnosuke_amd as xs
    from xshinnosuke_amd.layers import ReLU
    ta, tb = xs.tensor(a).to('cuda'), xs.tensor(b).to('cuda')
    with xs.no_grad():
        out = ta + tb
        out = ReLU(inplace=True)(out)
    np.testing.assert_array_equal(out.numpy(), np.maximum(a + b, 0.0))
    out2 = ta + tb                                                   # gradients tracked or not: same values
    np.testing.assert_array_equal(out2.numpy(), a + b)
    # tracked: the fused pass also delivers the ReLU's sign mask, and the gradient reaches both operands masked
    ta.requires_grad = True; tb.requires_grad = True
    out3 = ReLU(inplace=True)(ta + tb)
    np.testing.assert_array_equal(out3.numpy(), np.maximum(a + b, 0.0))
    out3.backward(xs.tensor(np.ones_like(a)).to('cuda'))
    expect = ((a + b) >= 0).astype(np.float32)
    np.testing.assert_array_equal(ta.grad.numpy(), expect)
    np.testing.assert_array_equal(tb.grad.numpy(), expect)
    # a second sweep adds into the gradients that are already there
    g2 = rng.standard_normal(a.shape).astype(np.float32)
    out4 = ReLU(inplace=True)(ta + tb)
    out4.backward(xs.tensor(g2).to('cuda'))
    np.testing.assert_array_equal(ta.grad.numpy(), expect + g2 * expect)
    np.testing.assert_array_equal(tb.grad.numpy(), expect + g2 * expect)


def test_masked_gradient_into_two_tensors(gpu):
    """xsmi_relu_mask_bwd2 against two single calls, overwrite and accumulate, with a ragged tail."""
    K = gpu.kernels
    rng = np.random.default_rng(21)
    n = 4 * 1000 + 3
    dy = rng.standard_normal(n).astype(np.float32)
    mask = (rng.random(n) < 0.4).astype(np.uint8)
    o1, o2 = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    ddy, dm = gpu.to_device(dy), gpu.to_device(mask)
    for acc in (False, True):
        d1, d2 = gpu.to_device(o1), gpu.to_device(o2)
        K.relu_mask_bwd2(ddy, dm, d1, d2, accumulate=acc)
        e1, e2 = gpu.to_device(o1), gpu.to_device(o2)
        K.relu_mask_bwd(ddy, dm, dx=e1, accumulate=acc)
        K.relu_mask_bwd(ddy, dm, dx=e2, accumulate=acc)
        np.testing.assert_array_equal(d1.numpy(), e1.numpy())
        np.testing.assert_array_equal(d2.numpy(), e2.numpy())
        np.testing.assert_array_equal(d1.numpy(), (o1 if acc else 0) + np.where(mask != 0, np.float32(0), dy))


@pytest.mark.parametrize("n,c,h,w,k,sh,sw", [(2, 3, 9, 11, 3, 2, 2), (1, 5, 8, 8, 2, 1, 1), (3, 2, 12, 10, 3, 4, 5),
                                             (2, 4, 7, 7, 5, 1, 2)])
def test_average_pool_with_overlapping_or_sparse_windows(gpu, n, c, h, w, k, sh, sw):
    """The im2col mode of avg_pool2d with stride != window (xs/nn/functional.py:563-571) and its gradient through the
    float64 col2im (xs/nn/grad_fn.py:296-307): per-window share dy / k^2 in float32, sums in float64, one rounding."""
    K = gpu.kernels
    rng = np.random.default_rng(11 * h + w + k + sh)
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    oh, ow = (h - k) // sh + 1, (w - k) // sw + 1
    ref = np.zeros((n, c, oh, ow))
    for i in range(oh):
        for j in range(ow):
            ref[:, :, i, j] = x[:, :, i * sh:i * sh + k, j * sw:j * sw + k].astype(np.float64).mean(axis=(2, 3))
    y = K.avgpool_fwd(gpu.to_device(x), k, (sh, sw)).numpy()
    assert y.shape == (n, c, oh, ow)
    np.testing.assert_allclose(y, ref, rtol=1e-6, atol=1e-7)
    dy = rng.standard_normal((n, c, oh, ow)).astype(np.float32)
    share = (dy / np.float32(k * k)).astype(np.float64)
    dref = np.zeros(x.shape)
    for i in range(oh):
        for j in range(ow):
            dref[:, :, i * sh:i * sh + k, j * sw:j * sw + k] += share[:, :, i:i + 1, j:j + 1]
    dx = K.avgpool_bwd(gpu.to_device(dy), x.shape, k, (sh, sw)).numpy()
    np.testing.assert_allclose(dx, dref.astype(np.float32), rtol=1e-6, atol=1e-7)
    # the host path of the functional op agrees with the device path
    import xshinnosuke_amd as xs
    t = xs.tensor(x, requires_grad=True)
    out = xs.nn.functional.avg_pool2d(t, k, (sh, sw))
    np.testing.assert_allclose(out.eval, ref, rtol=1e-6, atol=1e-7)
    out.backward(xs.tensor(dy))
    np.testing.assert_allclose(t.grad.eval, dref.astype(np.float32), rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("n,c,h,w,k", [(3, 5, 6, 6, 2), (4, 70, 7, 7, 7), (2, 3, 7, 8, 3), (1, 2, 13, 13, 13)])
def test_average_pool_blocks(gpu, n, c, h, w, k):
    """Mean over non-overlapping k x k blocks and its gradient (xs/nn/functional.py:539-583,
    xs/nn/grad_fn.py:284-309); k == H == W is the global pool in front of ResNet's dense layer."""
    K = gpu.kernels
    rng = np.random.default_rng(n + c + h + k)
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    oh, ow = h // k, w // k
    ref = x[:, :, :oh * k, :ow * k].astype(np.float64).reshape(n, c, oh, k, ow, k).mean(axis=(3, 5))
    y = K.avgpool_fwd(gpu.to_device(x), k).numpy()
    assert y.shape == (n, c, oh, ow)
    np.testing.assert_allclose(y, ref, rtol=1e-6, atol=1e-7)
    dy = rng.standard_normal((n, c, oh, ow)).astype(np.float32)
    dx = K.avgpool_bwd(gpu.to_device(dy), x.shape, k).numpy()
    dref = np.zeros_like(x)
    dref[:, :, :oh * k, :ow * k] = np.repeat(np.repeat(dy, k, axis=2), k, axis=3) / np.float32(k * k)
    np.testing.assert_allclose(dx, dref, rtol=1e-6, atol=0)


@pytest.mark.parametrize("kind", ["sigmoid", "tanh"])
@pytest.mark.parametrize("n", [1, 7, 4096, 100003])
def test_sigmoid_and_tanh_kernels(gpu, kind, n):
    """xs/nn/td_functional.py:63-70 and xs/nn/grad_fn.py:161-170, float32 kernels against float64 formulas."""
    K = gpu.kernels
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * 3).astype(np.float32)
    dy = rng.standard_normal(n).astype(np.float32)
    x64 = x.astype(np.float64)
    y_ref = 1 / (1 + np.exp(-x64)) if kind == "sigmoid" else np.tanh(x64)
    y = K.act_fwd(gpu.to_device(x), kind)
    np.testing.assert_allclose(y.numpy(), y_ref, rtol=2e-6, atol=1e-7)
    y32 = y.numpy().astype(np.float64)
    dx_ref = dy * y32 * (1 - y32) if kind == "sigmoid" else dy * (1 - y32 * y32)
    dx = K.act_bwd(gpu.to_device(dy), y, kind)
    np.testing.assert_allclose(dx.numpy(), dx_ref, rtol=2e-6, atol=1e-7)


def test_conv2d_layer_with_a_named_activation(gpu):
    """Conv2D(activation='tanh' | 'sigmoid') appends the named activation to the convolution (reference
    xs/layers/convolutional.py:16,76-77): values and gradients of a dynamic forward / backward on the device
    against the oracle convolution followed by the closed form."""
    import oracle
    import xshinnosuke_amd as xs
    from xshinnosuke_amd.layers import Conv2D
    rng = np.random.default_rng(77)
    x = rng.standard_normal((3, 4, 9, 9)).astype(np.float32)
    up = rng.standard_normal((3, 6, 9, 9)).astype(np.float32)
    try:
        for name in ("tanh", "sigmoid"):
            xs.GLOBAL.INPUTS = None
            xs.GLOBAL.USE_CUDA = True
            layer = Conv2D(6, 3, padding=1, activation=name)
            xt = xs.tensor(x, requires_grad=True).to('cuda')
            xt.retain_grad(True)
            out = layer(xt)
            w, b = (p.numpy() for p in layer.parameters())
            pre, col = oracle.conv2d_fwd(x, w.astype(np.float32), b.reshape(-1).astype(np.float32), (1, 1), 1)
            act = np.tanh(pre.astype(np.float64)) if name == "tanh" else 1 / (1 + np.exp(-pre.astype(np.float64)))
            assert out.device == 'cuda' and rel_l2(out.numpy(), act) <= 1e-5
            assert layer.data is out
            out.backward(xs.tensor(up).to('cuda'))
            dpre = up * ((1 - act ** 2) if name == "tanh" else act * (1 - act))
            dx, dw, db = oracle.conv2d_bwd(dpre.astype(np.float32), x.shape, w.astype(np.float32), col, (1, 1), 1,
                                           np.zeros_like(x), np.zeros(w.shape, np.float32), np.zeros(6, np.float32))
            assert rel_l2(xt.grad.numpy(), dx) <= 1e-5
            assert rel_l2(layer.parameters()[0].grad.numpy(), dw) <= 1e-5
            assert rel_l2(layer.parameters()[1].grad.numpy().reshape(-1), db) <= 1e-5
    finally:
        xs.GLOBAL.INPUTS = None
        xs.GLOBAL.USE_CUDA = False
