"""ResNet-18 at the benchmark sizes against the oracle.

Training configuration: N=32x3x224x224 fp32, one forward + backward + SGD step through the layer API with the
operands of every convolution and of the max-pool recorded at the backend's array-level entry points.  Convolutions
and pooling act on each image independently, so a two-image slice of the batch is checked against the oracle
(float64 GEMM, one rounding) at rel-L2 <= 1e-5; the weight gradient sums over the whole batch and is checked
against a float64 per-tap product of the full operands.  The 7x7 / 2 stem runs here at M = 401 408 pixels.

Inference configuration: N=256x3x224x224 with moving-statistics batch norm; images are then independent, and
the logits of four of them are compared with a NumPy/oracle forward of those four (bf16 <= 1e-2, fp32 <= 1e-4).
"""
import numpy as np
import pytest

import oracle
import xshinnosuke_amd as xs
from xshinnosuke_amd.backend import kernels as K
from xshinnosuke_amd.optim import SGD
from resnet18 import ResNet18
from test_gpu_resnet import _oracle_forward
from util import rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-5
SLICE = 2


@pytest.fixture(autouse=True)
def _fresh_state(gpu):
    xs.GLOBAL.INPUTS = None
    xs.GLOBAL.USE_CUDA = False
    xs.GLOBAL.TRAINING = True
    yield
    xs.GLOBAL.INPUTS = None
    xs.GLOBAL.USE_CUDA = False
    xs.GLOBAL.TRAINING = True
    gpu.release_cached_memory()


def _head(a, n=SLICE):
    """The first and the last `n` images of a batch (0, 1, 30, 31 of 32): the last ones sit in the tail of every
    kernel's pixel range, where ragged tiles and the ends of split reductions are."""
    total = a.shape[0]
    return np.concatenate([a[0:n].numpy(), a[total - n:total].numpy()])


def _ends(a, n=SLICE):
    return np.concatenate([a[:n], a[-n:]])


def _before(a, n=None):
    """Contents an accumulating kernel will add to: zeros while the buffer's clear is still pending."""
    if a is None:
        return None
    if a.is_fresh():
        shape = a.shape if n is None else (2 * n,) + tuple(a.shape[1:])
        return np.zeros(shape, np.float32)
    return a.numpy() if n is None else _head(a, n)


class _Recorder:
    """Wraps the array-level conv / pool entry points and copies their operands to the host."""

    def __init__(self, monkeypatch):
        self.fwd, self.bwd, self.pool_fwd, self.pool_bwd = [], [], [], []
        real_fwd, real_bwd, real_bww = K.conv2d_fwd, K.conv2d_bwd, K.conv2d_bwd_weight
        real_pf, real_pb = K.maxpool2d_fwd, K.maxpool2d_bwd

        def conv2d_fwd(x, w, bias=None, stride=(1, 1), pad=0, **kw):
            out = real_fwd(x, w, bias, stride, pad, **kw)
            self.fwd.append(dict(x=_head(x), w=w.numpy(), b=None if bias is None else bias.numpy().reshape(-1),
                                 y=_head(out), stride=tuple(stride), pad=pad, w_id=w.address()))
            return out

        def conv2d_bwd(dy, x, w, dx, dw, db=None, stride=(1, 1), pad=0, **kw):
            rec = dict(dy=dy.numpy(), x=x.numpy(), w=w.numpy(), stride=tuple(stride), pad=pad, w_id=w.address(),
                       dx0=_before(dx, SLICE), dw0=_before(dw), db0=_before(db))
            res = real_bwd(dy, x, w, dx, dw, db, stride, pad, **kw)
            rec.update(dx=_head(dx), dw=dw.numpy(), db=None if db is None else db.numpy().reshape(-1))
            self.bwd.append(rec)
            return res

        def conv2d_bwd_weight(dy, x, w_shape, stride=(1, 1), pad=0, dw=None, db=None, **kw):
            rec = dict(dy=dy.numpy(), x=x.numpy(), w=None, stride=tuple(stride), pad=pad, w_id=None, dx0=None,
                       dw0=_before(dw), db0=_before(db))
            dw_, db_ = real_bww(dy, x, w_shape, stride, pad, dw=dw, db=db, **kw)
            rec.update(dx=None, dw=dw_.numpy(), db=None if db_ is None else db_.numpy().reshape(-1))
            self.bwd.append(rec)
            return dw_, db_

        def maxpool2d_fwd(x, k, stride, pad=0, **kw):
            out, idx = real_pf(x, k, stride, pad, **kw)
            self.pool_fwd.append(dict(x=_head(x), y=_head(out), idx=_head(idx), k=k, stride=tuple(stride), pad=pad))
            return out, idx

        def maxpool2d_bwd(dy, idx, x_shape, k, stride, pad=0, dx=None, accumulate=False):
            rec = dict(dy=_head(dy), idx=_head(idx), k=k, stride=tuple(stride), pad=pad,
                       dx0=_before(dx, SLICE) if (dx is not None and accumulate) else None)
            out = real_pb(dy, idx, x_shape, k, stride, pad, dx=dx, accumulate=accumulate)
            rec.update(dx=_head(out))
            self.pool_bwd.append(rec)
            return out

        for name, fn in (("conv2d_fwd", conv2d_fwd), ("conv2d_bwd", conv2d_bwd), ("conv2d_bwd_weight", conv2d_bwd_weight),
                         ("maxpool2d_fwd", maxpool2d_fwd), ("maxpool2d_bwd", maxpool2d_bwd)):
            monkeypatch.setattr(K, name, fn)


def _dw_float64(dy, x, w_shape, stride, pad):
    """dw[k,c,r,s] = sum_{n,oh,ow} dy[n,k,oh,ow] * xpad[n,c,oh*sh+r,ow*sw+s] in float64: the reference's
    dot(grad, col) (xs/nn/grad_fn.py:191-194) tap by tap, without the unfolded matrix."""
    k, c, kh, kw = w_shape
    sh, sw = stride
    n, _, oh, ow = dy.shape
    xp = np.pad(x, ((0, 0), (0, 0), (pad, pad), (pad, pad)))
    g = dy.astype(np.float64).transpose(1, 0, 2, 3).reshape(k, -1)
    ref = np.empty((k, c, kh, kw))
    for r in range(kh):
        for s in range(kw):
            win = xp[:, :, r:r + sh * oh:sh, s:s + sw * ow:sw].astype(np.float64).transpose(1, 0, 2, 3).reshape(c, -1)
            ref[:, :, r, s] = g @ win.T
    return ref


def test_resnet18_training_step_at_full_size_against_oracle(gpu, monkeypatch):
    np.random.seed(6)
    x = xs.tensor(np.random.default_rng(6).standard_normal((32, 3, 224, 224), dtype=np.float32)).to('cuda')
    y = xs.tensor(np.random.default_rng(7).integers(0, 1000, size=(32,))).to('cuda')
    net = ResNet18(classes=1000, pool=7).to('cuda')
    crit = xs.nn.CrossEntropyLoss()
    with xs.no_grad():
        net(x)                                   # creates the parameters
    xs.GLOBAL.INPUTS = None
    params = list(net.parameters())
    assert len(params) == 82
    opt = SGD(params, lr=0.01)
    before = {id(p): p.numpy().copy() for p in params}

    rec = _Recorder(monkeypatch)
    opt.zero_grad()
    loss = crit(net(x), y)
    loss.backward()
    monkeypatch.undo()
    grads = {id(p): p.grad.numpy().copy() for p in params}
    opt.step()
    assert np.isfinite(loss.item())

    # ---- forward: the 20 convolutions and the max-pool on the first two and the last two images ----
    assert len(rec.fwd) == 20 and len(rec.bwd) == 20 and len(rec.pool_fwd) == 1 and len(rec.pool_bwd) == 1
    geoms = set()
    for f in rec.fwd:
        y_ref, _ = oracle.conv2d_fwd(f['x'], f['w'], f['b'], f['stride'], f['pad'], keep_col=False)
        assert rel_l2(f['y'], y_ref) <= TOL, (f['x'].shape, f['w'].shape, rel_l2(f['y'], y_ref))
        geoms.add((f['x'].shape[1:], f['w'].shape, f['stride'], f['pad']))
    assert len(geoms) == 11                      # the distinct conv geometries of ResNet-18
    assert rec.fwd[0]['x'].shape[1:] == (3, 224, 224) and rec.fwd[0]['w'].shape == (64, 3, 7, 7)
    pf = rec.pool_fwd[0]
    assert pf['x'].shape[1:] == (64, 112, 112) and (pf['k'], pf['stride'], pf['pad']) == (3, (2, 2), 1)
    py_ref, am = oracle.max_pool2d_fwd(pf['x'], pf['k'], pf['stride'], pf['pad'])
    assert pf['y'].tobytes() == py_ref.tobytes()
    assert np.array_equal(pf['idx'].transpose(0, 2, 3, 1).reshape(-1), am)

    # ---- backward ----
    pb = rec.pool_bwd[0]
    dx0 = pb['dx0'] if pb['dx0'] is not None else np.zeros(pf['x'].shape, np.float32)
    pdx_ref = oracle.max_pool2d_bwd(pb['dy'], am, pf['x'].shape, pb['k'], pb['stride'], pb['pad'], dx0.copy())
    assert pb['dx'].tobytes() == pdx_ref.tobytes()

    seen_stem = False
    for b in rec.bwd:
        n, c, h, w = b['x'].shape
        k = b['dy'].shape[1]
        w_shape = b['dw'].shape
        assert np.all(b['dw0'] == 0) and (b['db0'] is None or np.all(b['db0'] == 0))    # fresh after zero_grad
        dw_ref = _dw_float64(b['dy'], b['x'], w_shape, b['stride'], b['pad'])
        assert rel_l2(b['dw'], dw_ref) <= TOL, (b['x'].shape, w_shape, rel_l2(b['dw'], dw_ref))
        if b['db'] is not None:
            # every conv feeds a batch norm, so the true bias gradient is ~0: measure the error against the
            # size of the summands (the bound of a float32 sum), not against the sum
            db_ref = b['dy'].astype(np.float64).sum(axis=(0, 2, 3))
            scale = np.abs(b['dy']).astype(np.float64).sum(axis=(0, 2, 3))
            assert np.max(np.abs(b['db'] - db_ref) / scale) <= TOL
        if b['dx'] is None:
            assert (c, w_shape[2]) == (3, 7)     # only the stem has an input without a gradient
            seen_stem = True
            continue
        dx_ref, _, _ = oracle.conv2d_bwd(_ends(b['dy']), (2 * SLICE, c, h, w), b['w'], None, b['stride'], b['pad'],
                                         b['dx0'].copy(), None, None)
        assert rel_l2(b['dx'], dx_ref) <= TOL, (b['x'].shape, w_shape, rel_l2(b['dx'], dx_ref))
    assert seen_stem

    # ---- SGD: w <- w - lr * grad, every parameter moved by exactly that ----
    moved = 0
    for p in params:
        want = before[id(p)] - np.float32(0.01) * grads[id(p)]
        got = p.numpy()
        assert np.allclose(got, want, rtol=1e-6, atol=1e-8)
        moved += int(not np.array_equal(got, before[id(p)]))
    assert moved >= 60


def test_resnet18_inference_at_full_batch_against_oracle(gpu):
    """N=256x3x224x224, forward only, moving-statistics batch norm (images independent): the logits of the first
    and last two images against the NumPy/oracle forward of those four images."""
    np.random.seed(7)
    X = np.random.default_rng(7).standard_normal((256, 3, 224, 224), dtype=np.float32)
    pick = [0, 1, 254, 255]
    net = ResNet18(classes=1000, pool=7).to('cuda')
    with xs.no_grad():
        net(xs.tensor(X[:2]).to('cuda'))          # creates the parameters
    xs.GLOBAL.INPUTS = None
    rng = np.random.default_rng(3)

    def walk(layer):
        if type(layer).__name__ == 'BatchNormalization':
            layer.moving_mean.eval = (0.1 * rng.standard_normal(layer.moving_mean.shape)).astype(np.float32)
            layer.moving_variance.eval = rng.uniform(0.5, 1.5, layer.moving_variance.shape).astype(np.float32)
        for sub in getattr(layer, '_graph', []):
            walk(sub)
        if type(layer).__name__ == 'BasicBlock':
            walk(layer.conv1)
            walk(layer.shortcut)
    walk(net.conv1)
    for stage in (net.layer1, net.layer2, net.layer3, net.layer4):
        walk(stage)
    ref = _oracle_forward(net, X[pick])
    xd = xs.tensor(X).to('cuda')
    xs.GLOBAL.TRAINING = False
    with xs.no_grad():
        y32 = net(xd).numpy()
        xs.GLOBAL.INPUTS = None
        with xs.conv_precision('bf16'):
            y16 = net(xd).numpy()
    assert y32.shape == (256, 1000)
    assert rel_l2(y32[pick], ref) <= 1e-4
    assert rel_l2(y16[pick], ref) <= 1e-2
    assert rel_l2(y16, y32) > 1e-5                # the bf16 kernels really ran
