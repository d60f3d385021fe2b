"""ResNet-18 through the unchanged layer API: device-resident tensors against host tensors (whose
non-conv ops run in NumPy), and parameter discovery."""
import numpy as np
import pytest

import xshinnosuke_amd as xs
from resnet18 import ResNet18, oracle_forward as _oracle_forward, named_params as _named_params
from xshinnosuke_amd.optim import SGD
from util import rel_l2

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _fresh_state(gpu):
    xs.GLOBAL.INPUTS = None
    xs.GLOBAL.USE_CUDA = False
    xs.GLOBAL.TRAINING = True
    yield
    xs.GLOBAL.INPUTS = None
    xs.GLOBAL.USE_CUDA = False


def test_resnet18_device_path_matches_host_path():
    np.random.seed(0)
    X = np.random.randn(4, 3, 64, 64).astype(np.float32)
    Y = np.random.randint(0, 10, (4,))
    host = ResNet18(classes=10, pool=2)
    out_h = host(xs.tensor(X))
    assert len(host.parameters()) == 62 + 20      # 20 convs x (w, b) + 20 BNs x (gamma, beta) + FC (w, b) = 82
    loss_h = xs.nn.CrossEntropyLoss()(out_h, xs.tensor(Y))
    loss_h.backward()
    params_h = _named_params(host)
    assert len(params_h) == 82

    dev = ResNet18(classes=10, pool=2).to('cuda')
    xd = xs.tensor(X).to('cuda')
    dev(xd)                                       # creates the parameters (on the device)
    xs.GLOBAL.INPUTS = None
    params_d = _named_params(dev)
    for pd, ph in zip(params_d, params_h):
        assert pd.device == 'cuda' and pd.shape == ph.shape
        pd.eval = ph.numpy().astype(np.float32)
        if pd.grad is not None:
            pd.grad.zero_()
    out_d = dev(xs.tensor(X).to('cuda'))
    assert out_d.device == 'cuda'
    assert rel_l2(out_d.numpy(), out_h.numpy()) <= 2e-4
    loss_d = xs.nn.CrossEntropyLoss()(out_d, xs.tensor(Y).to('cuda'))
    assert abs(loss_d.item() - loss_h.item()) <= 2e-4 * abs(loss_h.item())
    loss_d.backward()
    for pd, ph in zip(params_d, params_h):
        g_h, g_d = ph.grad.numpy().astype(np.float64), pd.grad.numpy().astype(np.float64)
        # conv biases in front of a batch norm have an analytically zero gradient (both paths give ~1e-7 noise),
        # hence the absolute term
        assert np.linalg.norm(g_d - g_h) <= 1e-4 * np.linalg.norm(g_h) + 1e-5, (ph.shape, rel_l2(g_d, g_h))
    # one SGD step on the device changes the parameters and keeps everything finite
    before = params_d[0].numpy().copy()
    SGD(dev.parameters(), lr=0.01).step()
    after = params_d[0].numpy()
    assert np.isfinite(after).all() and not np.array_equal(before, after)


def test_resnet18_trains_on_device():
    np.random.seed(1)
    X = np.random.randn(8, 3, 32, 32).astype(np.float32)
    Y = np.random.randint(0, 4, (8,))
    net = ResNet18(classes=4, pool=1).to('cuda')
    crit = xs.nn.CrossEntropyLoss()
    x, y = xs.tensor(X).to('cuda'), xs.tensor(Y).to('cuda')
    net(x)
    xs.GLOBAL.INPUTS = None
    opt = SGD(net.parameters(), lr=0.05)
    losses = []
    for _ in range(6):
        opt.zero_grad()
        loss = crit(net(x), y)
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert np.isfinite(losses).all() and losses[-1] < losses[0]


def test_resnet18_steps_do_not_depend_on_the_weight_gradient_overlap(monkeypatch):
    """Conv layers leave their weight gradients running on the backend's second stream across the backward sweep.
    Three SGD steps with that overlap and three with every weight gradient joined at once end in the same bits."""
    from xshinnosuke_amd.backend import kernels as K

    def run(overlap):
        if not overlap:
            plain = K.conv2d_bwd
            monkeypatch.setattr(K, "conv2d_bwd", lambda *a, **kw: plain(*a, **dict(kw, async_dw=False)))
        np.random.seed(3)
        X = np.random.randn(8, 3, 64, 64).astype(np.float32)
        Y = np.random.randint(0, 10, (8,))
        net = ResNet18(classes=10, pool=2).to('cuda')
        x, y = xs.tensor(X).to('cuda'), xs.tensor(Y).to('cuda')
        net(x)
        xs.GLOBAL.INPUTS = None
        opt = SGD(net.parameters(), lr=0.05)
        crit = xs.nn.CrossEntropyLoss()
        losses = []
        for _ in range(3):
            opt.zero_grad()
            loss = crit(net(x), y)
            loss.backward()
            opt.step()
            losses.append(loss.item())
        out = [p.numpy().copy() for p in _named_params(net)]
        monkeypatch.undo()
        xs.GLOBAL.INPUTS = None
        return losses, out

    la, pa = run(True)
    lb, pb = run(False)
    assert la == lb
    for u, v in zip(pa, pb):
        np.testing.assert_array_equal(u, v)


def test_resnet18_steps_do_not_depend_on_filter_layouts_made_ahead(monkeypatch):
    """After each optimizer step the backend lays every filter out again on its second stream and the next
    step's convolutions skip their own layout launch.  Five SGD steps with that and five without end in the same
    bits, also when a filter is overwritten from the host between two steps (its layout made ahead is then stale
    and must not be used) and when the batch size changes for one step."""
    from xshinnosuke_amd.backend import kernels as K, capi

    def run(ahead, lanes=None):
        monkeypatch.setattr(K, "_PREPACK", ahead)
        if lanes is not None:
            be.set_option("pack_lanes", lanes)
        np.random.seed(4)
        X = np.random.randn(8, 3, 64, 64).astype(np.float32)
        Y = np.random.randint(0, 10, (8,))
        net = ResNet18(classes=10, pool=2).to('cuda')
        x, y = xs.tensor(X).to('cuda'), xs.tensor(Y).to('cuda')
        x6, y6 = xs.tensor(X[:6]).to('cuda'), xs.tensor(Y[:6]).to('cuda')
        net(x)
        xs.GLOBAL.INPUTS = None
        opt = SGD(net.parameters(), lr=0.05)
        crit = xs.nn.CrossEntropyLoss()
        params = _named_params(net)
        flags = []
        real = capi.lib.call
        monkeypatch.setattr(capi.lib, "call", lambda name, *a: (flags.append((name, a[15])) if name == "xsmi_conv2d_fwd" else None,
                                                                real(name, *a))[1])
        losses = []
        for i in range(5):
            if i == 2:                               # a filter changes behind the optimizer's back
                w = [p for p in params if len(p.shape) == 4 and p.shape[1] == 64][1]     # a layer1 filter
                w.eval = w.numpy() * np.float32(0.5)
            bx, by = (x6, y6) if i == 3 else (x, y)
            opt.zero_grad()
            loss = crit(net(bx), by)
            loss.backward()
            opt.step()
            losses.append(loss.item())
        out = [p.numpy().copy() for p in params]
        monkeypatch.undo()
        xs.GLOBAL.INPUTS = None
        return losses, out, sum(1 for _, f in flags if f & capi.CONV_WS_PACKED)

    from xshinnosuke_amd import backend as be
    lanes0 = be.get_option("pack_lanes")
    try:
        la, pa, skipped_a = run(True)
        lb, pb, skipped_b = run(False)
        lc, pc, skipped_c = run(True, 1)                 # the layout launches in a row on one stream ...
        ld, pd, skipped_d = run(True, 4)                 # ... and dealt over four
    finally:
        be.set_option("pack_lanes", lanes0)
    assert skipped_b == 0 and skipped_a >= 19 * 2        # steps 2 and 5 at least find every layout in place
    assert skipped_c == skipped_a and skipped_d == skipped_a
    assert la == lb and la == lc and la == ld
    for u, v, w1, w4 in zip(pa, pb, pc, pd):
        np.testing.assert_array_equal(u, v)
        np.testing.assert_array_equal(u, w1)
        np.testing.assert_array_equal(u, w4)


def test_resnet18_bf16_inference_against_oracle():
    """Inference configuration: moving-statistics batch norm, forward only, convolutions allowed to use bf16
    MFMA operands.  Logits against the NumPy/oracle forward: rel-L2 <= 1e-2 for bf16, <= 1e-4 for fp32."""
    np.random.seed(7)
    X = np.random.randn(4, 3, 64, 64).astype(np.float32)
    net = ResNet18(classes=10, pool=2).to('cuda')
    xd = xs.tensor(X).to('cuda')
    net(xd)                                        # creates the parameters
    xs.GLOBAL.INPUTS = None
    # moving statistics that are not the identity, so the inference formula is exercised
    rng = np.random.default_rng(3)

    def walk(layer):
        if type(layer).__name__ == 'BatchNormalization':
            layer.moving_mean.eval = (0.1 * rng.standard_normal(layer.moving_mean.shape)).astype(np.float32)
            layer.moving_variance.eval = rng.uniform(0.5, 1.5, layer.moving_variance.shape).astype(np.float32)
        for sub in getattr(layer, '_graph', []):
            walk(sub)
        for attr in ('conv1', 'shortcut'):
            if hasattr(layer, attr) and type(layer).__name__ == 'BasicBlock':
                walk(getattr(layer, attr))
    walk(net.conv1)
    for stage in (net.layer1, net.layer2, net.layer3, net.layer4):
        walk(stage)
    ref = _oracle_forward(net, X)
    xs.GLOBAL.TRAINING = False
    try:
        with xs.no_grad():
            y32 = net(xs.tensor(X).to('cuda')).numpy()
            xs.GLOBAL.INPUTS = None
            with xs.conv_precision('bf16'):
                y16 = net(xs.tensor(X).to('cuda')).numpy()
    finally:
        xs.GLOBAL.TRAINING = True
    assert rel_l2(y32, ref) <= 1e-4
    assert rel_l2(y16, ref) <= 1e-2
    assert rel_l2(y16, y32) > 1e-5                 # the bf16 kernels really ran
