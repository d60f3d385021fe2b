"""The conv / max-pool path through the xs-style API (functional ops, layers, Sequential / Model / Module)
on the GPU, checked against the oracle.  Host (NumPy-backed) tensors are staged through device memory;
device tensors stay resident."""
import numpy as np
import pytest

import oracle
import xshinnosuke_amd as xs
from xshinnosuke_amd.nn import functional as F
from xshinnosuke_amd.layers import Conv2D, MaxPooling2D, Flatten, Dense, ReLU, Input
from xshinnosuke_amd.nn.models import Sequential, Model, Module
from xshinnosuke_amd.optim import SGD
from util import rel_l2, he_normal, idx_nchw_to_ref

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.fixture(autouse=True)
def _fresh_state(gpu):
    xs.GLOBAL.INPUTS = None
    xs.GLOBAL.USE_CUDA = False
    xs.GLOBAL.TRAINING = True
    yield
    xs.GLOBAL.INPUTS = None
    xs.GLOBAL.USE_CUDA = False


@pytest.mark.parametrize("device", ["cpu", "cuda"])
def test_functional_conv2d_reference_script_shapes(device):
    """tests/gradient_check/xs_pytorch/cnn.py: x 1x1x4x4, w 3x1x3x3, bias (3,), seed 0; loss = 0.5*(sum(out)-y)^2."""
    np.random.seed(0)
    n_x = np.random.randn(1, 1, 4, 4).astype(np.float32)
    n_y = np.random.randn(1).astype(np.float32)
    n_w = np.random.randn(3, 1, 3, 3).astype(np.float32)
    n_b = np.random.randn(3).astype(np.float32)
    x = xs.tensor(n_x, requires_grad=True); w = xs.tensor(n_w, requires_grad=True); b = xs.tensor(n_b, requires_grad=True)
    if device == "cuda":
        x, w, b = x.to('cuda'), w.to('cuda'), b.to('cuda')
    for t in (x, w, b):
        t.retain_grad(True)
    out = F.conv2d(x, w, b)
    assert out.device == device and out.dtype == 'float32'
    assert out.grad_fn is F.Conv2DBackward and out.in_bounds == [x, w, b]
    assert out.cache['stride'] == (1, 1) and out.cache['padding'] == 0
    y_ref, col = oracle.conv2d_fwd(n_x, n_w, n_b, (1, 1), 0)
    assert rel_l2(out.numpy(), y_ref) <= TOL
    up = (y_ref.sum() - n_y[0]) * np.ones_like(y_ref)            # d/d out of 0.5*(sum(out) - y)^2
    out.backward(up)
    dx, dw, db = oracle.conv2d_bwd(up, n_x.shape, n_w, col, (1, 1), 0, np.zeros_like(n_x), np.zeros_like(n_w),
                                   np.zeros_like(n_b))
    assert rel_l2(x.grad.numpy(), dx) <= TOL
    assert rel_l2(w.grad.numpy(), dw) <= TOL
    assert rel_l2(b.grad.numpy(), db) <= TOL


@pytest.mark.parametrize("device", ["cpu", "cuda"])
def test_functional_max_pool2d_reference_script_shapes(device):
    """tests/gradient_check/xs_pytorch/pooling.py: x 1x3x5x5, max_pool2d(x, 3, 2)."""
    np.random.seed(0)
    n_x = np.random.randn(1, 3, 5, 5).astype(np.float32)
    x = xs.tensor(n_x, requires_grad=True)
    if device == "cuda":
        x = x.to('cuda')
    x.retain_grad(True)
    out = F.max_pool2d(x, 3, 2)
    y_ref, am = oracle.max_pool2d_fwd(n_x, 3, 2, 0)
    assert out.numpy().tobytes() == y_ref.tobytes()
    assert out.cache['mode'] == 'im2col' and out.cache['kernel_size'] == 3 and out.cache['stride'] == (2, 2)
    np.testing.assert_array_equal(idx_nchw_to_ref(out.cache['pool_argmax'].numpy()), am)
    dy = np.arange(y_ref.size, dtype=np.float32).reshape(y_ref.shape) / 3 + 1
    out.backward(dy)
    dx_ref = oracle.max_pool2d_bwd(dy, am, n_x.shape, 3, (2, 2), 0, np.zeros_like(n_x))
    assert x.grad.numpy().tobytes() == dx_ref.tobytes()


def test_gradients_accumulate_across_backward_calls():
    rng = np.random.default_rng(3)
    n_x = rng.standard_normal((2, 3, 8, 8)).astype(np.float32); n_w = he_normal(rng, (4, 3, 3, 3))
    x = xs.tensor(n_x, requires_grad=True).to('cuda'); w = xs.tensor(n_w, requires_grad=True).to('cuda')
    grads = []
    for _ in range(2):
        out = F.max_pool2d(F.conv2d(x, w, None, (1, 1), 1), 2)
        out.backward(np.ones(out.shape, dtype=np.float32))
        grads.append((x.grad.numpy().copy(), w.grad.numpy().copy()))
    np.testing.assert_allclose(grads[1][0], 2 * grads[0][0], rtol=1e-6)
    np.testing.assert_allclose(grads[1][1], 2 * grads[0][1], rtol=1e-6)


def test_out_argument_is_written_in_place_and_sliced():
    rng = np.random.default_rng(4)
    n_x = rng.standard_normal((5, 2, 6, 6)).astype(np.float32); n_w = he_normal(rng, (3, 2, 3, 3))
    w = xs.tensor(n_w).to('cuda')
    buf = xs.zeros(8, 3, 4, 4, dtype=np.float32).to('cuda')
    buf.slices(slice(None, 5, None))                       # capacity 8, active batch 5
    storage_ptr = buf.shape_capacity and buf._data.ptr
    out = F.conv2d(xs.tensor(n_x).to('cuda'), w, None, (1, 1), 0, out=buf)
    assert out is buf and buf._data.ptr == storage_ptr and buf.shape == (5, 3, 4, 4)
    y_ref, _ = oracle.conv2d_fwd(n_x, n_w, None, (1, 1), 0)
    assert rel_l2(buf.numpy(), y_ref) <= TOL
    assert np.all(buf._data.numpy()[5:] == 0)              # rows beyond the slice are untouched


def test_float64_host_tensors_keep_their_dtype():
    rng = np.random.default_rng(5)
    n_x = rng.standard_normal((2, 2, 7, 7)); n_w = rng.standard_normal((3, 2, 3, 3)) * 0.3     # float64, like xs.randn
    x = xs.tensor(n_x, requires_grad=True); w = xs.tensor(n_w, requires_grad=True)
    out = F.conv2d(x, w, None, (2, 2), 1)
    assert out.dtype == 'float64'
    y_ref, _ = oracle.conv2d_fwd(n_x, n_w, None, (2, 2), 1)
    assert rel_l2(out.numpy(), y_ref) <= TOL                # computed in fp32 on the device, stored as float64


def _readme_net_oracle(x, wc, bc, wd, bd, labels, lr):
    """README functional net, one fwd+bwd+SGD step, with the oracle for conv / pool and NumPy for the rest."""
    y1, col = oracle.conv2d_fwd(x, wc, bc, (1, 1), 0)
    a1 = oracle.relu_fwd(y1)
    p1, am = oracle.max_pool2d_fwd(a1, 2, None, 0)
    flat = p1.reshape(p1.shape[0], -1)
    logits = flat.astype(np.float64) @ wd + bd
    z = logits - logits.max(axis=1, keepdims=True)
    sm = np.exp(z) / np.exp(z).sum(axis=1, keepdims=True)
    loss = -np.log(sm[np.arange(len(labels)), labels]).mean()
    g = sm.copy(); g[np.arange(len(labels)), labels] -= 1; g /= len(labels)
    dwd = flat.astype(np.float64).T @ g; dbd = g.sum(axis=0, keepdims=True)
    dflat = (g @ wd.T).astype(np.float32)
    da1 = oracle.max_pool2d_bwd(dflat.reshape(p1.shape), am, a1.shape, 2, (2, 2), 0, np.zeros_like(a1))
    dy1 = oracle.relu_bwd(da1, y1)
    _, dwc, dbc = oracle.conv2d_bwd(dy1, x.shape, wc, col, (1, 1), 0, None, np.zeros_like(wc), np.zeros_like(bc))
    return loss, logits, (wc - lr * dwc, bc - lr * dbc, wd - lr * dwd, bd - lr * dbd)


@pytest.mark.parametrize("kind", ["sequential", "functional"])
def test_readme_network_one_training_step(kind):
    """The README network of the reference at its benchmark size: N=256x1x28x28, Conv2D(8, 2x2, relu) -> MaxPool 2x2 -> Flatten -> Dense(10), CE, SGD lr 0.01."""
    rng = np.random.default_rng(0)
    n = 256
    x = rng.standard_normal((n, 1, 28, 28)).astype(np.float32)
    labels = rng.integers(0, 10, size=n)
    wc = (rng.standard_normal((8, 1, 2, 2)) * np.sqrt(2.0 / 4)).astype(np.float32)
    bc = np.zeros((1, 8), dtype=np.float32)
    wd = (rng.standard_normal((1352, 10)) * 0.1).astype(np.float32)
    bd = np.zeros((1, 10), dtype=np.float32)
    if kind == "sequential":
        model = Sequential(Conv2D(8, 2, activation='relu', input_shape=(1, 28, 28)), MaxPooling2D(2), Flatten(), Dense(10))
        model.compile(SGD(lr=0.01), 'cross_entropy')
        layers = model._graph
    else:
        xin = Input(input_shape=(1, 28, 28))
        h = Conv2D(8, (2, 2), activation='relu')(xin)
        h = MaxPooling2D((2, 2))(h)
        h = Flatten()(h)
        h = Dense(10)(h)
        model = Model(inputs=xin, outputs=h)
        model.compile(SGD(lr=0.01), 'cross_entropy')
        layers = model._graph[1:]
    conv, dense = layers[0], layers[3]
    for p, v in zip(conv.parameters() + dense.parameters(), (wc, bc, wd, bd)):
        p.eval = v.astype(np.float64)
    hist = model.fit(x, labels, batch_size=n, epochs=1, verbose=0, shuffle=False)
    loss_ref, _, new = _readme_net_oracle(x, wc, bc, wd.astype(np.float64), bd.astype(np.float64), labels, 0.01)
    assert abs(hist['train_loss'][0] - loss_ref) <= 1e-5 * abs(loss_ref)
    for p, v in zip(conv.parameters() + dense.parameters(), new):
        assert rel_l2(p.numpy(), v) <= TOL


def test_static_graph_handles_a_short_last_batch():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((70, 1, 12, 12)).astype(np.float32)
    labels = rng.integers(0, 4, size=70)
    model = Sequential(Conv2D(4, 3, padding=1, activation='relu', input_shape=(1, 12, 12)), MaxPooling2D(3, 2, 1),
                       Flatten(), Dense(4))
    model.compile(SGD(lr=0.05), 'cross_entropy')
    hist = model.fit(x, labels, batch_size=32, epochs=3, verbose=0, shuffle=True)     # batches of 32, 32, 6
    assert hist['train_loss'][-1] < hist['train_loss'][0]
    conv_out = model._graph[0].data
    assert conv_out.shape_capacity[0] == 32 and conv_out.shape[0] == 6
    acc, loss = model.evaluate(x, labels, batch_size=32)
    assert 0.0 <= acc <= 1.0 and np.isfinite(loss)
    assert model.predict(x[:10]).shape == (10, 4)


class _Net(Module):
    def __init__(self):
        super().__init__()
        self.conv1 = Conv2D(out_channels=8, kernel_size=3)
        self.relu = ReLU(inplace=True)
        self.flat = Flatten()
        self.fc = Dense(10)

    def forward(self, x, *args):
        x = self.conv1(x)
        x = self.relu(x)
        x = F.max_pool2d(x, kernel_size=2)
        x = self.flat(x)
        return self.fc(x)


def test_readme_dynamic_module_trains_and_matches_oracle_gradients():
    np.random.seed(0)
    X = np.random.randn(20, 3, 12, 12).astype(np.float32)
    Y = np.random.randint(0, 10, (20,))
    net = _Net()
    x, y = xs.tensor(X), xs.tensor(Y)
    out = net(x)
    assert len(net.parameters()) == 4                       # conv w, b and dense w, b found by the graph walk
    loss = xs.nn.CrossEntropyLoss()(out, y)
    wc, bc = (p.numpy().copy() for p in net.conv1.parameters())
    wd, bd = (p.numpy().copy() for p in net.fc.parameters())
    loss.backward()
    # oracle for the same graph
    y1, col = oracle.conv2d_fwd(X, wc.astype(np.float32), bc.astype(np.float32), (1, 1), 0)
    a1 = oracle.relu_fwd(y1)
    p1, am = oracle.max_pool2d_fwd(a1, 2, None, 0)
    flat = p1.reshape(20, -1).astype(np.float64)
    logits = flat @ wd + bd
    z = logits - logits.max(axis=1, keepdims=True)
    sm = np.exp(z) / np.exp(z).sum(axis=1, keepdims=True)
    g = sm.copy(); g[np.arange(20), Y] -= 1; g /= 20
    da1 = oracle.max_pool2d_bwd((g @ wd.T).astype(np.float32).reshape(p1.shape), am, a1.shape, 2, (2, 2), 0, np.zeros_like(a1))
    _, dwc, dbc = oracle.conv2d_bwd(oracle.relu_bwd(da1, y1), X.shape, wc.astype(np.float32), col, (1, 1), 0, None,
                                    np.zeros_like(wc, dtype=np.float32), np.zeros((1, 8), dtype=np.float32))
    assert rel_l2(net.conv1.parameters()[0].grad.numpy(), dwc) <= 2e-5
    assert rel_l2(net.conv1.parameters()[1].grad.numpy(), dbc) <= 2e-5
    assert rel_l2(net.fc.parameters()[0].grad.numpy(), flat.T @ g) <= 2e-5
    # a few SGD steps reduce the loss
    opt = SGD(net.parameters(), lr=0.1)
    first = last = None
    for _ in range(8):
        opt.zero_grad()
        l = xs.nn.CrossEntropyLoss()(net(xs.tensor(X)), xs.tensor(Y))
        l.backward()
        opt.step()
        first = l.item() if first is None else first
        last = l.item()
    assert last < first


def test_conv2d_rejects_what_the_reference_rejects():
    x = xs.tensor(np.zeros((1, 3, 4, 4), dtype=np.float32)); w = xs.tensor(np.zeros((2, 4, 3, 3), dtype=np.float32))
    with pytest.raises(ValueError):
        F.conv2d(x, w)                                        # channel mismatch (NumPy dot raises ValueError there)
    with pytest.raises(TypeError):
        F.conv2d(x, xs.tensor(np.zeros((2, 3, 3, 3), dtype=np.float32)), padding=(1, 1))
    with pytest.raises(ValueError):
        F.max_pool2d(x, (2, 3))


def test_pending_zero_gradient_buffers(gpu):
    """Gradient buffers are cleared lazily: they read as zero, an op that overwrites all of one skips the
    clear, and accumulation into a used buffer still adds."""
    z = gpu.zeros((4, 8), lazy=True)
    assert z.is_fresh()
    np.testing.assert_array_equal(z.numpy(), np.zeros((4, 8), np.float32))      # reading clears it for real
    assert not z.is_fresh()
    z = gpu.zeros((4, 8), lazy=True)
    view = z.leading(1, 3)                                                      # part of the allocation
    assert not view.take_fresh()
    np.testing.assert_array_equal(z.numpy(), np.zeros((4, 8), np.float32))
    K = gpu.kernels
    g = gpu.to_device(np.arange(32, dtype=np.float32).reshape(4, 8))
    acc = gpu.zeros((4, 8), lazy=True)
    K.axpy(acc, g, 1.0)                                                          # fresh: becomes a copy
    K.axpy(acc, g, 0.5)                                                          # used: adds
    np.testing.assert_array_equal(acc.numpy(), 1.5 * g.numpy())
    # conv weight gradient: dw pending, db already used -> both must end up accumulated correctly
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, 3, 6, 6)).astype(np.float32); dy = rng.standard_normal((2, 4, 4, 4)).astype(np.float32)
    dw = gpu.zeros((4, 3, 3, 3), lazy=True); db = gpu.to_device(np.ones(4, np.float32))
    K.conv2d_bwd_weight(gpu.to_device(dy), gpu.to_device(x), (4, 3, 3, 3), (1, 1), 0, dw=dw, db=db, accumulate=True)
    dw_ref, db_ref = K.conv2d_bwd_weight(gpu.to_device(dy), gpu.to_device(x), (4, 3, 3, 3), (1, 1), 0, want_db=True)
    np.testing.assert_allclose(dw.numpy(), dw_ref.numpy(), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(db.numpy(), db_ref.numpy() + 1.0, rtol=1e-6, atol=1e-6)


def _small_cnn():
    return Sequential(Conv2D(4, 3, padding=1, activation='relu', input_shape=(1, 12, 12)), MaxPooling2D(3, 2, 1),
                      Flatten(), Dense(4))


def test_device_fit_matches_host_fit_batch_for_batch():
    """Static graph on the device: the loader's fixed device tensors are refilled through page-locked staging
    memory; three epochs of batches 32/32/6 must follow the host path (same seeds, same order)."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal((70, 1, 12, 12)).astype(np.float32)
    labels = rng.integers(0, 4, size=70)
    np.random.seed(3)
    host = _small_cnn(); host.compile(SGD(lr=0.05), 'cross_entropy')
    hh = host.fit(x, labels, batch_size=32, epochs=3, verbose=0, shuffle=True)
    np.random.seed(3)
    xs.GLOBAL.USE_CUDA = True
    try:
        devm = _small_cnn(); devm.compile(SGD(lr=0.05), 'cross_entropy')
        assert devm._device == 'cuda' and all(p.device == 'cuda' for p in devm.parameters())
        hd = devm.fit(x, labels, batch_size=32, epochs=3, verbose=0, shuffle=True)
        np.testing.assert_allclose(hd['train_loss'], hh['train_loss'], rtol=2e-4)
        ph, pd = host.predict(x[:9]).numpy(), devm.predict(x[:9]).numpy()
        assert rel_l2(pd, ph) <= 2e-4
    finally:
        xs.GLOBAL.USE_CUDA = False


def test_device_fit_allocates_nothing_in_the_steady_state():
    """Static graph on the device: from the third step on, a training step calls neither the device allocator
    nor the pinned-memory allocator (blocks come from the size-keyed pool, layer outputs are preallocated)."""
    from xshinnosuke_amd.backend import capi
    rng = np.random.default_rng(15)
    x = rng.standard_normal((96, 1, 12, 12)).astype(np.float32)
    labels = rng.integers(0, 4, size=96)
    np.random.seed(5)
    xs.GLOBAL.USE_CUDA = True
    graph_switch, xs.GLOBAL.STEP_GRAPH = xs.GLOBAL.STEP_GRAPH, False      # every step is to be issued launch by launch
    calls = []
    real = capi.lib.call
    try:
        m = _small_cnn(); m.compile(SGD(lr=0.05), 'cross_entropy')
        capi.lib.call = lambda name, *a: (calls.append(name), real(name, *a))[1]
        m.fit(x, labels, batch_size=16, epochs=1, verbose=0, shuffle=False)       # six steps of 16
    finally:
        capi.lib.call = real
        xs.GLOBAL.USE_CUDA = False
        xs.GLOBAL.STEP_GRAPH = graph_switch
    steps = [i for i, name in enumerate(calls) if name == "xsmi_axpy_multi"]       # one optimizer step each
    assert len(steps) == 6
    steady = calls[steps[1] + 1:steps[5] + 1]                                       # steps 3..6
    assert "xsmi_conv2d_fwd" in steady and "xsmi_conv2d_bwd_weight" in steady or "xsmi_conv2d_bwd" in steady
    for name in ("xsmi_malloc", "xsmi_free", "xsmi_host_alloc", "xsmi_host_free"):
        assert name not in steady, (name, steady.count(name))
    assert "xsmi_malloc" in calls[:steps[0]]                                       # the counter does see allocations


def test_checkpoint_round_trip_from_the_device(tmp_path):
    """save() writes host arrays; load() puts them back on the device; predictions and the next epoch agree."""
    rng = np.random.default_rng(6)
    x = rng.standard_normal((40, 1, 12, 12)).astype(np.float32)
    labels = rng.integers(0, 4, size=40)
    np.random.seed(4)
    xs.GLOBAL.USE_CUDA = True
    try:
        m = _small_cnn(); m.compile(SGD(lr=0.05), 'cross_entropy')
        m.fit(x, labels, batch_size=16, epochs=1, verbose=0)
        p1 = m.predict(x).numpy()
        m.save(str(tmp_path / 'ck'))
        import pickle
        with open(str(tmp_path / 'ck.pkl'), 'rb') as f:
            assert b'DeviceArray' not in f.read().replace(b'_rebuild_array', b'')    # arrays travel as NumPy data
        m2 = Sequential(); m2.load(str(tmp_path / 'ck'))
        assert m2._device == 'cuda' and len(m2.parameters()) == 4
        np.testing.assert_array_equal(m2.predict(x).numpy(), p1)
        h1 = m.fit(x, labels, batch_size=16, epochs=1, verbose=0, shuffle=False)
        h2 = m2.fit(x, labels, batch_size=16, epochs=1, verbose=0, shuffle=False)
        np.testing.assert_allclose(h2['train_loss'], h1['train_loss'], rtol=1e-6)
    finally:
        xs.GLOBAL.USE_CUDA = False


def test_checkpoint_of_a_conv_batch_norm_model_after_inference(tmp_path):
    """fit with validation and predict run the folded Conv2D -> BatchNormalization inference path, which keeps
    folded filters between forwards; a checkpoint written afterwards holds parameters only, and the loaded
    model predicts the same values."""
    from xshinnosuke_amd.layers import BatchNormalization
    rng = np.random.default_rng(16)
    x = rng.standard_normal((48, 2, 10, 10)).astype(np.float32)
    labels = rng.integers(0, 3, size=48)
    np.random.seed(9)
    xs.GLOBAL.USE_CUDA = True
    try:
        m = Sequential(Conv2D(6, 3, padding=1, input_shape=(2, 10, 10)), BatchNormalization(), ReLU(True),
                       MaxPooling2D(2), Flatten(), Dense(3))
        m.compile(SGD(lr=0.05), 'cross_entropy')
        m.fit(x, labels, batch_size=16, epochs=2, verbose=0, validation_data=(x[:16], labels[:16]))
        p1 = m.predict(x).numpy()
        m.save(str(tmp_path / 'ckbn'))
        raw = open(str(tmp_path / 'ckbn.pkl'), 'rb').read()
        assert b'_Block' not in raw and b'Workspace' not in raw and b'_folded_filter' not in raw
        m2 = Sequential(); m2.load(str(tmp_path / 'ckbn'))
        assert m2._device == 'cuda'
        p2 = m2.predict(x).numpy()
        np.testing.assert_array_equal(p2, p1)
        np.testing.assert_array_equal(m.predict(x).numpy(), p1)      # the saved model still works, too
    finally:
        xs.GLOBAL.TRAINING = True
        xs.GLOBAL.USE_CUDA = False


def test_inference_folds_batch_norm_into_the_convolution(gpu):
    """Conv2D -> BatchNormalization [-> ReLU] in a Sequential, moving statistics, nothing to differentiate: the
    normalisation is folded into the filter.  Same values as the layer-by-layer forward (which runs whenever
    gradients are tracked), layer outputs shared, and the kernel-level fold against its closed form."""
    from xshinnosuke_amd.layers import Conv2D, BatchNormalization, ReLU
    K = gpu.kernels
    rng = np.random.default_rng(31)
    w = rng.standard_normal((5, 3, 3, 3)).astype(np.float32)
    b = rng.standard_normal(5).astype(np.float32)
    g, bt, mu = (rng.standard_normal(5).astype(np.float32) for _ in range(3))
    var = rng.uniform(0.5, 2.0, 5).astype(np.float32)
    w2, b2 = K.bn_fold(gpu.to_device(w), gpu.to_device(b), gpu.to_device(g), gpu.to_device(bt), gpu.to_device(mu),
                       gpu.to_device(var), 1e-3)
    scale = g / np.sqrt(var + np.float32(1e-3))
    np.testing.assert_allclose(w2.numpy(), w * scale[:, None, None, None], rtol=1e-6)
    np.testing.assert_allclose(b2.numpy(), bt + (b - mu) * scale, rtol=1e-5, atol=1e-6)
    w3, b3 = K.bn_fold(gpu.to_device(w), None, gpu.to_device(g), gpu.to_device(bt), gpu.to_device(mu), gpu.to_device(var), 1e-3)
    np.testing.assert_allclose(b3.numpy(), bt - mu * scale, rtol=1e-5, atol=1e-6)

    np.random.seed(8)
    xs.GLOBAL.USE_CUDA = True
    try:
        net = Sequential(Conv2D(8, 3, padding=1, input_shape=(3, 10, 12)), BatchNormalization(), ReLU(True),
                         Conv2D(6, 3, stride=2, padding=1, use_bias=False), BatchNormalization())
        x = xs.tensor(rng.standard_normal((4, 3, 10, 12)).astype(np.float32)).to('cuda')
        with xs.no_grad():
            net(x)                                   # creates the parameters
        for layer in net._graph:
            if isinstance(layer, BatchNormalization):
                c = layer.moving_mean.shape[0] if hasattr(layer.moving_mean, 'shape') else len(layer.moving_mean)
                layer.moving_mean = xs.tensor(rng.standard_normal(c).astype(np.float32)).to('cuda')
                layer.moving_variance = xs.tensor(rng.uniform(0.5, 2.0, c).astype(np.float32)).to('cuda')
                layer._parameters[0].eval = gpu.to_device(rng.standard_normal(c).astype(np.float32))
                layer._parameters[1].eval = gpu.to_device(rng.standard_normal(c).astype(np.float32))
        xs.GLOBAL.TRAINING = False
        plain = net(x).numpy()                       # gradients tracked: layer by layer
        with xs.no_grad():
            folded = net(x)
        assert rel_l2(folded.numpy(), plain) <= 1e-5
        assert net._graph[0].data is net._graph[1].data is net._graph[2].data
        assert net._graph[3].data is net._graph[4].data is folded
        assert folded.grad_fn is None and not folded.requires_grad
        # The folded and packed filters are kept while the parameters are untouched: the next forward launches no
        # fold, and the same values come out for another (smaller) batch; a changed statistic, scale or filter is seen.
        from xshinnosuke_amd.backend import capi
        calls = []
        real = capi.lib.call
        capi.lib.call = lambda name, *a: (calls.append(name), real(name, *a))[1]
        try:
            with xs.no_grad():
                again = net(x).numpy()
        finally:
            capi.lib.call = real
        assert "xsmi_bn_fold" not in calls and calls.count("xsmi_conv2d_fwd") == 2
        np.testing.assert_array_equal(again, folded.numpy())
        x2 = xs.tensor(x.numpy()[:2]).to('cuda')
        with xs.no_grad():
            part = net(x2).numpy()
        np.testing.assert_array_equal(part, again[:2])
        conv2, bn2 = net._graph[3], net._graph[4]
        for change in ("mean", "gamma", "filter", "bf16"):
            if change == "mean":
                bn2.moving_mean.eval = gpu.to_device(rng.standard_normal(6).astype(np.float32))
            elif change == "gamma":
                K.scale(bn2._parameters[0].eval, 2.0, out=bn2._parameters[0].eval)      # in place, through a kernel
            elif change == "filter":
                conv2._parameters[0].eval.fill_zero(lazy=True)                          # only a pending clear
            with xs.conv_precision('bf16' if change == "bf16" else 'fp32'), xs.no_grad():
                out = net(x).numpy()                 # first: nothing else has looked at the parameters since the change
            plain = net(x).numpy()
            assert rel_l2(out, plain) <= (1e-2 if change == "bf16" else 1e-5), change
            if change == "filter":
                assert np.abs(plain).max() > 0 and np.array_equal(out[:, :, 0, 0], out[:, :, 1, 1])   # bias only
    finally:
        xs.GLOBAL.TRAINING = True
        xs.GLOBAL.USE_CUDA = False
