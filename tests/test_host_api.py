"""Host-only behaviour of the model classes (no convolution, so no GPU): checkpoints and the re-wiring of
reused static output tensors."""
import numpy as np

from xshinnosuke_amd.nn.models import Sequential
from xshinnosuke_amd.layers import Dense, ReLU
from xshinnosuke_amd.utils.data import DataSet, DataLoader


def _mlp():
    m = Sequential(Dense(8, input_shape=(6,)), ReLU(), Dense(3))
    m.compile('sgd', 'cross_entropy', lr=0.1)
    return m


def test_save_load_round_trip(tmp_path):
    np.random.seed(0)
    x = np.random.randn(20, 6).astype(np.float32)
    y = np.random.randint(0, 3, (20,))
    m = _mlp()
    m.fit(x, y, batch_size=8, epochs=2, verbose=0)
    before = m.predict(x).numpy()
    m.save(str(tmp_path / 'ck'))                      # '.pkl' is appended, as in the reference
    assert (tmp_path / 'ck.pkl').exists()
    m2 = Sequential()
    m2.load(str(tmp_path / 'ck.pkl'))
    assert len(m2.parameters()) == 4
    np.testing.assert_array_equal(m2.predict(x).numpy(), before)
    h1 = m.fit(x, y, batch_size=8, epochs=1, verbose=0)
    h2 = m2.fit(x, y, batch_size=8, epochs=1, verbose=0)
    assert h1['train_loss'] == h2['train_loss']       # the optimizer state and the parameters it updates came along


def test_fit_after_predict_reads_the_new_batches():
    """A layer's reused output tensor must take its input from the tensor that feeds it now (a second loader
    hands in different batch tensors)."""
    np.random.seed(1)
    x = np.random.randn(20, 6).astype(np.float32)
    y = np.random.randint(0, 3, (20,))
    np.random.seed(2)
    a = _mlp()
    np.random.seed(2)
    b = _mlp()
    a.predict(x)                                       # output tensors with capacity 20 exist before training
    ha = a.fit(x, y, batch_size=8, epochs=2, verbose=0, shuffle=False)
    hb = b.fit(x, y, batch_size=8, epochs=2, verbose=0, shuffle=False)
    np.testing.assert_allclose(ha['train_loss'], hb['train_loss'], rtol=1e-12)


def test_loader_reuses_its_tensors_and_slices_the_last_batch():
    x = np.arange(50, dtype=np.float32).reshape(10, 5)
    loader = DataLoader(DataSet(x), batch_size=4)
    seen = [(id(t), t.shape, t.numpy().copy()) for t in loader]
    assert len({i for i, _, _ in seen}) == 1
    assert [s for _, s, _ in seen] == [(4, 5), (4, 5), (2, 5)]
    np.testing.assert_array_equal(np.concatenate([v for _, _, v in seen]), x)


def test_checkpoints_carry_no_device_state():
    """A pickled Parameter holds its values only: filters kept between inference forwards live in a side table
    of the functional module, and device memory blocks / workspaces refuse to be pickled at all."""
    import pickle
    import pytest
    from xshinnosuke_amd.core.base import Parameter
    from xshinnosuke_amd.nn import functional as F
    from xshinnosuke_amd.backend import array as dev

    p = Parameter(np.arange(6, dtype=np.float32).reshape(2, 3))
    F._FOLDED[p] = {'key': None, 'w': None, 'b': None, 'ws': dev.Workspace(), 'of': []}
    q = pickle.loads(pickle.dumps(p))
    assert F._FOLDED.get(q) is None and '_folded_filter' not in vars(q)
    np.testing.assert_array_equal(q.numpy(), p.numpy())
    del F._FOLDED[p]

    with pytest.raises(TypeError):
        pickle.dumps(dev.Workspace())
    blk = object.__new__(dev._Block)
    blk.ptr = None                                    # never allocated: nothing to return on deletion
    with pytest.raises(TypeError):
        pickle.dumps(blk)


def test_dense_activation_names_one_training_step():
    """Dense(activation='tanh' | 'sigmoid' | 'relu') appends the named activation (reference
    xs/layers/linear.py:12,48-49, xs/layers/activators.py:74-87); one SGD step of a static graph against the
    closed-form gradients.  An unknown name means no activation, as in the reference."""
    from xshinnosuke_amd.layers import get_activator
    np.random.seed(3)
    x = np.random.randn(12, 6)
    y = np.random.randint(0, 3, (12,))
    m = Sequential(Dense(8, activation='tanh', input_shape=(6,)), Dense(5, activation='sigmoid'),
                   Dense(4, activation='relu'), Dense(3))
    m.compile('sgd', 'cross_entropy', lr=0.1)
    (w1, b1), (w2, b2), (w3, b3), (w4, b4) = [[p.numpy().astype(np.float64).copy() for p in l.parameters()] for l in m._graph]
    m.fit(x, y, batch_size=12, epochs=1, verbose=0, shuffle=False)
    a1 = x @ w1 + b1; h1 = np.tanh(a1)
    a2 = h1 @ w2 + b2; h2 = 1 / (1 + np.exp(-a2))
    a3 = h2 @ w3 + b3; h3 = np.maximum(a3, 0)
    z = h3 @ w4 + b4
    p = np.exp(z - z.max(1, keepdims=True)); p /= p.sum(1, keepdims=True)
    dz = p.copy(); dz[np.arange(12), y] -= 1; dz /= 12
    d3 = (dz @ w4.T) * (a3 >= 0)
    d2 = (d3 @ w3.T) * h2 * (1 - h2)
    d1 = (d2 @ w2.T) * (1 - h1 ** 2)
    want = [w1 - 0.1 * x.T @ d1, b1 - 0.1 * d1.sum(0), w2 - 0.1 * h1.T @ d2, b2 - 0.1 * d2.sum(0),
            w3 - 0.1 * h2.T @ d3, b3 - 0.1 * d3.sum(0), w4 - 0.1 * h3.T @ dz, b4 - 0.1 * dz.sum(0)]
    got = [p.numpy() for l in m._graph for p in l.parameters()]
    for g, w in zip(got, want):
        np.testing.assert_allclose(g.reshape(w.shape) if g.size == w.size else g, w.reshape(g.shape), rtol=1e-9, atol=1e-12)
    assert get_activator('no-such-activation') is None and get_activator(None) is None
    assert Dense(3, activation='no-such-activation')._act_layer is None


def test_bench_reads_its_traffic_figure_from_the_committed_profile():
    """bench.py's roofline.traffic is the figure kept beside its measurement in profiles/, not a number typed into
    the benchmark: the line is there and parses to a plausible byte count (algorithmic bytes of the launch: 51.5 MB)."""
    import importlib.util
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("bench_for_test", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    traffic = bench.tap_sk_traffic_bytes()
    assert traffic is not None and 51.5e6 <= traffic <= 200e6
