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
