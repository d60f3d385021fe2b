"""Step graphs: a recorded ResNet-18 training step and a recorded inference forward, replayed several times with
eager work and synchronisations between the replays, must give bit for bit what the same steps give when every
launch is issued from Python."""
import numpy as np
import pytest

import xshinnosuke_amd as xs
from xshinnosuke_amd import backend as be
from xshinnosuke_amd.backend import StepGraph
from xshinnosuke_amd.backend import array as dev_array
from xshinnosuke_amd.optim import SGD
from resnet18 import ResNet18, named_params

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _fresh_state(gpu):
    xs.GLOBAL.INPUTS = None
    xs.GLOBAL.USE_CUDA = False
    xs.GLOBAL.TRAINING = True
    yield
    xs.GLOBAL.INPUTS = None
    xs.GLOBAL.USE_CUDA = False
    xs.GLOBAL.TRAINING = True


def _batches(count, n, size, classes, seed):
    rng = np.random.default_rng(seed)
    return [(rng.standard_normal((n, 3, size, size), dtype=np.float32), rng.integers(0, classes, size=(n,)))
            for _ in range(count)]


def _eager_noise(i):
    """Unrelated eager work between two replays: allocations of many sizes, a convolution, a host read."""
    rng = np.random.default_rng(100 + i)
    junk = [be.zeros((rng.integers(1, 1 << 16),)) for _ in range(8)]
    a = xs.tensor(rng.standard_normal((2, 8, 12, 12), dtype=np.float32)).to('cuda')
    w = xs.tensor(rng.standard_normal((8, 8, 3, 3), dtype=np.float32)).to('cuda')
    with xs.no_grad():
        y = xs.nn.functional.conv2d(a, w, None, 1, 1)
    xs.GLOBAL.INPUTS = None
    out = y.numpy()
    del junk
    return out


def _training_run(batches, graph_from=None):
    """Losses and final parameters of len(batches) SGD steps; from step `graph_from` on the step is a replay."""
    np.random.seed(11)
    net = ResNet18(classes=10, pool=2).to('cuda')
    x = xs.tensor(batches[0][0]).to('cuda')
    y = xs.tensor(batches[0][1]).to('cuda')
    with xs.no_grad():
        net(x)                                    # creates the parameters
    xs.GLOBAL.INPUTS = None
    opt = SGD(net.parameters(), lr=0.05)
    crit = xs.nn.CrossEntropyLoss()

    def step():
        opt.zero_grad()
        loss = crit(net(x), y)
        loss.backward()
        opt.step()
        return loss

    losses, graph, loss = [], None, None
    for i, (bx, by) in enumerate(batches):
        x.eval.set(bx)
        y.eval.set(by)
        if graph_from is not None and i >= graph_from:
            if graph is None:
                graph = StepGraph()
                with graph.capture():
                    loss = step()
                    with pytest.raises(be.XsmiError):
                        loss.item()               # nothing has run yet
            graph.replay()
        else:
            loss = step()
        losses.append(loss.item())
        _eager_noise(i)
        be.synchronize()
    params = [p.numpy().copy() for p in named_params(net)]
    if graph is not None:
        assert graph.replays == len(batches) - graph_from
        graph.close()
    return losses, params


def test_replayed_training_steps_equal_eager_steps():
    batches = _batches(6, 4, 64, 10, seed=5)
    eager_losses, eager_params = _training_run(batches)
    graph_losses, graph_params = _training_run(batches, graph_from=2)
    assert len(set(eager_losses)) == len(eager_losses)          # the steps really differ
    assert graph_losses == eager_losses
    assert len(graph_params) == len(eager_params) == 82
    for a, b in zip(graph_params, eager_params):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("mode", ["fp32", "bf16"])
def test_replayed_inference_equals_eager_inference(mode):
    batches = _batches(4, 8, 64, 10, seed=9)
    np.random.seed(12)
    net = ResNet18(classes=10, pool=2).to('cuda')
    x = xs.tensor(batches[0][0]).to('cuda')
    xs.GLOBAL.TRAINING = False
    with xs.no_grad(), xs.conv_precision(mode):
        net(x)                                    # creates the parameters; the first fold of a filter may take another kernel
        eager = []
        for bx, _ in batches:
            x.eval.set(bx)
            eager.append(net(x).numpy().copy())
        xs.GLOBAL.INPUTS = None
        graph = StepGraph()
        with graph.capture():
            out = net(x)
        xs.GLOBAL.INPUTS = None
        for i, (bx, _) in enumerate(batches):
            x.eval.set(bx)
            graph.replay()
            got = out.numpy()
            assert np.array_equal(got, eager[i]), i
            # eager inference with the same weights between two replays sees valid folded filters
            x.eval.set(batches[(i + 1) % len(batches)][0])
            again = net(x).numpy()
            xs.GLOBAL.INPUTS = None
            assert np.array_equal(again, eager[(i + 1) % len(batches)]), i
            _eager_noise(i)
    graph.close()


def test_a_failed_recording_leaves_the_library_usable():
    a = xs.tensor(np.ones((2, 8, 12, 12), dtype=np.float32)).to('cuda')
    graph = StepGraph()
    with pytest.raises(RuntimeError, match="boom"):
        with graph.capture():
            a.eval.fill_zero()
            raise RuntimeError("boom")
    assert dev_array._CAPTURE[0] is None
    assert np.array_equal(a.numpy(), np.ones((2, 8, 12, 12), dtype=np.float32))    # the recorded clear never ran
    with pytest.raises(be.XsmiError):
        graph.replay()
    assert _eager_noise(0).shape == (2, 8, 12, 12)


def _small_cnn():
    from xshinnosuke_amd.layers import Conv2D, MaxPooling2D, Flatten, Dense, BatchNormalization, ReLU
    from xshinnosuke_amd.nn.models import Sequential
    # the 32 -> 32 layer takes the tap-major kernels, whose filter layouts are made ahead of the step and read by the
    # recording as already in place
    return Sequential(Conv2D(32, 3, padding=1, input_shape=(1, 12, 12)), BatchNormalization(), ReLU(),
                      MaxPooling2D(2), Conv2D(32, 3, padding=1, activation='relu'),
                      Conv2D(8, 3, padding=1, activation='relu'), Flatten(), Dense(4))


def test_fit_with_a_recorded_step_equals_fit_without():
    """fit() on the device with GLOBAL.STEP_GRAPH: four epochs of batches 16/16/16/16/6 with validation between the
    epochs; from the third step on every full batch is a replay, the short batches run launch by launch.  Losses,
    accuracies and predictions must equal those of the launch-by-launch fit bit for bit."""
    rng = np.random.default_rng(21)
    x = rng.standard_normal((70, 1, 12, 12)).astype(np.float32)
    labels = rng.integers(0, 4, size=70)
    xv, lv = rng.standard_normal((20, 1, 12, 12)).astype(np.float32), rng.integers(0, 4, size=20)
    results = []
    from xshinnosuke_amd.backend import capi
    real = capi.lib.call
    xs.GLOBAL.USE_CUDA = True
    try:
        for use_graph in (False, True):
            np.random.seed(3)
            xs.GLOBAL.STEP_GRAPH = use_graph
            calls = []
            m = _small_cnn()
            m.compile(SGD(lr=0.05), 'cross_entropy')
            capi.lib.call = lambda name, *a: (calls.append(name), real(name, *a))[1]
            try:
                h = m.fit(x, labels, batch_size=16, epochs=4, verbose=0, shuffle=True, validation_data=(xv, lv))
            finally:
                capi.lib.call = real
            results.append((h, m.predict(x[:9]).numpy().copy(), m.optimizer.iterations, calls.count("xsmi_graph_launch")))
            if use_graph:
                # the eager short batch at each epoch's end changed the filters: the first replay of the next epoch
                # laid the recorded filters out again before it launched
                at = [i for i, name in enumerate(calls) if name == "xsmi_graph_launch"]
                assert sum(calls[i - 1] == "xsmi_conv2d_pack" for i in at) >= 3
            xs.GLOBAL.INPUTS = None
    finally:
        xs.GLOBAL.STEP_GRAPH = False
        xs.GLOBAL.USE_CUDA = False
    (h0, p0, it0, launches0), (h1, p1, it1, launches1) = results
    assert launches0 == 0 and launches1 == 4 * 4 - 2          # 16 full batches, the first two run eagerly
    assert it0 == it1 == 20
    for key in ('train_loss', 'train_acc', 'validation_loss', 'validation_acc'):
        assert h1[key] == h0[key], key
    assert np.array_equal(p1, p0)
