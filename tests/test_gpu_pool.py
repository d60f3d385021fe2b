"""Max-pool parity on the GPU through the C ABI: values, window indices and routed gradients bit-exact."""
import numpy as np
import pytest

import oracle
from util import with_ties, idx_nchw_to_ref

pytestmark = pytest.mark.gpu

CASES = [  # n c h w k sh sw pad
    (2, 3, 7, 7, 3, 2, 2, 1),
    (3, 5, 16, 12, 3, 2, 2, 1),      # vectorised 3x3/2/1 path (W % 4 == 0, H even)
    (2, 4, 112, 112, 3, 2, 2, 1),    # the benchmark max-pool geometry, fewer images
    (1, 2, 8, 8, 2, 2, 2, 0),
    (4, 8, 27, 27, 2, 2, 2, 0),      # README net: last row/column dropped
    (1, 2, 9, 7, 3, 1, 1, 1),
    (2, 1, 5, 5, 3, 2, 2, 0),        # shape of tests/gradient_check/xs_pytorch/pooling.py
    (1, 3, 6, 6, 2, 1, 2, 1),
    (1, 1, 9, 9, 3, 3, 3, 2),
    (1, 2, 11, 13, 5, 2, 3, 2),
    (1, 1, 3, 3, 3, 1, 1, 0),        # single window
    (2, 3, 14, 10, 3, 2, 2, 1),      # W % 4 != 0 -> generic path
    (3, 2, 6, 8, 3, 2, 2, 1),        # W % 8 == 0: eight gradient columns per thread, one thread per row pair
    (1, 3, 4, 136, 3, 2, 2, 1),      # ... rows longer than one wavefront's 64 x 8 columns... and a lane at the wave edge
    (5, 7, 6, 8, 3, 2, 2, 1),        # one thread per row pair: 105 row pairs in a single workgroup of the gradient kernel
    (3, 37, 10, 16, 3, 2, 2, 1),     # 555 row pairs for workgroups of 128: a partial last workgroup
    (2, 3, 38, 112, 3, 2, 2, 1),     # 114 row pairs for workgroups of 18: planes change inside a workgroup
    (1, 1, 2, 2056, 3, 2, 2, 1),     # 257 threads per row pair: wider than a workgroup, the per-thread form serves it
]


def _run(gpu, x, k, stride, pad, dy, dx0=None):
    K = gpu.kernels
    dx_ = gpu.to_device(x)
    y, idx = K.maxpool2d_fwd(dx_, k, stride, pad)
    ddy = gpu.to_device(dy)
    if dx0 is None:
        g = K.maxpool2d_bwd(ddy, idx, x.shape, k, stride, pad)
    else:
        g = gpu.to_device(dx0)
        K.maxpool2d_bwd(ddy, idx, x.shape, k, stride, pad, dx=g, accumulate=True)
    return y.numpy(), idx.numpy(), g.numpy()


@pytest.mark.parametrize("n,c,h,w,k,sh,sw,pad", CASES)
def test_pool_bit_exact(gpu, n, c, h, w, k, sh, sw, pad):
    rng = np.random.default_rng(100 + h * w + k)
    x = with_ties(rng, rng.standard_normal((n, c, h, w)).astype(np.float32), 0.2)
    x[0, 0, 0, :] = -np.abs(x[0, 0, 0, :])
    y_ref, am = oracle.max_pool2d_fwd(x, k, (sh, sw), pad)
    dy = rng.standard_normal(y_ref.shape).astype(np.float32)
    dx_ref = oracle.max_pool2d_bwd(dy, am, x.shape, k, (sh, sw), pad, np.zeros_like(x))
    y, idx, dx = _run(gpu, x, k, (sh, sw), pad, dy)
    assert y.tobytes() == y_ref.tobytes()
    np.testing.assert_array_equal(idx_nchw_to_ref(idx), am)
    assert dx.tobytes() == dx_ref.tobytes()
    # accumulate into an existing gradient (what the reference always does)
    dx0 = rng.standard_normal(x.shape).astype(np.float32)
    dx_ref2 = oracle.max_pool2d_bwd(dy, am, x.shape, k, (sh, sw), pad, dx0.copy())
    _, _, dx2 = _run(gpu, x, k, (sh, sw), pad, dy, dx0)
    assert dx2.tobytes() == dx_ref2.tobytes()


def test_pool_golden_fixture(gpu):
    import os
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "conv_pool_small.npz"))
    k, ps, pp = int(g["pool_k"]), tuple(int(v) for v in g["pool_stride"]), int(g["pool_pad"])
    y, idx, dx = _run(gpu, g["pool_x"], k, ps, pp, g["pool_dy"])
    np.testing.assert_array_equal(y, g["pool_y"])
    np.testing.assert_array_equal(idx, g["pool_idx"])
    np.testing.assert_array_equal(dx, g["pool_dx"])


def test_pool_full_size_properties(gpu):
    """The benchmark max-pool configuration at full size (32x64x112x112), checked through size-independent properties
    plus an exact comparison on a slice of images."""
    rng = np.random.default_rng(4)
    n, c, h, w = 32, 64, 112, 112
    x = with_ties(rng, rng.standard_normal((n, c, h, w), dtype=np.float32), 0.05)
    dy = np.random.default_rng(5).standard_normal((n, c, 56, 56), dtype=np.float32)
    y, idx, dx = _run(gpu, x, 3, (2, 2), 1, dy)
    assert idx.max() < 9
    # y equals the padded input at the recorded position
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    r, s = np.divmod(idx.astype(np.int64), 3)
    oh, ow = np.meshgrid(np.arange(56), np.arange(56), indexing="ij")
    picked = xp[np.arange(n)[:, None, None, None], np.arange(c)[None, :, None, None], 2 * oh + r, 2 * ow + s]
    assert picked.tobytes() == y.tobytes()
    # gradient mass is conserved except for windows that chose a pad cell
    on_pad = (2 * oh + r == 0) | (2 * ow + s == 0)
    total = dy[~on_pad].astype(np.float64).sum()
    assert abs(dx.astype(np.float64).sum() - total) < 1e-3 * max(1.0, abs(total)) + 0.5
    # exact comparison on two images
    y_ref, am = oracle.max_pool2d_fwd(x[:2], 3, 2, 1)
    dx_ref = oracle.max_pool2d_bwd(dy[:2], am, x[:2].shape, 3, (2, 2), 1, np.zeros_like(x[:2]))
    assert y[:2].tobytes() == y_ref.tobytes()
    np.testing.assert_array_equal(idx_nchw_to_ref(idx[:2]), am)
    assert dx[:2].tobytes() == dx_ref.tobytes()


def test_pool_rejects_bad_geometry(gpu):
    K = gpu.kernels
    x = gpu.zeros((1, 1, 2, 2))
    with pytest.raises(ValueError):
        K.maxpool2d_fwd(x, 5, (1, 1), 0)
    with pytest.raises(ValueError):
        K.maxpool2d_fwd(x, 2, (0, 1), 0)
