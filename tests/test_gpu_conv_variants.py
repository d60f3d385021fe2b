"""Every fp32 convolution kernel variant the library can select, reached through its tuning switches and compared
with the oracle (relative L2 error <= 1e-5, the fp32 path's bar), and the error path of the even-split kernel's
bounded wait."""
import contextlib

import numpy as np
import pytest

import oracle
from util import rel_l2, he_normal

pytestmark = pytest.mark.gpu
TOL = 1e-5


@contextlib.contextmanager
def options(gpu, **kv):
    old = {k: gpu.set_option(k, v) for k, v in kv.items()}
    try:
        yield
    finally:
        for k, v in old.items():
            gpu.set_option(k, v)


def _run(gpu, n, c, h, w, k, r, s, sh, sw, pad, seed=5):
    """forward with bias / ReLU / mask and accumulating backward-data, each against the oracle"""
    K = gpu.kernels
    rng = np.random.default_rng(seed + c + k + h)
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    wt = he_normal(rng, (k, c, r, s))
    b = rng.standard_normal((k,)).astype(np.float32)
    oh, ow = K.conv_out_hw(h, w, r, s, (sh, sw), pad)
    dy = rng.standard_normal((n, k, oh, ow)).astype(np.float32)
    dx0 = rng.standard_normal(x.shape).astype(np.float32)
    y_ref, col = oracle.conv2d_fwd(x, wt, b, (sh, sw), pad)
    dx_ref, _, _ = oracle.conv2d_bwd(dy, x.shape, wt, col, (sh, sw), pad, dx0.copy(), np.zeros_like(wt),
                                     np.zeros((k,), dtype=np.float32))
    dx_, dw_, db_, ddy = gpu.to_device(x), gpu.to_device(wt), gpu.to_device(b), gpu.to_device(dy)
    y = K.conv2d_fwd(dx_, dw_, db_, (sh, sw), pad).numpy()
    assert rel_l2(y, y_ref) <= TOL
    mask = gpu.empty(y.shape, np.uint8)
    act = K.conv2d_fwd(dx_, dw_, db_, (sh, sw), pad, relu=True, neg_mask=mask).numpy()
    np.testing.assert_array_equal(act, np.maximum(y, 0.0))
    np.testing.assert_array_equal(mask.numpy(), (y < 0).astype(np.uint8))
    gx = gpu.to_device(dx0)
    K.conv2d_bwd_data(ddy, dw_, x.shape, (sh, sw), pad, dx=gx, accumulate=True)
    assert rel_l2(gx.numpy(), dx_ref) <= TOL
    return y


GEOMETRIES = [   # n c h w k r s sh sw pad
    (3, 64, 56, 56, 64, 3, 3, 1, 1, 1),      # rows 56 wide: 16-byte activation loads, borders inside every tile
    (5, 128, 28, 28, 128, 3, 3, 1, 1, 1),    # two row tiles
    (2, 64, 12, 20, 70, 3, 3, 1, 1, 1),      # ragged last row tile, pixel tail
    (2, 32, 9, 8, 64, 3, 3, 1, 1, 0),        # no padding: taps reach no border, input wider than output
    (3, 256, 14, 14, 256, 3, 3, 1, 1, 1),    # rows not a multiple of four pixels: one-dword loads
    (2, 64, 28, 28, 128, 3, 3, 2, 2, 1),     # strided: four residue classes in the backward pass
    (2, 512, 7, 7, 512, 3, 3, 1, 1, 1),      # fewer tiles than compute units: every tile split many ways
    (2, 64, 16, 16, 64, 1, 1, 1, 1, 0),      # 1 x 1
    (2, 32, 6, 112, 32, 3, 3, 1, 1, 1),      # rows longer than a tile of 64 pixels
    (3, 32, 7, 24, 96, 3, 3, 1, 1, 1),       # short images: tiles that span two images, 16-channel units in twos
    (2, 32, 9, 3, 64, 3, 3, 1, 1, 1),        # rows of three pixels: one-dword pieces, 21 row ends inside a tile
    (5, 32, 3, 2, 64, 3, 3, 1, 1, 1),        # rows of two pixels, images of six: a tile spans eleven images
]


@pytest.mark.parametrize("tap_sk,sk_wide", [(3, 3), (3, 2), (3, 1), (3, 0), (1, 2), (0, 2)])
@pytest.mark.parametrize("geom", GEOMETRIES)
def test_even_split_and_whole_tile_kernels(gpu, geom, tap_sk, sk_wide):
    """tap_sk 3: the even-split kernel wherever it applies (sk_wide 2: input rows staged once for a filter row's three
    taps where that form pays, 3: wherever it applies; 1: 16-byte activation loads tap by tap; 0: one-dword loads);
    1: where the library finds it pays; 0: whole tiles per workgroup only."""
    with options(gpu, tap_sk=tap_sk, sk_wide=sk_wide):
        _run(gpu, *geom)


@pytest.mark.parametrize("tap_persist,tap_stages", [(0, 0), (2, 0), (1, 2), (1, 3), (0, 3)])
@pytest.mark.parametrize("geom", [GEOMETRIES[0], GEOMETRIES[1], GEOMETRIES[4], GEOMETRIES[6]])
def test_whole_tile_kernel_forms(gpu, geom, tap_persist, tap_stages):
    """the whole-tile kernel with and without its persistent form, with two and three load stages"""
    with options(gpu, tap_sk=0, tap_persist=tap_persist, tap_stages=tap_stages):
        _run(gpu, *geom)


def test_wide_and_narrow_loads_give_the_same_bits(gpu):
    """the same chunks in the same order: the width of the activation loads does not touch the arithmetic"""
    with options(gpu, tap_sk=3, sk_wide=1):
        a = _run(gpu, *GEOMETRIES[0])
    with options(gpu, tap_sk=3, sk_wide=0):
        b = _run(gpu, *GEOMETRIES[0])
    assert a.tobytes() == b.tobytes()


def test_a_wait_that_runs_out_is_reported_and_the_library_recovers(gpu):
    """sk_spin_limit 0 makes every wait for a partial tile count as run out: every kernel still finishes, the tiles
    concerned are not stored, and the next call that waits for the device raises; after that the same call with the
    default limit is exact again."""
    K = gpu.kernels
    n, c, h, w, k = 2, 512, 7, 7, 512                    # 16 tiles for 768 workgroups: every tile is split
    rng = np.random.default_rng(3)
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    wt = he_normal(rng, (k, c, 3, 3))
    y_ref, _ = oracle.conv2d_fwd(x, wt, None, (1, 1), 1)
    dx_, dw_ = gpu.to_device(x), gpu.to_device(wt)
    y = gpu.empty(y_ref.shape)
    gpu.synchronize()
    with options(gpu, tap_sk=3, sk_spin_limit=0):
        K.conv2d_fwd(dx_, dw_, None, (1, 1), 1, out=y)
        with pytest.raises(gpu.XsmiError, match="gave up waiting"):
            gpu.synchronize()
        gpu.synchronize()                                 # reported once; the library is usable again
    with options(gpu, tap_sk=3):
        K.conv2d_fwd(dx_, dw_, None, (1, 1), 1, out=y)
        assert rel_l2(y.numpy(), y_ref) <= TOL
        K.conv2d_fwd(dx_, dw_, None, (1, 1), 1, out=y)    # and a second time: no flag was left raised
        assert rel_l2(y.numpy(), y_ref) <= TOL


def test_unknown_option_is_refused(gpu):
    with pytest.raises(ValueError, match="no option named"):
        gpu.set_option("no_such_switch", 1)
