"""Writes tests/golden/conv_pool_small.npz.

Expected outputs come from the brute-force index-formula code in
oracle/brute.py (float64 sums, rounded once to float32 -- the reference's
arithmetic, xs/utils/common.py:37 and xs/core/base.py:73-75), NOT from the
unfold/GEMM restatement that the fixture is later used to check, and not from
running the reference (its tests hold no stored vectors for this path).
Inputs are dyadic rationals (multiples of 1/8 with small magnitude) so that every
float64 sum is exact and the expected values do not depend on summation order.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
from oracle import brute  # noqa: E402


def dyadic(rng, shape, span=16):
    return (rng.integers(-span, span + 1, size=shape) / 8.0).astype(np.float32)


def main():
    rng = np.random.default_rng(2024)
    out = {}
    x = dyadic(rng, (2, 3, 9, 8)); w = dyadic(rng, (5, 3, 3, 3)); b = dyadic(rng, (1, 5))
    stride, pad = (2, 1), 1
    y = brute.conv2d_fwd_brute(x, w, b, stride, pad)
    dy = dyadic(rng, y.shape)
    dx, dw, db = brute.conv2d_bwd_brute(dy, x, w, stride, pad)
    out.update(conv_x=x, conv_w=w, conv_b=b, conv_stride=np.array(stride), conv_pad=np.array(pad),
               conv_y=y.astype(np.float32), conv_dy=dy, conv_dx=dx.astype(np.float32),
               conv_dw=dw.astype(np.float32), conv_db=db.reshape(1, -1).astype(np.float32))
    px = dyadic(rng, (2, 3, 10, 8), span=3)          # few distinct values -> many ties
    px[0, 0, 0, :] = -np.abs(px[0, 0, 0, :]) - 0.125  # negative border row: the zero pad cell wins
    k, ps, pp = 3, (2, 2), 1
    py, pidx = brute.max_pool2d_fwd_brute(px, k, ps, pp)
    pdy = dyadic(rng, py.shape)
    pdx = brute.max_pool2d_bwd_brute(pdy, pidx, px.shape, k, ps, pp)
    out.update(pool_x=px, pool_k=np.array(k), pool_stride=np.array(ps), pool_pad=np.array(pp),
               pool_y=py.astype(np.float32), pool_idx=pidx.astype(np.uint8), pool_dy=pdy,
               pool_dx=pdx.astype(np.float32))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "conv_pool_small.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
