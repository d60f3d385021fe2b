"""CPU oracle for the conv / max-pool hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; it is used by ``tests/``, by ``__graft_entry__.smoke()`` as the
checker, and by ``bench.py``'s ``cpu_baseline`` leg as the thing timed on the
host cores.  The product path never routes through it.
"""
from .xs_oracle import (  # noqa: F401
    im2col, col2im, conv2d_fwd, conv2d_bwd, max_pool2d_fwd, max_pool2d_bwd,
    relu_fwd, relu_bwd, out_size,
)
from .brute import (  # noqa: F401
    conv2d_fwd_brute, conv2d_bwd_brute, max_pool2d_fwd_brute, max_pool2d_bwd_brute,
)
