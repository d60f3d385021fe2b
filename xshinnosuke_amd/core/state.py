"""Process-wide graph state and flags (counterpart of the reference's xs/core/__global.py:1-6).

The reference switches devices by swapping a global array module (``np`` -> CuPy,
xs/core/__global.py:9).  Here ``USE_CUDA`` only records that new parameters
should be created on the device; each Tensor knows where its own data lives.
"""
import os as _os

INPUTS = None
OUTPUTS = None
GRAPH = None
TRAINING = True
COMPUTE_GRAD = True
USE_CUDA = False
# Opt-in: convolutions may round their MFMA operands to bf16 (fp32 accumulate).  Off by
# default; the reference has no counterpart (its GEMMs run in float64).
CONV_BF16 = False
# Opt-in (also XSMI_STEP_GRAPH=1 in the environment): fit() on device-resident data records its full-batch training
# step once as a step graph and replays it for every later full batch (backend/graph.py); a shorter last batch
# runs launch by launch as before.  No counterpart in the reference.
STEP_GRAPH = _os.environ.get("XSMI_STEP_GRAPH", "0") not in ("", "0")


class no_grad:
    """Context manager that switches gradient bookkeeping off (reference xs/utils/common.py:18-26)."""

    def __enter__(self):
        global COMPUTE_GRAD
        self._saved = COMPUTE_GRAD
        COMPUTE_GRAD = False

    def __exit__(self, *exc):
        global COMPUTE_GRAD
        COMPUTE_GRAD = self._saved


class conv_precision:
    """``with conv_precision('bf16'):`` lets conv2d forward / backward-data use bf16 MFMA operands
    inside the block; ``'fp32'`` restores the default.  No counterpart in the reference."""

    def __init__(self, mode):
        if mode not in ('fp32', 'bf16'):
            raise ValueError("conv_precision: mode must be 'fp32' or 'bf16', got %r" % (mode,))
        self._mode = mode

    def __enter__(self):
        global CONV_BF16
        self._saved = CONV_BF16
        CONV_BF16 = self._mode == 'bf16'

    def __exit__(self, *exc):
        global CONV_BF16
        CONV_BF16 = self._saved
