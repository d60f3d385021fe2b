"""Process-wide graph state and flags (counterpart of the reference's xs/core/__global.py:1-6).

The reference switches devices by swapping a global array module (``np`` -> CuPy,
xs/core/__global.py:9).  Here ``USE_CUDA`` only records that new parameters
should be created on the device; each Tensor knows where its own data lives.
"""
INPUTS = None
OUTPUTS = None
GRAPH = None
TRAINING = True
COMPUTE_GRAD = True
USE_CUDA = False


class no_grad:
    """Context manager that switches gradient bookkeeping off (reference xs/utils/common.py:18-26)."""

    def __enter__(self):
        global COMPUTE_GRAD
        self._saved = COMPUTE_GRAD
        COMPUTE_GRAD = False

    def __exit__(self, *exc):
        global COMPUTE_GRAD
        COMPUTE_GRAD = self._saved
