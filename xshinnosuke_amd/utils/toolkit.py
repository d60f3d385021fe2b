"""Central-difference gradient check (the technique of the reference's xs/utils/toolkit.py:160-194)."""
import numpy as np


def gradient_check(loss_fn, tensors, eps=1e-4):
    """For each host Tensor in ``tensors`` compare its analytic ``grad`` (already computed by the caller)
    with central differences of ``loss_fn()`` (a callable returning a float).  Returns the list of
    Euclidean distances."""
    dists = []
    for t in tensors:
        a = t.eval
        num = np.zeros_like(a)
        it = np.nditer(a, flags=['multi_index'])
        for _ in it:
            i = it.multi_index
            old = a[i]
            a[i] = old + eps
            lp = loss_fn()
            a[i] = old - eps
            lm = loss_fn()
            a[i] = old
            num[i] = (lp - lm) / (2 * eps)
        dists.append(float(np.linalg.norm(num - t.grad.eval)))
    return dists
