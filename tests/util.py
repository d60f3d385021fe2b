import numpy as np


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    den = np.linalg.norm(b.ravel())
    num = np.linalg.norm((a - b).ravel())
    return num / den if den > 0 else num


def he_normal(rng, shape):
    """He-normal filter (std = sqrt(2 / fan_in)), fan_in = C*R*S (reference xs/nn/initializers.py:11-21, 88-94)."""
    fan_in = int(np.prod(shape[1:]))
    return (rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(np.float32)


def with_ties(rng, x, frac=0.05):
    """Overwrite a fraction of positions with their right-hand neighbour (wrapping inside the row)."""
    x = x.copy()
    flat_rows = x.reshape(-1, x.shape[-1])
    n = flat_rows.size
    pick = rng.choice(n, size=int(n * frac), replace=False)
    r, c = np.divmod(pick, x.shape[-1])
    flat_rows[r, c] = flat_rows[r, (c + 1) % x.shape[-1]]
    return x


def idx_nchw_to_ref(idx_nchw):
    """uint8 NCHW window indices -> the reference's flat int64 vector over (n, oh, ow, c)."""
    return np.ascontiguousarray(idx_nchw.transpose(0, 2, 3, 1)).reshape(-1).astype(np.int64)


def idx_ref_to_nchw(argmax, n, c, oh, ow):
    return np.ascontiguousarray(argmax.reshape(n, oh, ow, c).transpose(0, 3, 1, 2))


def round_bf16(a):
    """float32 array rounded to the nearest bf16 value (ties to even), returned as float32."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))
