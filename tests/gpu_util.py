"""Shared helpers of the GPU parity tests."""
import numpy as np


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64).ravel()
    b = np.asarray(b, dtype=np.float64).ravel()
    d = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / d) if d > 0 else float(np.linalg.norm(a - b))


def gaussian_weights(n, seed, sigma=0.02, outlier_every=0):
    """N(0, sigma) weights (the configs' recipe), optionally with x8 outlier blocks."""
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal(n) * sigma).astype(np.float32)
    if outlier_every:
        nb = n // 256
        for b in range(0, nb, outlier_every):
            w[b * 256:(b + 1) * 256] *= np.float32(8.0)
    return w


def to_orc_blocks(blocks):
    """oilhip_block_t records -> the oracle's descriptor dtype (same fields)."""
    import oracle as O
    out = np.zeros(blocks.size, dtype=O.BLOCK_DTYPE)
    for k in ("cb_off", "idx_off", "cb_bytes", "idx_bytes", "nw", "fmt"):
        out[k] = blocks[k]
    return out
