"""Shared synthetic-input builders for the tests (numpy, seeded, machine independent)."""
import numpy as np


def make_kv(B, H, T, D=128, seed=0, outliers=8, student_t=False):
    """K ~ N(0,1) (or Student-t nu=3) with `outliers` channels per head scaled x10; V ~ N(0,1)."""
    rng = np.random.default_rng(seed)
    if student_t:
        k = rng.standard_t(3, size=(B, H, T, D))
    else:
        k = rng.standard_normal((B, H, T, D))
    for h in range(H):
        ch = rng.permutation(D)[:outliers]
        k[:, h, :, ch] *= 10.0
    v = rng.standard_normal((B, H, T, D))
    return k.astype(np.float16), v.astype(np.float16)


def make_q(B, HQ, D=128, seed=0):
    rng = np.random.default_rng(seed + 7919)
    return rng.standard_normal((B, HQ, 1, D)).astype(np.float16)
