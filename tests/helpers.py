"""Seeded synthetic tensors shared by the tests (kept tiny so the CPU suite stays fast)."""
import numpy as np


def sparse_filter(rng, K, C, ks, sparsity, neg_zero=True):
    w = rng.normal(0.0, 0.05, size=(K, C, ks, ks)).astype(np.float32)
    n = w.size
    zeros = rng.permutation(n)[: int(round(sparsity * n))]
    flat = w.reshape(-1)
    flat[zeros] = 0.0
    if neg_zero and len(zeros):
        flat[zeros[::3]] = -0.0  # the shipped weight files are full of "-0.0"
    return w


def relu_like(rng, shape):
    x = rng.random(shape, dtype=np.float32)
    x[rng.random(shape) < 0.5] = 0.0
    return x


def max_rel_err(got, ref, eps=1e-3):
    """max |got-ref| / max(|ref|, eps): the denominator floor keeps exact-zero outputs meaningful."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), eps))) if ref.size else 0.0
