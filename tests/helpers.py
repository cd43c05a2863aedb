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


def max_rel_err(got, ref, eps=None):
    """max |got-ref| / max(|ref|, eps) with eps = max(1e-3, 1% of the largest |ref|).

    The floor is needed because ReLU-like inputs and cancelling sums give outputs at or near zero, where two
    correct fp32 summation orders differ by a few 1e-8 absolute; tying it to the tensor's scale keeps the bar
    at 1e-6 of the largest output.  (The reference's own predicate allows 1e-5 absolute, tensor_utils.cc:17-19.)
    """
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    if not ref.size:
        return 0.0
    if eps is None:
        eps = max(1e-3, 1e-2 * float(np.max(np.abs(ref))))
    return float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), eps)))
