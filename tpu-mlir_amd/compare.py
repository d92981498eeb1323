"""Tensor similarity metrics used to accept a backend against the CPU interpreter
(python/numpy_helper/tensor_compare.py:65-83,160-191 in the reference)."""
import numpy as np


def _prep(x):
    x = np.asarray(x, dtype=np.float64).reshape(-1).copy()
    x[np.isnan(x)] = 0.0
    x[np.isposinf(x)] = 10000.0
    x[np.isneginf(x)] = -10000.0
    return x


def cosine_similarity(a, b):
    a, b = _prep(a), _prep(b)
    na, nb = np.linalg.norm(a), np.linalg.norm(b)
    if na == 0.0 or nb == 0.0:  # the reference reports 0.0 when either side is all zero
        return 0.0
    return float(np.dot(a, b) / (na * nb))


def euclidean_similarity(a, b):
    a, b = _prep(a), _prep(b)
    return float(1.0 - np.linalg.norm(a - b) / (np.linalg.norm((a + b) / 2.0) + 1e-7))


def sqnr(raw, deq):
    raw, deq = _prep(raw), _prep(deq)
    noise = raw - deq
    vr, vn = np.var(raw), np.var(noise)
    if vn == 0.0 or vr == 0.0:
        return float("inf")
    return float(10.0 * np.log10(vr / vn))


def max_abs_over_rms(got, want):
    """The bf16-path acceptance metric: max |got - want| / RMS(want)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    rms = np.sqrt(np.mean(want * want))
    return float(np.max(np.abs(got - want)) / (rms if rms > 0 else 1.0))
