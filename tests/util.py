"""Shared helpers for the parity tests."""
import numpy as np


def rng(seed):
    return np.random.default_rng(seed)


def randn(r, *shape):
    return r.standard_normal(shape).astype(np.float32)


def max_rel_err(a, b, floor=1e-6):
    """max |a-b| / max(|b|, floor): the 'max relative error' metric for elementwise ops."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.max(np.abs(a - b) / np.maximum(np.abs(b), floor))) if a.size else 0.0


def nl2(a, b):
    """normalised L2 error ||a-b|| / ||b||: the metric for conv / BN reductions."""
    a = np.asarray(a, dtype=np.float64).ravel()
    b = np.asarray(b, dtype=np.float64).ravel()
    d = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / (d if d > 0 else 1.0))


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def assert_bit_equal(a, b, what=""):
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    assert a.shape == b.shape, (what, a.shape, b.shape)
    # +0.0 and -0.0 compare equal here on purpose only if both are zero-valued
    same = (bits(a) == bits(b)) | ((a == 0) & (b == 0))
    assert bool(np.all(same)), "%s: %d of %d elements differ, first at %s" % (
        what, int((~same).sum()), a.size, np.argwhere(~same)[:3].tolist())
