"""Helpers shared by the tests."""
import numpy as np


def rel_max(a, b):
    """max|a-b| / max|b| over the whole tensor (the norm every parity gate is stated in)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    den = np.abs(b).max()
    return float(np.abs(a - b).max() / (den if den > 0 else 1.0))


def bits_equal(a, b):
    """Bitwise equality of two float arrays (distinguishes +0/-0, compares NaN payloads)."""
    a = np.ascontiguousarray(np.asarray(a))
    b = np.ascontiguousarray(np.asarray(b))
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    it = {4: np.uint32, 8: np.uint64}[a.dtype.itemsize]
    return bool(np.array_equal(a.view(it), b.view(it)))


def count_bit_mismatches(a, b):
    a = np.ascontiguousarray(np.asarray(a))
    b = np.ascontiguousarray(np.asarray(b))
    it = {4: np.uint32, 8: np.uint64}[a.dtype.itemsize]
    return int((a.view(it) != b.view(it)).sum())


def F(a, dtype=np.float32):
    return np.asfortranarray(a, dtype=dtype)
