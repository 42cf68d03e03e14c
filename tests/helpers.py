"""Shared comparison helpers for the parity tests."""
import numpy as np


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    d = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / d) if d > 0 else float(np.linalg.norm(a - b))


def ulp_diff_f16(a, b):
    """Distance in fp16 representable steps between two fp16 arrays (finite values)."""

    def key(x):
        u = np.asarray(x, dtype=np.float16).view(np.uint16).astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7FFF), u)

    return np.abs(key(a) - key(b))


def f16(bits):
    return np.asarray(bits, dtype=np.uint16).view(np.float16)
