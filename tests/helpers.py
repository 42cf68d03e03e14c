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


def assert_close_f16(got, want, ulps=2, floor=2e-4):
    """Each element within `ulps` fp16 steps of `want`, or within floor * rms(want) absolutely.

    The absolute floor covers outputs that land near zero through cancellation, where an fp32
    summation-order difference of ~1e-6 of the operand magnitude spans many fp16 steps.
    """
    got = np.asarray(got, dtype=np.float16)
    want = np.asarray(want, dtype=np.float16)
    d = ulp_diff_f16(got, want)
    rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    absd = np.abs(got.astype(np.float64) - want.astype(np.float64))
    bad = (d > ulps) & (absd > floor * rms)
    assert not bad.any(), f"{int(bad.sum())} elements differ: worst {int(d[bad].max())} steps, abs {absd[bad].max():.3g} (rms {rms:.3g})"
