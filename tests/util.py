"""Shared helpers for the tests: seeded inputs and error measures."""
import numpy as np


def q8_weights(rng, N, K, lo=0.001, hi=0.01):
    """Random Q8_0 matrix as GGUF blocks (uint8 [N, K/32*34]) the way
    the single-GEMV benchmark configuration describes it: int8 uniform in [-127,127], fp16 scale
    uniform in (lo, hi).  Returns (raw, dequantised float64 [N, nb*32])."""
    nb = (K + 31) // 32
    q = rng.integers(-127, 128, size=(N, nb, 32), dtype=np.int8)
    if K % 32:
        q[:, -1, K % 32:] = 0
    d = rng.uniform(lo, hi, size=(N, nb)).astype(np.float16)
    raw = np.empty((N, nb, 34), np.uint8)
    raw[:, :, :2] = d.view(np.uint8).reshape(N, nb, 2)
    raw[:, :, 2:] = q.view(np.uint8)
    deq = (q.astype(np.float64) * d.astype(np.float64)[:, :, None]).reshape(N, nb * 32)
    return raw.reshape(N, nb * 34), deq


def rel_err(got, want):
    """max |got-want| / max(|want|, floor) with the floor at 1e-2 of the
    largest reference magnitude, so near-zero outputs do not dominate."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    floor = max(np.abs(want).max() * 1e-2, 1e-6)
    return float(np.max(np.abs(got - want) / np.maximum(np.abs(want), floor)))


def ulp_diff_f16(a, b):
    """distance in fp16 ulps between two float16 arrays (same sign assumed
    near zero is handled through the monotone integer mapping)."""
    def key(x):
        u = np.ascontiguousarray(x, np.float16).view(np.uint16).astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7fff), u)
    return np.abs(key(a) - key(b))


def within_one_ulp_or_cancelled(got, want, frac=1e-3):
    """True where two fp16 results of the same sum agree to one ulp, or, for a
    sum whose terms cancel to a value far below the row's scale, to `frac` of
    the largest magnitude in `want`: fp32 partial sums taken in another order
    differ by rounding noise of the TERMS, which can exceed one ulp of a tiny
    result."""
    g = np.asarray(got, np.float64)
    w = np.asarray(want, np.float64)
    return (ulp_diff_f16(got, want) <= 1) | (np.abs(g - w) <= frac * np.abs(w).max())

