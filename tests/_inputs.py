"""Seeded synthetic inputs shared by the tests, the fixtures and bench.py's CPU leg.

numpy's PCG64 `Generator.standard_normal(dtype=float32)` stream; the fixtures store a
SHA-256 of every generated input so a change of stream is detected rather than absorbed.
"""
import hashlib

import numpy as np


def normal(seed, shape, scale=1.0):
    x = np.random.default_rng(seed).standard_normal(shape, dtype=np.float32)
    if scale != 1.0:
        x = (x * np.float32(scale)).astype(np.float32)
    return x


def qkv(seed, B, Hq, Hkv, T, L, D, scale=1.0):
    """q [B,Hq,T,D], k,v [B,Hkv,L,D] with seeds seed, seed+1, seed+2."""
    return (normal(seed, (B, Hq, T, D), scale), normal(seed + 1, (B, Hkv, L, D), scale),
            normal(seed + 2, (B, Hkv, L, D), scale))


def seq_lens(seed, B, lo, hi):
    """Integer-uniform context lengths in [lo, hi]."""
    return np.random.default_rng(seed).integers(lo, hi + 1, size=B, dtype=np.int64).astype(np.int32)


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()
