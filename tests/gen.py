"""Seeded synthetic inputs shared by the CPU oracle and the GPU tests.

numpy's Philox bit generator is counter based and platform independent, so the
same seed gives the same fp16 bits here and on the GPU box.
"""
from __future__ import annotations

import numpy as np


def rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.Philox(seed))


def normal_f16(r: np.random.Generator, shape, scale: float = 1.0) -> np.ndarray:
    return (r.standard_normal(shape, dtype=np.float32) * np.float32(scale)).astype(np.float16)


def kv_rows_with_outliers(r: np.random.Generator, shape, kv_dim: int, frac: float = 0.01, gain: float = 8.0):
    """fp16 N(0,1) rows with a fixed 1 % of the kv_dim channels scaled by 8."""
    x = r.standard_normal(shape, dtype=np.float32)
    n_out = max(1, int(round(frac * kv_dim)))
    chans = r.choice(kv_dim, size=n_out, replace=False)
    x[..., chans] *= np.float32(gain)
    return x.astype(np.float16), np.sort(chans)


def ragged_contexts(r: np.random.Generator, G: int, lo: int, hi: int) -> np.ndarray:
    return r.integers(lo, hi + 1, size=G).astype(np.int32)


def shuffled_block_table(r: np.random.Generator, G: int, pages_per_seq: int):
    """Every sequence gets pages_per_seq distinct pages of a common pool, in random order."""
    perm = r.permutation(G * pages_per_seq).astype(np.int32)
    return perm.reshape(G, pages_per_seq)
