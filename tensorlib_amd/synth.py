"""Deterministic synthetic inputs for the parity tests and the benchmark.

The reference's own ``randn`` is unseeded (tensorLib/src/device/cpu/CPU.cpp:100-115,
tensorLib/src/device/cuda/CUDA.cu:51-69), so "identical seeded inputs" come from here:
a Philox counter-based stream -> standard normal in fp32 -> scale -> round to fp16.
"""
from __future__ import annotations

import numpy as np


def normal_f16(seed: int, shape, std: float = 1.0) -> np.ndarray:
    """N(0, std^2) samples rounded to fp16; the same (seed, shape, std) always gives the same bits."""
    rng = np.random.Generator(np.random.Philox(key=int(seed)))
    x = rng.standard_normal(size=shape, dtype=np.float32)
    if std != 1.0:
        x *= np.float32(std)
    return x.astype(np.float16)


def small_ints_f16(seed: int, shape, lo: int = -3, hi: int = 3) -> np.ndarray:
    """Integer-valued fp16 samples in [lo, hi]: products and short sums are exact in fp32 and fp16."""
    rng = np.random.Generator(np.random.Philox(key=int(seed)))
    return rng.integers(lo, hi + 1, size=shape).astype(np.float16)


def token_ids(seed: int, n: int, vocab: int, lo: int = 3) -> np.ndarray:
    rng = np.random.Generator(np.random.Philox(key=int(seed)))
    return rng.integers(lo, vocab, size=n).astype(np.int32)


def gemv_bytes(N: int, K: int) -> int:
    """Algorithmic HBM bytes of one fp16 GEMV: W once, x once, y once."""
    return 2 * N * K + 2 * K + 2 * N


def gemm_flops(M: int, N: int, K: int) -> int:
    return 2 * M * N * K


def gemm_min_bytes(M: int, N: int, K: int) -> int:
    return 2 * (M * K + N * K + M * N)
