"""Seeded synthetic GGUF blocks and activations for the benchmark configurations.

Block field distributions: super-block scales ``d``/``dmin`` are f16 of a uniform draw,
every packed byte (6-bit scale field, nibbles, high-bit planes) is uniform, Q6_K
sub-block scales are int8 uniform in [-64, 63], activations are N(0, 1) float32.
Every byte pattern of the packed fields is a valid encoding, so uniform bytes give
uniform 6-bit scales/mins and uniform quants.
"""
from __future__ import annotations

import numpy as np

from .ggml import GgmlDType, block_bytes, block_size, row_bytes


def _rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed))


def _f16_bytes(rng, n: int, lo: float, hi: float) -> np.ndarray:
    return rng.uniform(lo, hi, size=n).astype(np.float16).view(np.uint8).reshape(n, 2)


def random_blocks(dtype: int, n_blocks: int, seed: int = 0) -> np.ndarray:
    """``n_blocks`` random blocks of ``dtype`` as a flat uint8 array."""
    dtype = int(dtype)
    rng = _rng(seed)
    bb = block_bytes(dtype)
    b = rng.integers(0, 256, size=(n_blocks, bb), dtype=np.uint8)
    if dtype in (GgmlDType.Q4_K, GgmlDType.Q5_K):
        b[:, 0:2] = _f16_bytes(rng, n_blocks, 0.001, 0.05)
        b[:, 2:4] = _f16_bytes(rng, n_blocks, 0.001, 0.05)
    elif dtype == GgmlDType.Q6_K:
        b[:, 192:208] = rng.integers(-64, 64, size=(n_blocks, 16), dtype=np.int8).view(np.uint8)
        b[:, 208:210] = _f16_bytes(rng, n_blocks, 0.001, 0.02)
    elif dtype == GgmlDType.Q8_0:
        b[:, 0:2] = _f16_bytes(rng, n_blocks, 0.001, 0.05)
    else:
        raise NotImplementedError(f"random_blocks: ggml dtype {dtype}")
    return b.reshape(-1)


def random_weight(dtype: int, n: int, k: int, seed: int = 0) -> np.ndarray:
    """An [n x k] weight as n rows of whole blocks (rows padded to the block size)."""
    bs = block_size(dtype)
    per_row = -(-k // bs)
    w = random_blocks(dtype, n * per_row, seed)
    assert w.size == n * row_bytes(dtype, k)
    return w


def random_activations(m: int, k: int, seed: int = 0) -> np.ndarray:
    return _rng(seed + 0x5EED).standard_normal((m, k), dtype=np.float32)


def random_gate_logits(tokens: int, experts: int, seed: int = 0) -> np.ndarray:
    return _rng(seed + 0x10617).standard_normal((tokens, experts), dtype=np.float32)
