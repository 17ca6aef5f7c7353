"""GGUF block-format constants for the formats on the quantized matmul path.

Mirrors ``GgmlDType`` ids, ``block_size``/``block_bytes`` and the row-size rule of
``tensor_nbytes`` (reference: src/loader/gguf/types.rs:57-94, 152-236, 443-472) and the
dtype -> QuantType names of src/loader/adapter.rs:138-191.
"""
from __future__ import annotations

import enum


class GgmlDType(enum.IntEnum):
    Q8_0 = 8
    Q4_K = 12
    Q5_K = 13
    Q6_K = 14


class QuantType(enum.Enum):
    """Names as in gllm-kernels' ``quant::QuantType``; value = GGUF type id."""
    Q8_0 = 8
    Q4K = 12
    Q5K = 13
    Q6K = 14

    @property
    def ggml_dtype(self) -> int:
        return int(self.value)

    def block_size(self) -> int:
        return block_size(self.value)

    def block_bytes(self) -> int:
        return block_bytes(self.value)


_BLOCK = {8: (32, 34), 12: (256, 144), 13: (256, 176), 14: (256, 210)}


def supported(dtype: int) -> bool:
    return int(dtype) in _BLOCK


def block_size(dtype: int) -> int:
    return _BLOCK[int(dtype)][0]


def block_bytes(dtype: int) -> int:
    return _BLOCK[int(dtype)][1]


def row_bytes(dtype: int, k: int) -> int:
    """Bytes of one weight row of k elements: whole blocks, the last one padded."""
    bs, bb = _BLOCK[int(dtype)]
    return -(-k // bs) * bb


def tensor_nbytes(dtype: int, shape) -> int:
    """GGUF order: shape[0] is the innermost (blocked) dimension."""
    if len(shape) == 0:
        return 0
    total = row_bytes(dtype, int(shape[0]))
    for d in shape[1:]:
        total *= int(d)
    return total
