"""Numpy twin of the C oracle, written in per-element form.

The C file walks each block the way llama.cpp's ``dequantize_row_*`` does
(group loops); this file computes, for every output index ``i`` of a block, which
bytes and bit fields feed it.  Two restatements with different structure that
agree bit for bit are the circularity guard asked for by
docs/domain-knowledge/gguf-classic-quant-layout.md:124 of the reference.

Formulas: docs/domain-knowledge/quant-kquant-iq-proprietary.md:45-64,123-154 and
tests/test_diag_q5km_block_bytes.rs:13-39 of the reference.
"""
from __future__ import annotations

import numpy as np

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
BLOCK_SIZE = {Q8_0: 32, Q4_K: 256, Q5_K: 256, Q6_K: 256}
BLOCK_BYTES = {Q8_0: 34, Q4_K: 144, Q5_K: 176, Q6_K: 210}


def row_bytes(dtype: int, k: int) -> int:
    bs = BLOCK_SIZE[dtype]
    return -(-k // bs) * BLOCK_BYTES[dtype]


def _f16(col: np.ndarray) -> np.ndarray:
    """Two little-endian bytes per row -> float32 (numpy's half conversion is IEEE exact)."""
    return np.ascontiguousarray(col).view("<f2").astype(np.float32).reshape(-1)


def scale_min_k4(scales: np.ndarray):
    """scales: (nb, 12) uint8 -> (sc, m) each (nb, 8) uint8."""
    s = scales.astype(np.uint8)
    sc = np.empty((s.shape[0], 8), np.uint8)
    mn = np.empty((s.shape[0], 8), np.uint8)
    for j in range(8):
        if j < 4:
            sc[:, j] = s[:, j] & 63
            mn[:, j] = s[:, j + 4] & 63
        else:
            sc[:, j] = (s[:, j + 4] & 0x0F) | ((s[:, j - 4] >> 6) << 4)
            mn[:, j] = (s[:, j + 4] >> 4) | ((s[:, j] >> 6) << 4)
    return sc, mn


def _blocks(raw, dtype: int) -> np.ndarray:
    raw = np.frombuffer(raw, dtype=np.uint8) if not isinstance(raw, np.ndarray) else raw.reshape(-1).view(np.uint8)
    bb = BLOCK_BYTES[dtype]
    nb = raw.size // bb
    return raw[: nb * bb].reshape(nb, bb)


def _parts_q4_k(raw):
    """(d sc q, dmin m) per element: the two terms whose difference is the weight."""
    b = _blocks(raw, Q4_K)
    d, dmin = _f16(b[:, 0:2]), _f16(b[:, 2:4])
    sc, mn = scale_min_k4(b[:, 4:16])
    qs = b[:, 16:144]
    i = np.arange(256)
    sub, l = i // 32, i % 32
    q = (qs[:, 32 * (sub // 2) + l] >> (4 * (sub % 2)).astype(np.uint8)) & 0x0F
    ds = d[:, None] * sc[:, sub].astype(np.float32)
    ms = dmin[:, None] * mn[:, sub].astype(np.float32)
    return ds * q.astype(np.float32), ms


def dequant_q4_k(raw) -> np.ndarray:
    a, ms = _parts_q4_k(raw)
    return (a - ms).astype(np.float32)


def _parts_q5_k(raw):
    b = _blocks(raw, Q5_K)
    d, dmin = _f16(b[:, 0:2]), _f16(b[:, 2:4])
    sc, mn = scale_min_k4(b[:, 4:16])
    qh, qs = b[:, 16:48], b[:, 48:176]
    i = np.arange(256)
    sub, l = i // 32, i % 32
    lo4 = (qs[:, 32 * (sub // 2) + l] >> (4 * (sub % 2)).astype(np.uint8)) & 0x0F
    hi1 = (qh[:, l] >> sub.astype(np.uint8)) & 1
    q = lo4.astype(np.int32) + 16 * hi1.astype(np.int32)
    ds = d[:, None] * sc[:, sub].astype(np.float32)
    ms = dmin[:, None] * mn[:, sub].astype(np.float32)
    return ds * q.astype(np.float32), ms


def dequant_q5_k(raw) -> np.ndarray:
    a, ms = _parts_q5_k(raw)
    return (a - ms).astype(np.float32)


def _parts_q6_k(raw):
    """(d s, q - 32) per element: the weight is their product."""
    b = _blocks(raw, Q6_K)
    ql, qh = b[:, 0:128], b[:, 128:192]
    sc = b[:, 192:208].view(np.int8)
    d = _f16(b[:, 208:210])
    i = np.arange(256)
    n, quarter, l = i // 128, (i % 128) // 32, i % 32
    lo4 = (ql[:, 64 * n + l + 32 * (quarter % 2)] >> (4 * (quarter >= 2)).astype(np.uint8)) & 0x0F
    hi2 = (qh[:, 32 * n + l] >> (2 * quarter).astype(np.uint8)) & 3
    q = lo4.astype(np.int32) + 16 * hi2.astype(np.int32) - 32
    s = sc[:, 8 * n + l // 16 + 2 * quarter].astype(np.float32)
    return d[:, None] * s, q.astype(np.float32)


def dequant_q6_k(raw) -> np.ndarray:
    ds, q = _parts_q6_k(raw)
    return (ds * q).astype(np.float32)


def dequant_q8_0(raw) -> np.ndarray:
    b = _blocks(raw, Q8_0)
    d = _f16(b[:, 0:2])
    return (d[:, None] * b[:, 2:34].view(np.int8).astype(np.float32)).astype(np.float32)


_DEQ = {Q4_K: dequant_q4_k, Q5_K: dequant_q5_k, Q6_K: dequant_q6_k, Q8_0: dequant_q8_0}


def dequantize(raw, dtype: int) -> np.ndarray:
    """Flat float32 array of all whole blocks in ``raw``."""
    return _DEQ[dtype](raw).reshape(-1)


def term_magnitudes(raw, dtype: int) -> np.ndarray:
    """Per element, the sum of the magnitudes of the terms a fused kernel may form separately
    before they cancel into the weight: |d sc q| + |dmin m| for Q4_K and Q5_K (the weight is
    their difference), |d s| (q + 32) + 32 |d s| with the unsigned 6-bit q for Q6_K (the weight is
    d s (q - 32)), |d q| for Q8_0.  Never below |weight|; the rounding errors of a kernel that
    multiplies the quants and the offsets apart are bounded in terms of this, not of |weight|.
    Flat float64 array over all whole blocks of ``raw``."""
    if dtype == Q4_K or dtype == Q5_K:
        a, ms = (_parts_q4_k if dtype == Q4_K else _parts_q5_k)(raw)
        return (np.abs(a.astype(np.float64)) + np.abs(ms.astype(np.float64))).reshape(-1)
    if dtype == Q6_K:
        ds, q = _parts_q6_k(raw)
        return (np.abs(ds.astype(np.float64)) * (q.astype(np.float64) + 64.0)).reshape(-1)
    return np.abs(dequant_q8_0(raw).astype(np.float64)).reshape(-1)


def quantized_matmul(w, x: np.ndarray, dtype: int, m: int, n: int, k: int) -> np.ndarray:
    """y[m,n] = x[m,k] . deq(W)[n,k]^T with float64 products and sums, returned as float64."""
    bs = BLOCK_SIZE[dtype]
    kp = -(-k // bs) * bs
    wf = dequantize(w, dtype).reshape(n, kp)[:, :k].astype(np.float64)
    return np.asarray(x, np.float64).reshape(m, k) @ wf.T


def bf16_rne(a: np.ndarray) -> np.ndarray:
    """float32 -> nearest bf16 (ties to even) -> float32."""
    u = np.asarray(a, np.float32).view(np.uint32)
    r = (u + (0x7FFF + ((u >> 16) & 1))) & 0xFFFF0000
    return r.astype(np.uint32).view(np.float32)


ELEM_F32, ELEM_F16, ELEM_BF16 = 0, 1, 2


def elem_bits_to_f32(bits: np.ndarray, elem: int) -> np.ndarray:
    """Activations of a 16-bit element type (their bit patterns) as float32: exact in both types
    (half::f16::to_f32 / half::bf16::to_f32, the Element conversions behind Backend<E>,
    src/compat/mod.rs:376-378 and src/compat/jit_helpers.rs:35-50 of the reference)."""
    b = np.asarray(bits, np.uint16)
    if elem == ELEM_F16:
        return b.view(np.float16).astype(np.float32)
    return (b.astype(np.uint32) << 16).view(np.float32)


def f32_to_elem_bits(y: np.ndarray, elem: int) -> np.ndarray:
    """float32 results as bit patterns of a 16-bit element type: nearest, ties to even
    (E::from_f32); f16 through numpy's IEEE conversion, bf16 through bf16_rne above (known answers
    1.0 -> 0x3F80, -1.0 -> 0xBF80, src/compat/weight_helpers.rs:1202-1215).  NaN patterns are
    whatever the conversion leaves: compare them as NaN, not bit for bit."""
    v = np.asarray(y, np.float32)
    if elem == ELEM_F16:
        with np.errstate(over="ignore"):
            return v.astype(np.float16).view(np.uint16)
    out = (bf16_rne(v).view(np.uint32) >> 16).astype(np.uint16)
    nan = np.isnan(v)
    out[nan] = ((v.view(np.uint32)[nan] >> 16) | 0x40).astype(np.uint16)
    return out


def softmax(logits: np.ndarray) -> np.ndarray:
    z = np.asarray(logits, np.float32)
    e = np.exp(z - z.max())
    s = e.sum(dtype=np.float32)
    return (e / s).astype(np.float32) if s > 0 else np.full_like(z, 1.0 / z.size)


def topk_with_weights(logits: np.ndarray, k: int):
    p = softmax(logits)
    order = np.argsort(-p, kind="stable")[:k]
    w = p[order]
    s = w.sum(dtype=np.float32)
    if s > 0:
        w = w / s
    return order.astype(np.uint32), w.astype(np.float32)
