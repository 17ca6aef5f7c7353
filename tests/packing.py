"""Encoders used by the tests to build blocks with chosen field values.

They are written from the *quantizer* side of the published format (llama.cpp's
quantize_row_q4_K_ref / quantize_row_q6_K_ref packing statements), i.e. independently of
the decoders under test: a decoder with a wrong index, shift or plane fails the round trip.
"""
import numpy as np


def pack_scales_k4(sc, mn) -> np.ndarray:
    """8 six-bit scales + 8 six-bit mins -> the 12-byte field of Q4_K/Q5_K."""
    q = np.zeros(12, np.uint8)
    for j in range(8):
        ls, lm = int(sc[j]), int(mn[j])
        assert 0 <= ls < 64 and 0 <= lm < 64
        if j < 4:
            q[j] |= ls
            q[j + 4] |= lm
        else:
            q[j + 4] |= (ls & 0xF) | ((lm & 0xF) << 4)
            q[j - 4] |= (ls >> 4) << 6
            q[j] |= (lm >> 4) << 6
    return q


def f16_bytes(v: float) -> np.ndarray:
    return np.array([v], np.float16).view(np.uint8)


def pack_q4_k(d, dmin, sc, mn, q) -> np.ndarray:
    """q: 256 ints in 0..15."""
    q = np.asarray(q, np.int64).reshape(4, 2, 32)
    b = np.zeros(144, np.uint8)
    b[0:2], b[2:4] = f16_bytes(d), f16_bytes(dmin)
    b[4:16] = pack_scales_k4(sc, mn)
    b[16:144] = (q[:, 0, :] | (q[:, 1, :] << 4)).astype(np.uint8).reshape(-1)
    return b


def pack_q5_k(d, dmin, sc, mn, q) -> np.ndarray:
    """q: 256 ints in 0..31."""
    q = np.asarray(q, np.int64).reshape(8, 32)
    b = np.zeros(176, np.uint8)
    b[0:2], b[2:4] = f16_bytes(d), f16_bytes(dmin)
    b[4:16] = pack_scales_k4(sc, mn)
    qh = np.zeros(32, np.int64)
    for sub in range(8):
        qh |= ((q[sub] >> 4) & 1) << sub
    b[16:48] = qh.astype(np.uint8)
    lo = (q & 0xF).reshape(4, 2, 32)
    b[48:176] = (lo[:, 0, :] | (lo[:, 1, :] << 4)).astype(np.uint8).reshape(-1)
    return b


def pack_q6_k(d, scales, q) -> np.ndarray:
    """q: 256 ints in -32..31, scales: 16 int8."""
    u = (np.asarray(q, np.int64) + 32).reshape(2, 4, 32)  # [half][quarter][l]
    b = np.zeros(210, np.uint8)
    for h in range(2):
        lo = u[h] & 0xF
        hi = u[h] >> 4
        b[64 * h: 64 * h + 32] = (lo[0] | (lo[2] << 4)).astype(np.uint8)
        b[64 * h + 32: 64 * h + 64] = (lo[1] | (lo[3] << 4)).astype(np.uint8)
        b[128 + 32 * h: 128 + 32 * h + 32] = (hi[0] | (hi[1] << 2) | (hi[2] << 4) | (hi[3] << 6)).astype(np.uint8)
    b[192:208] = np.asarray(scales, np.int8).view(np.uint8)
    b[208:210] = f16_bytes(d)
    return b


def pack_q8_0(d, q) -> np.ndarray:
    b = np.zeros(34, np.uint8)
    b[0:2] = f16_bytes(d)
    b[2:34] = np.asarray(q, np.int8).view(np.uint8)
    return b
