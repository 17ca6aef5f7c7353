"""ctypes binding of the C oracle (``libgllmq_oracle.so``, built by ``make -C oracle``).

Test infrastructure only: see ``gllmq_oracle.h`` for what is restated and what pins it.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libgllmq_oracle.so")

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
ACC_F32, ACC_F64 = 0, 1
OK, ERR_UNIMPLEMENTED, ERR_BAD_SHAPE = 0, 1, 2


def build(force: bool = False) -> str:
    """Compile the oracle with its Makefile (needs only gcc)."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        u8p, f32p, u32p = C.POINTER(C.c_uint8), C.POINTER(C.c_float), C.POINTER(C.c_uint32)
        sz = C.c_size_t
        L.gq_block_size.restype = sz
        L.gq_block_size.argtypes = [C.c_uint32]
        L.gq_block_bytes.restype = sz
        L.gq_block_bytes.argtypes = [C.c_uint32]
        L.gq_row_bytes.restype = sz
        L.gq_row_bytes.argtypes = [C.c_uint32, sz]
        L.gq_f16_to_f32.restype = C.c_float
        L.gq_f16_to_f32.argtypes = [C.c_uint16]
        L.gq_f32_to_bf16_rne.restype = C.c_uint16
        L.gq_f32_to_bf16_rne.argtypes = [C.c_float]
        L.gq_scale_min_k4.restype = None
        L.gq_scale_min_k4.argtypes = [C.c_int, u8p, u8p, u8p]
        L.gq_dequantize.restype = C.c_int
        L.gq_dequantize.argtypes = [u8p, sz, f32p, sz, C.c_uint32]
        L.gq_quant_gather.restype = C.c_int
        L.gq_quant_gather.argtypes = [u8p, C.c_uint32, sz, sz, u32p, sz, C.c_float, C.c_int, f32p]
        L.gq_ffn_swiglu.restype = C.c_int
        L.gq_ffn_swiglu.argtypes = [u8p, u8p, C.c_uint32, u8p, C.c_uint32, f32p, f32p, sz, sz, sz, C.c_int, C.c_int, C.c_int]
        L.gq_argmax_token.restype = C.c_int64
        L.gq_argmax_token.argtypes = [f32p, sz]
        L.gq_quantized_matmul.restype = C.c_int
        L.gq_quantized_matmul.argtypes = [u8p, f32p, f32p, C.c_uint32, sz, sz, sz, C.c_int, C.c_int]
        L.gq_quantized_matmul_bf16.restype = C.c_int
        L.gq_quantized_matmul_bf16.argtypes = [u8p, f32p, f32p, C.c_uint32, sz, sz, sz, C.c_int]
        L.gq_quantized_matmul_avx2.restype = C.c_int
        L.gq_quantized_matmul_avx2.argtypes = [u8p, f32p, f32p, C.c_uint32, sz, sz, sz, C.c_int]
        L.gq_have_avx2.restype = C.c_int
        L.gq_have_avx2.argtypes = []
        L.gq_dequant_block_avx2.restype = C.c_int
        L.gq_dequant_block_avx2.argtypes = [C.c_uint32, u8p, f32p]
        L.gq_quantized_matmul_avx512.restype = C.c_int
        L.gq_quantized_matmul_avx512.argtypes = [u8p, f32p, f32p, C.c_uint32, sz, sz, sz, C.c_int]
        L.gq_have_avx512.restype = C.c_int
        L.gq_have_avx512.argtypes = []
        L.gq_dequant_block_avx512.restype = C.c_int
        L.gq_dequant_block_avx512.argtypes = [C.c_uint32, u8p, f32p]
        L.gq_softmax.restype = None
        L.gq_softmax.argtypes = [f32p, sz, f32p]
        L.gq_topk_with_weights.restype = sz
        L.gq_topk_with_weights.argtypes = [f32p, sz, sz, u32p, f32p]
        L.gq_topk_indices.restype = sz
        L.gq_topk_indices.argtypes = [f32p, sz, sz, u32p]
        L.gq_expert_capacity.restype = sz
        L.gq_expert_capacity.argtypes = [C.c_float, sz, sz]
        L.gq_route.restype = sz
        L.gq_route.argtypes = [f32p, sz, sz, sz, C.c_float, u32p, f32p, u32p, u32p, u32p]
        L.gq_moe_ffn.restype = C.c_int
        L.gq_moe_ffn.argtypes = [u8p, C.c_uint32, u8p, C.c_uint32, f32p, f32p, sz, sz, sz, sz, sz,
                                 u32p, f32p, u32p, C.c_int, C.c_int, C.c_int]
        _lib = L
    return _lib


def _u8(a):
    return a.ctypes.data_as(C.POINTER(C.c_uint8))


def _f32(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _u32(a):
    return a.ctypes.data_as(C.POINTER(C.c_uint32))


def _bytes_arr(raw) -> np.ndarray:
    if isinstance(raw, np.ndarray):
        return np.ascontiguousarray(raw).reshape(-1).view(np.uint8)
    return np.frombuffer(bytes(raw), dtype=np.uint8)


def block_size(dtype: int) -> int:
    return lib().gq_block_size(dtype)


def block_bytes(dtype: int) -> int:
    return lib().gq_block_bytes(dtype)


def row_bytes(dtype: int, k: int) -> int:
    return lib().gq_row_bytes(dtype, k)


def f16_to_f32(h: int) -> float:
    return lib().gq_f16_to_f32(h)


def f32_to_bf16(f: float) -> int:
    return lib().gq_f32_to_bf16_rne(f)


def scale_min_k4(j: int, scales12) -> tuple[int, int]:
    s = _bytes_arr(scales12)
    sc, m = C.c_uint8(), C.c_uint8()
    lib().gq_scale_min_k4(j, _u8(s), C.byref(sc), C.byref(m))
    return sc.value, m.value


def dequantize(raw, dtype: int, n_out: int | None = None) -> np.ndarray:
    """Backend::dequantize; returns float32 of ``n_out`` elements (default: all whole blocks)."""
    b = _bytes_arr(raw)
    bb, bs = block_bytes(dtype), block_size(dtype)
    if bb == 0:
        raise NotImplementedError(f"dequantize: ggml dtype {dtype}")
    if n_out is None:
        n_out = (b.size // bb) * bs
    out = np.zeros(n_out, np.float32)
    rc = lib().gq_dequantize(_u8(b), b.size, _f32(out), n_out, dtype)
    if rc != OK:
        raise NotImplementedError(f"dequantize: rc={rc}")
    return out


def ffn_swiglu(gate, up, dtype_gu: int, down, dtype_dn: int, x, m: int, hidden: int, ffn: int,
               relu_gate: bool = False, acc: int = 1, threads: int = 1) -> np.ndarray:
    """Dense feed-forward block: (silu(x gate^T) * (x up^T)) down^T; ``acc`` as in quantized_matmul."""
    g, u, d = _bytes_arr(gate), _bytes_arr(up), _bytes_arr(down)
    xx = np.ascontiguousarray(x, np.float32).reshape(m, hidden)
    out = np.zeros((m, hidden), np.float32)
    rc = lib().gq_ffn_swiglu(_u8(g), _u8(u), dtype_gu, _u8(d), dtype_dn, _f32(xx), _f32(out), m, hidden, ffn,
                             1 if relu_gate else 0, acc, threads)
    if rc == 1:
        raise NotImplementedError(f"ffn_swiglu: ggml dtype {dtype_gu}/{dtype_dn}")
    if rc != OK:
        raise ValueError(f"ffn_swiglu: rc={rc}")
    return out


def argmax_token(logits):
    """argmax_token of the reference: None for an empty or all-NaN vector."""
    a = np.ascontiguousarray(logits, np.float32).reshape(-1)
    r = lib().gq_argmax_token(_f32(a), a.size)
    return None if r < 0 else int(r)


def quant_gather(table, dtype: int, vocab: int, hidden: int, ids, scale: float | None = None) -> np.ndarray:
    """Op::QuantGather: rows ``ids`` of the quantized table, decoded, times ``scale`` if given."""
    t = _bytes_arr(table)
    idx = np.ascontiguousarray(ids, dtype=np.uint32)
    if t.size < vocab * row_bytes(dtype, hidden):
        raise ValueError("quant_gather: table shorter than vocab rows")
    out = np.zeros((idx.size, hidden), np.float32)
    rc = lib().gq_quant_gather(_u8(t), dtype, vocab, hidden, _u32(idx), idx.size,
                               1.0 if scale is None else float(scale), 0 if scale is None else 1, _f32(out))
    if rc == 1:
        raise NotImplementedError(f"quant_gather: ggml dtype {dtype}")
    if rc != OK:
        raise ValueError(f"quant_gather: rc={rc} (an id outside the table?)")
    return out


def quantized_matmul(w, x: np.ndarray, dtype: int, m: int, n: int, k: int,
                     acc: int = ACC_F64, threads: int = 1) -> np.ndarray:
    wb = _bytes_arr(w)
    if block_bytes(dtype) == 0:
        raise NotImplementedError(f"quantized_matmul: ggml dtype {dtype}")
    assert wb.size >= n * row_bytes(dtype, k), "weight buffer shorter than n rows"
    xa = np.ascontiguousarray(x, np.float32).reshape(m, k)
    y = np.zeros((m, n), np.float32)
    rc = lib().gq_quantized_matmul(_u8(wb), _f32(xa), _f32(y), dtype, m, n, k, acc, threads)
    if rc != OK:
        raise RuntimeError(f"quantized_matmul: rc={rc}")
    return y


def have_avx2() -> bool:
    return bool(lib().gq_have_avx2())


def dequant_block_avx2(block, dtype: int) -> np.ndarray:
    """One block through the vectorised decoder of the CPU baseline's AVX2 flavour."""
    b = _bytes_arr(block)
    assert b.size == block_bytes(dtype)
    out = np.zeros(block_size(dtype), np.float32)
    rc = lib().gq_dequant_block_avx2(dtype, _u8(b), _f32(out))
    if rc != OK:
        raise NotImplementedError(f"dequant_block_avx2: rc={rc}")
    return out


def quantized_matmul_avx2(w, x: np.ndarray, dtype: int, m: int, n: int, k: int,
                          threads: int = 1) -> np.ndarray:
    """The vectorised flavour of the CPU baseline (AVX2 decode, f32 dot over eight-lane sums)."""
    wb = _bytes_arr(w)
    assert wb.size >= n * row_bytes(dtype, k), "weight buffer shorter than n rows"
    xa = np.ascontiguousarray(x, np.float32).reshape(m, k)
    y = np.zeros((m, n), np.float32)
    rc = lib().gq_quantized_matmul_avx2(_u8(wb), _f32(xa), _f32(y), dtype, m, n, k, threads)
    if rc != OK:
        raise NotImplementedError(f"quantized_matmul_avx2: rc={rc}")
    return y


def have_avx512() -> bool:
    return bool(lib().gq_have_avx512())


def dequant_block_avx512(block, dtype: int) -> np.ndarray:
    """One block through the decoder of the CPU baseline's AVX-512 flavour."""
    b = _bytes_arr(block)
    assert b.size == block_bytes(dtype)
    out = np.zeros(block_size(dtype), np.float32)
    rc = lib().gq_dequant_block_avx512(dtype, _u8(b), _f32(out))
    if rc != OK:
        raise NotImplementedError(f"dequant_block_avx512: rc={rc}")
    return out


def quantized_matmul_avx512(w, x: np.ndarray, dtype: int, m: int, n: int, k: int,
                          threads: int = 1) -> np.ndarray:
    """The vectorised flavour of the CPU baseline (AVX-512 decode, f32 dot over sixteen-lane sums)."""
    wb = _bytes_arr(w)
    assert wb.size >= n * row_bytes(dtype, k), "weight buffer shorter than n rows"
    xa = np.ascontiguousarray(x, np.float32).reshape(m, k)
    y = np.zeros((m, n), np.float32)
    rc = lib().gq_quantized_matmul_avx512(_u8(wb), _f32(xa), _f32(y), dtype, m, n, k, threads)
    if rc != OK:
        raise NotImplementedError(f"quantized_matmul_avx512: rc={rc}")
    return y


def quantized_matmul_bf16(w, x: np.ndarray, dtype: int, m: int, n: int, k: int,
                          threads: int = 1) -> np.ndarray:
    wb = _bytes_arr(w)
    xa = np.ascontiguousarray(x, np.float32).reshape(m, k)
    y = np.zeros((m, n), np.float32)
    rc = lib().gq_quantized_matmul_bf16(_u8(wb), _f32(xa), _f32(y), dtype, m, n, k, threads)
    if rc != OK:
        raise RuntimeError(f"quantized_matmul_bf16: rc={rc}")
    return y


def softmax(logits) -> np.ndarray:
    z = np.ascontiguousarray(logits, np.float32)
    p = np.zeros_like(z)
    lib().gq_softmax(_f32(z), z.size, _f32(p))
    return p


def topk_with_weights(logits, k: int):
    z = np.ascontiguousarray(logits, np.float32)
    idx = np.zeros(max(k, 1), np.uint32)
    w = np.zeros(max(k, 1), np.float32)
    n = lib().gq_topk_with_weights(_f32(z), z.size, k, _u32(idx), _f32(w))
    return idx[:n].copy(), w[:n].copy()


def topk_indices(logits, k: int) -> np.ndarray:
    z = np.ascontiguousarray(logits, np.float32)
    idx = np.zeros(max(k, 1), np.uint32)
    n = lib().gq_topk_indices(_f32(z), z.size, k, _u32(idx))
    return idx[:n].copy()


def expert_capacity(capacity_factor: float, total_tokens: int, num_experts: int) -> int:
    return lib().gq_expert_capacity(capacity_factor, total_tokens, num_experts)


def route(logits, top_k: int, capacity_factor: float = 1.25):
    """ExpertRouteTable::from_gate_logits.  Returns a dict of arrays."""
    z = np.ascontiguousarray(logits, np.float32)
    tokens, experts = z.shape
    kk = max(top_k, 1)
    re = np.zeros((tokens, kk), np.uint32)
    rw = np.zeros((tokens, kk), np.float32)
    rp = np.zeros((tokens, kk), np.uint32)
    rl = np.zeros(tokens, np.uint32)
    ec = np.zeros(max(experts, 1), np.uint32)
    ov = lib().gq_route(_f32(z), tokens, experts, top_k, capacity_factor,
                        _u32(re), _f32(rw), _u32(rp), _u32(rl), _u32(ec))
    return dict(expert=re, weight=rw, pos=rp, len=rl, counts=ec[:experts], overflow=ov)


def moe_ffn(gate_up, dtype_gu: int, down, dtype_dn: int, x, hidden: int, ffn: int, experts: int,
            route_expert, route_weight, route_len, relu_gate: bool = False,
            acc: int = ACC_F64, threads: int = 1) -> np.ndarray:
    gu, dn = _bytes_arr(gate_up), _bytes_arr(down)
    xa = np.ascontiguousarray(x, np.float32).reshape(-1, hidden)
    tokens = xa.shape[0]
    re = np.ascontiguousarray(route_expert, np.uint32).reshape(tokens, -1)
    rw = np.ascontiguousarray(route_weight, np.float32).reshape(tokens, -1)
    rl = np.ascontiguousarray(route_len, np.uint32)
    top_k = re.shape[1]
    assert gu.size >= experts * 2 * ffn * row_bytes(dtype_gu, hidden)
    assert dn.size >= experts * hidden * row_bytes(dtype_dn, ffn)
    out = np.zeros((tokens, hidden), np.float32)
    rc = lib().gq_moe_ffn(_u8(gu), dtype_gu, _u8(dn), dtype_dn, _f32(xa), _f32(out), tokens, hidden,
                          ffn, experts, top_k, _u32(re), _f32(rw), _u32(rl), int(relu_gate), acc, threads)
    if rc != OK:
        raise RuntimeError(f"moe_ffn: rc={rc}")
    return out
