"""Host-side mirror of the reference's backend interface for the quantized matmul path.

``HipBackend.quantized_matmul`` / ``HipBackend.dequantize`` keep the names, argument
order and error behaviour of ``Backend::quantized_matmul`` / ``Backend::dequantize``
(reference: src/compat/mod.rs:233-256; CPU implementation src/compat/cpu_backend.rs:991-1159;
error enum src/engine/executor_types.rs:322-329).  All arithmetic happens in
``libgllm_hip_quant.so`` (hand-written gfx950 kernels behind a C ABI, see
``include/gllm_hip_quant.h``); this module only moves pointers.  There is no CPU fallback:
without the library or without a GPU every call raises.

Buffers may be host slices (``bytes`` / numpy arrays, as in the reference's signature) or
torch tensors that already live on the GPU.  torch is used for device memory and streams only.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from .ggml import GgmlDType, QuantType, block_bytes, block_size, row_bytes, supported

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgllm_hip_quant.so")

OK, ERR_UNIMPLEMENTED, ERR_BAD_SHAPE, ERR_BAD_ALIGNMENT, ERR_HIP, ERR_INVALID = range(6)
ACT_F32_SPLIT, ACT_BF16 = 0, 1
DESC_AFTER_PREVIOUS = 1  # gllmq_matmul_desc.flags: the entry depends on the entries before it
DESC_ELEM_F16, DESC_ELEM_BF16 = 0x100, 0x200  # gllmq_matmul_desc.flags: element type of the entry's x and y


ELEM_F32, ELEM_F16, ELEM_BF16 = 0, 1, 2  # gllmq_quantized_matmul_elem: element type of activations and outputs
OUT_ACCUMULATE = 1  # flags of gllmq_ffn_swiglu_elem / gllmq_moe_matvec_elem: add to the output instead of replacing it
ARGMAX_NONE = 0xFFFFFFFF  # gllmq_argmax: the row has no entry that is not NaN


class BackendError(Exception):
    """``BackendError`` of the reference; subclasses are its variants."""


class Unimplemented(BackendError):
    pass


class HipError(BackendError):
    pass


class OtherError(BackendError):
    pass


class MatmulDesc(C.Structure):
    _fields_ = [("w_dev", C.c_void_p), ("w_bytes", C.c_size_t), ("x_dev", C.c_void_p),
                ("y_dev", C.c_void_p), ("ggml_dtype", C.c_uint32), ("flags", C.c_uint32),
                ("m", C.c_size_t), ("n", C.c_size_t), ("k", C.c_size_t)]


_lib = None


def load_library() -> C.CDLL:
    """dlopen the in-tree library and declare every prototype of the public header."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HipError(f"{LIB_PATH} is missing: build it with `python -m gllm_amd.build`")
    try:  # when torch is in the process, its HIP runtime must be the one the library binds to
        import torch  # noqa: F401
    except ImportError:  # the library runs without torch (host-pointer entry points)
        pass
    L = C.CDLL(LIB_PATH)
    vp, sz, u32 = C.c_void_p, C.c_size_t, C.c_uint32
    L.gllmq_init.restype = C.c_int
    L.gllmq_init.argtypes = [C.POINTER(vp), C.c_int]
    L.gllmq_destroy.restype = None
    L.gllmq_destroy.argtypes = [vp]
    L.gllmq_last_error.restype = C.c_char_p
    L.gllmq_last_error.argtypes = [vp]
    L.gllmq_status_string.restype = C.c_char_p
    L.gllmq_status_string.argtypes = [C.c_int]
    L.gllmq_version.restype = C.c_char_p
    L.gllmq_version.argtypes = []
    for name in ("gllmq_block_size", "gllmq_block_bytes"):
        getattr(L, name).restype = sz
        getattr(L, name).argtypes = [u32]
    L.gllmq_row_bytes.restype = sz
    L.gllmq_row_bytes.argtypes = [u32, sz]
    L.gllmq_dequantize.restype = C.c_int
    L.gllmq_dequantize.argtypes = [vp, vp, sz, vp, sz, u32, vp]
    L.gllmq_quantized_matmul.restype = C.c_int
    L.gllmq_quantized_matmul.argtypes = [vp, vp, sz, vp, vp, u32, sz, sz, sz, vp]
    L.gllmq_quantized_matmul_ex.restype = C.c_int
    L.gllmq_quantized_matmul_ex.argtypes = [vp, vp, sz, vp, vp, u32, sz, sz, sz, C.c_int, vp]
    L.gllmq_quantized_matmul_noalloc.restype = C.c_int
    L.gllmq_quantized_matmul_noalloc.argtypes = [vp, vp, sz, vp, vp, u32, sz, sz, sz, vp]
    L.gllmq_quantized_matmul_batch.restype = C.c_int
    L.gllmq_quantized_matmul_batch.argtypes = [vp, C.POINTER(MatmulDesc), sz, vp]
    L.gllmq_moe_matvec.restype = C.c_int
    L.gllmq_moe_matvec.argtypes = [vp, vp, sz, sz, vp, sz, sz, u32, vp, sz, sz, u32, vp, vp, sz, sz, sz, sz, sz, vp, vp, vp,
                                   C.c_int, vp]
    L.gllmq_moe_route.restype = C.c_int
    L.gllmq_moe_route.argtypes = [vp, vp, sz, sz, sz, C.c_float, vp, vp, vp, vp, vp, vp, vp]
    L.gllmq_set_option.restype = C.c_int
    L.gllmq_set_option.argtypes = [vp, C.c_char_p, C.c_long]
    L.gllmq_last_kernel_name.restype = C.c_char_p
    L.gllmq_last_kernel_name.argtypes = [vp]
    L.gllmq_reserve_matmul.restype = C.c_int
    L.gllmq_reserve_matmul.argtypes = [vp, u32, sz, sz, sz, vp]
    L.gllmq_reserve_ffn.restype = C.c_int
    L.gllmq_reserve_ffn.argtypes = [vp, u32, u32, sz, sz, sz, vp]
    L.gllmq_reserve_moe.restype = C.c_int
    L.gllmq_reserve_moe.argtypes = [vp, sz, sz, sz, sz, vp]
    L.gllmq_weights_forget.restype = None
    L.gllmq_weights_forget.argtypes = [vp, vp]
    L.gllmq_chain_status.restype = C.c_int
    L.gllmq_chain_status.argtypes = [vp]
    L.gllmq_weight_uploads.restype = C.c_uint64
    L.gllmq_weight_uploads.argtypes = [vp]
    L.gllmq_quant_gather.restype = C.c_int
    L.gllmq_quant_gather.argtypes = [vp, vp, sz, u32, sz, sz, vp, sz, C.c_float, vp, vp]
    L.gllmq_ffn_swiglu.restype = C.c_int
    L.gllmq_ffn_swiglu.argtypes = [vp, vp, vp, sz, u32, vp, sz, u32, vp, vp, sz, sz, sz, C.c_int, vp]
    L.gllmq_ffn_swiglu_elem.restype = C.c_int
    L.gllmq_ffn_swiglu_elem.argtypes = [vp, vp, vp, sz, u32, vp, sz, u32, vp, vp, sz, sz, sz, C.c_int, C.c_int, C.c_int, vp]
    L.gllmq_moe_matvec_elem.restype = C.c_int
    L.gllmq_moe_matvec_elem.argtypes = [vp, vp, sz, sz, vp, sz, sz, u32, vp, sz, sz, u32, vp, vp, sz, sz, sz, sz, sz, vp, vp, vp,
                                        C.c_int, C.c_int, C.c_int, vp]
    L.gllmq_quant_gather_elem.restype = C.c_int
    L.gllmq_quant_gather_elem.argtypes = [vp, vp, sz, u32, sz, sz, vp, sz, C.c_float, vp, C.c_int, vp]
    L.gllmq_argmax.restype = C.c_int
    L.gllmq_argmax.argtypes = [vp, vp, sz, sz, sz, vp, vp, vp]
    L.gllmq_quantized_matmul_elem.restype = C.c_int
    L.gllmq_quantized_matmul_elem.argtypes = [vp, vp, sz, vp, vp, C.c_uint32, sz, sz, sz, C.c_int, vp]
    L.gllmq_reserve_matmul_elem.restype = C.c_int
    L.gllmq_reserve_matmul_elem.argtypes = [vp, C.c_uint32, sz, sz, sz, C.c_int, vp]
    L.gllmq_lm_head_argmax.restype = C.c_int
    L.gllmq_lm_head_argmax.argtypes = [vp, vp, sz, vp, C.c_uint32, sz, sz, vp, vp, vp, vp]
    L.gllmq_dequantize_host.restype = C.c_int
    L.gllmq_dequantize_host.argtypes = [vp, vp, sz, vp, sz, u32]
    L.gllmq_quant_gather_host.restype = C.c_int
    L.gllmq_quant_gather_host.argtypes = [vp, vp, sz, u32, sz, sz, vp, sz, C.c_float, vp]
    L.gllmq_quantized_matmul_host.restype = C.c_int
    L.gllmq_quantized_matmul_host.argtypes = [vp, vp, sz, vp, vp, u32, sz, sz, sz]
    _lib = L
    return L


EXPORTED_SYMBOLS = [
    "gllmq_init", "gllmq_destroy", "gllmq_last_error", "gllmq_status_string", "gllmq_version",
    "gllmq_block_size", "gllmq_block_bytes", "gllmq_row_bytes", "gllmq_dequantize",
    "gllmq_quantized_matmul", "gllmq_quantized_matmul_ex", "gllmq_quantized_matmul_batch",
    "gllmq_quantized_matmul_noalloc", "gllmq_chain_status", "gllmq_ffn_swiglu_elem", "gllmq_moe_matvec_elem", "gllmq_quant_gather_elem",
    "gllmq_moe_matvec", "gllmq_ffn_swiglu", "gllmq_argmax", "gllmq_lm_head_argmax", "gllmq_quantized_matmul_elem", "gllmq_reserve_matmul_elem", "gllmq_quant_gather", "gllmq_moe_route", "gllmq_set_option", "gllmq_last_kernel_name",
    "gllmq_reserve_matmul", "gllmq_reserve_ffn", "gllmq_reserve_moe", "gllmq_weights_forget", "gllmq_weight_uploads",
    "gllmq_dequantize_host", "gllmq_quant_gather_host", "gllmq_quantized_matmul_host",
    "gllmq_gguf_open", "gllmq_gguf_parse", "gllmq_gguf_close", "gllmq_gguf_version", "gllmq_gguf_tensor_count",
    "gllmq_gguf_kv_count", "gllmq_gguf_alignment", "gllmq_gguf_data_offset", "gllmq_gguf_tensor_at",
    "gllmq_gguf_find_tensor", "gllmq_gguf_tensor_data", "gllmq_gguf_meta_type", "gllmq_gguf_meta_u64",
    "gllmq_gguf_meta_i64", "gllmq_gguf_meta_f64", "gllmq_gguf_meta_bool", "gllmq_gguf_meta_str", "gllmq_gguf_meta_array",
    "gllmq_gguf_meta_array_str", "gllmq_gguf_upload",
    "gllmq_gguf_layer_count", "gllmq_gguf_layer_tensors", "gllmq_gguf_layer_tensor", "gllmq_gguf_mixed_quant_groups",
]


def _dtype_id(quant_type) -> int:
    if isinstance(quant_type, QuantType):
        return quant_type.ggml_dtype
    return int(quant_type)


def _is_torch(t) -> bool:
    return type(t).__module__.startswith("torch")


def _host_bytes(buf) -> np.ndarray:
    if isinstance(buf, np.ndarray):
        return np.ascontiguousarray(buf).reshape(-1).view(np.uint8)
    return np.frombuffer(buf, dtype=np.uint8)


class HipBackend:
    """The MI355X backend for ``Op::QuantGemm``: quantized weights x f32 activations."""

    def __init__(self, device: int = 0, options: dict | None = None):
        """``options``: kernel-family choices by name (``gllmq_set_option``), used by the tests to
        reach the kernels the default dispatch does not pick."""
        self._lib = load_library()
        import torch
        if not torch.cuda.is_available():
            raise HipError("no HIP device is visible; this backend has no CPU path")
        self._torch = torch
        self.device = device
        ctx = C.c_void_p()
        rc = self._lib.gllmq_init(C.byref(ctx), device)
        if rc != OK:
            raise HipError(f"gllmq_init(device={device}): {self._lib.gllmq_status_string(rc).decode()}")
        self._ctx = ctx
        for name, value in (options or {}).items():
            self.set_option(name, value)

    def set_option(self, name: str, value: int) -> None:
        rc = self._lib.gllmq_set_option(self._ctx, name.encode(), int(value))
        if rc != OK:
            self._raise(rc, "set_option")

    def last_kernel_name(self) -> str:
        """Name of the kernel this context launched last."""
        return self._lib.gllmq_last_kernel_name(self._ctx).decode()

    def weight_uploads(self) -> int:
        """Host-to-device weight copies the host-slice calls of this context have made."""
        return int(self._lib.gllmq_weight_uploads(self._ctx))

    def weights_forget(self, host_array=None) -> None:
        ptr = None if host_array is None else _host_bytes(host_array).ctypes.data
        self._lib.gllmq_weights_forget(self._ctx, ptr)

    def reserve_matmul(self, quant_type, m: int, n: int, k: int, elem: int = ELEM_F32) -> None:
        rc = self._lib.gllmq_reserve_matmul_elem(self._ctx, _dtype_id(quant_type), m, n, k, elem, self._stream())
        if rc != OK:
            self._raise(rc, "reserve_matmul")

    def reserve_ffn(self, dtype_gate_up, dtype_down, m: int, hidden: int, ffn: int) -> None:
        rc = self._lib.gllmq_reserve_ffn(self._ctx, _dtype_id(dtype_gate_up), _dtype_id(dtype_down), m, hidden, ffn,
                                         self._stream())
        if rc != OK:
            self._raise(rc, "reserve_ffn")

    def reserve_moe(self, tokens: int, top_k: int, hidden: int, ffn: int) -> None:
        rc = self._lib.gllmq_reserve_moe(self._ctx, tokens, top_k, hidden, ffn, self._stream())
        if rc != OK:
            self._raise(rc, "reserve_moe")

    def close(self) -> None:
        if getattr(self, "_ctx", None):
            self._lib.gllmq_destroy(self._ctx)
            self._ctx = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ------------------------------------------------------------------ helpers
    def _raise(self, rc: int, what: str):
        msg = self._lib.gllmq_last_error(self._ctx).decode(errors="replace") or what
        if rc == ERR_UNIMPLEMENTED:
            raise Unimplemented(msg)
        if rc == ERR_HIP:
            raise HipError(msg)
        raise OtherError(f"{self._lib.gllmq_status_string(rc).decode()}: {msg}")

    def _stream(self):
        return C.c_void_p(self._torch.cuda.current_stream(self.device).cuda_stream)

    def upload_weights(self, weight_blocks):
        """Raw GGUF block bytes -> device buffer, untouched (the reference passes quantized
        tensors through verbatim, src/engine/executor_compile.rs:207-211)."""
        host = _host_bytes(weight_blocks)
        return self._torch.from_numpy(host.copy()).to(f"cuda:{self.device}")

    # ------------------------------------------------------------ trait methods
    def quantized_matmul(self, weight_blocks, input, output, quant_type, m: int, n: int, k: int,
                         act_mode: int = ACT_F32_SPLIT) -> None:
        """output[m x n] = input[m x k] . W[n x k]^T, W given as raw GGUF blocks."""
        dt = _dtype_id(quant_type)
        if _is_torch(weight_blocks):
            w, x, y = weight_blocks, input, output
            if not (w.is_cuda and x.is_cuda and y.is_cuda):
                raise OtherError("quantized_matmul: tensors must live on the GPU")
            elem = self._elem_of(x.dtype)
            if elem is None or y.dtype != x.dtype:
                raise Unimplemented("quantized_matmul: activations and outputs are f32, f16 or bf16, both of one type")
            if not (w.is_contiguous() and x.is_contiguous() and y.is_contiguous()):
                raise OtherError("quantized_matmul: tensors must be contiguous")
            if x.numel() < m * k or y.numel() < m * n:
                raise OtherError("quantized_matmul: input/output shorter than m*k / m*n")
            if elem != ELEM_F32:
                if act_mode != ACT_F32_SPLIT:
                    raise Unimplemented("quantized_matmul: the bf16 activation mode is for f32 tensors")
                rc = self._lib.gllmq_quantized_matmul_elem(
                    self._ctx, w.data_ptr(), w.numel() * w.element_size(), x.data_ptr(), y.data_ptr(),
                    dt, m, n, k, elem, self._stream())
            else:
                rc = self._lib.gllmq_quantized_matmul_ex(
                    self._ctx, w.data_ptr(), w.numel() * w.element_size(), x.data_ptr(), y.data_ptr(),
                    dt, m, n, k, act_mode, self._stream())
        else:
            w = _host_bytes(weight_blocks)
            x = np.ascontiguousarray(input, np.float32).reshape(-1)
            if not (isinstance(output, np.ndarray) and output.dtype == np.float32 and output.flags.c_contiguous):
                raise OtherError("quantized_matmul: output must be a contiguous float32 numpy array")
            if x.size < m * k or output.size < m * n:
                raise OtherError("quantized_matmul: input/output shorter than m*k / m*n")
            rc = self._lib.gllmq_quantized_matmul_host(
                self._ctx, w.ctypes.data, w.size, x.ctypes.data, output.ctypes.data, dt, m, n, k)
        if rc != OK:
            self._raise(rc, "quantized_matmul")

    def _elem_of(self, torch_dtype):
        """Backend<E>: the element types the reference instantiates (src/compat/mod.rs:376-378)."""
        t = self._torch
        return {t.float32: ELEM_F32, t.float16: ELEM_F16, t.bfloat16: ELEM_BF16}.get(torch_dtype)

    def quantized_matmul_noalloc(self, weight_blocks, input, output, quant_type, m: int, n: int, k: int) -> None:
        """``quantized_matmul`` on device tensors through the entry point that allocates nothing
        (its scratch is a fixed array in device memory)."""
        w, x, y = weight_blocks, input, output
        if not (_is_torch(w) and w.is_cuda and x.is_cuda and y.is_cuda):
            raise OtherError("quantized_matmul_noalloc: tensors must live on the GPU")
        if x.dtype != self._torch.float32 or y.dtype != self._torch.float32:
            raise Unimplemented("quantized_matmul_noalloc: activations and outputs are f32 on this backend")
        if x.numel() < m * k or y.numel() < m * n:
            raise OtherError("quantized_matmul_noalloc: input/output shorter than m*k / m*n")
        rc = self._lib.gllmq_quantized_matmul_noalloc(self._ctx, w.data_ptr(), w.numel() * w.element_size(), x.data_ptr(),
                                                      y.data_ptr(), _dtype_id(quant_type), m, n, k, self._stream())
        if rc != OK:
            self._raise(rc, "quantized_matmul_noalloc")

    def dequantize(self, block_data, output, quant_type) -> None:
        """Whole blocks of ``block_data`` -> f32 into ``output`` (chunks_exact on both sides)."""
        dt = _dtype_id(quant_type)
        if _is_torch(block_data):
            b, o = block_data, output
            if not (b.is_cuda and o.is_cuda and o.dtype == self._torch.float32):
                raise OtherError("dequantize: tensors must live on the GPU, output f32")
            rc = self._lib.gllmq_dequantize(self._ctx, b.data_ptr(), b.numel() * b.element_size(),
                                            o.data_ptr(), o.numel(), dt, self._stream())
        else:
            b = _host_bytes(block_data)
            if not (isinstance(output, np.ndarray) and output.dtype == np.float32 and output.flags.c_contiguous):
                raise OtherError("dequantize: output must be a contiguous float32 numpy array")
            rc = self._lib.gllmq_dequantize_host(self._ctx, b.ctypes.data, b.size, output.ctypes.data,
                                                 output.size, dt)
        if rc != OK:
            self._raise(rc, "dequantize")

    # --------------------------------------------------------------- extensions
    def make_batch(self, descs, after_previous=None):
        """A descriptor array for ``run_batch``; descs: iterable of (w, x, y, quant_type, m, n, k)
        device tensors, which must stay alive while the array is used.  ``after_previous``: a
        function of the entry's index that says whether the entry depends on the ones before it
        (``GLLMQ_DESC_AFTER_PREVIOUS``); by default the entries are independent."""
        items = list(descs)
        arr = (MatmulDesc * len(items))()
        for i, (w, x, y, qt, m, n, k) in enumerate(items):
            flags = DESC_AFTER_PREVIOUS if after_previous is not None and after_previous(i) else 0
            elem = self._elem_of(x.dtype)
            if elem is None or y.dtype != x.dtype:
                raise Unimplemented("make_batch: activations and outputs are f32, f16 or bf16, both of one type")
            flags |= {ELEM_F32: 0, ELEM_F16: DESC_ELEM_F16, ELEM_BF16: DESC_ELEM_BF16}[elem]
            arr[i] = MatmulDesc(w.data_ptr(), w.numel() * w.element_size(), x.data_ptr(), y.data_ptr(),
                                _dtype_id(qt), flags, m, n, k)
        return arr

    def run_batch(self, arr, start: int = 0, count: int | None = None) -> None:
        """One C call over ``count`` descriptors of ``arr`` from ``start``."""
        count = len(arr) - start if count is None else count
        if start < 0 or count < 0 or start + count > len(arr):
            raise OtherError("run_batch: range outside the descriptor array")
        first = C.cast(C.byref(arr, start * C.sizeof(MatmulDesc)), C.POINTER(MatmulDesc))
        rc = self._lib.gllmq_quantized_matmul_batch(self._ctx, first, count, self._stream())
        if rc != OK:
            self._raise(rc, "quantized_matmul_batch")

    def chain_status(self) -> bool:
        """After a synchronisation: whether a chained launch of a batch since the last look gave up
        waiting for the entry before it (``gllmq_chain_status``; the look sets the flag back)."""
        return bool(self._lib.gllmq_chain_status(self._ctx))

    def quantized_matmul_batch(self, descs) -> None:
        """descs: iterable of (w, x, y, quant_type, m, n, k) device tensors; one C call."""
        self.run_batch(self.make_batch(descs))

    def quant_gather(self, table, quant_type, vocab_size: int, hidden_dim: int, token_ids, output,
                     scale: float | None = None) -> None:
        """Op::QuantGather: ``output[i] = scale * dequantize(table row token_ids[i])``.

        ``table``: device bytes of ``vocab_size`` rows of ``hidden_dim`` quantized elements;
        ``token_ids``: device int32/uint32 tensor; ``output``: device f32 ``[len(ids), hidden_dim]``;
        ``scale``: the embedding scale, None for none (the reference's ``Option<f32>``)."""
        dt = _dtype_id(quant_type)
        if not (_is_torch(table) and table.is_cuda and token_ids.is_cuda and output.is_cuda):
            raise OtherError("quant_gather: tensors must live on the GPU")
        elem = self._elem_of(output.dtype)
        if token_ids.element_size() != 4 or token_ids.is_floating_point() or elem is None:
            raise OtherError("quant_gather: token ids must be 32-bit integers, output f32, f16 or bf16")
        count = token_ids.numel()
        if output.numel() < count * hidden_dim:
            raise OtherError("quant_gather: output shorter than len(ids) * hidden_dim")
        if elem == ELEM_F32:
            rc = self._lib.gllmq_quant_gather(self._ctx, table.data_ptr(), table.numel() * table.element_size(), dt,
                                              vocab_size, hidden_dim, token_ids.data_ptr(), count,
                                              1.0 if scale is None else float(scale), output.data_ptr(), self._stream())
        else:
            rc = self._lib.gllmq_quant_gather_elem(self._ctx, table.data_ptr(), table.numel() * table.element_size(), dt,
                                                   vocab_size, hidden_dim, token_ids.data_ptr(), count,
                                                   1.0 if scale is None else float(scale), output.data_ptr(), elem, self._stream())
        if rc != OK:
            self._raise(rc, "quant_gather")

    def ffn_swiglu(self, gate, up, dtype_gate_up, down, dtype_down, x, out, m: int, hidden: int, ffn: int,
                   relu_gate: bool = False, accumulate: bool = False) -> None:
        """Dense feed-forward block on device tensors: ``out = (silu(x gate^T) * (x up^T)) down^T``;
        ``gate`` and ``up`` are ``[ffn x hidden]`` blocks of ``dtype_gate_up`` (``up`` may be the second
        half of one stacked tensor), ``down`` is ``[hidden x ffn]`` of ``dtype_down``; ``x`` and ``out``
        f32, f16 or bf16 (both of one type); ``accumulate``: ``out += ...`` (the shared-expert and
        residual adds behind the block)."""
        for t in (gate, up, down, x, out):
            if not (_is_torch(t) and t.is_cuda):
                raise OtherError("ffn_swiglu: tensors must live on the GPU")
        elem = self._elem_of(x.dtype)
        if elem is None or out.dtype != x.dtype:
            raise OtherError("ffn_swiglu: x and out must be f32, f16 or bf16, both of one type")
        if x.numel() < m * hidden or out.numel() < m * hidden:
            raise OtherError("ffn_swiglu: x/out shorter than m * hidden")
        gb, ub = gate.numel() * gate.element_size(), up.numel() * up.element_size()
        if elem == ELEM_F32 and not accumulate:
            rc = self._lib.gllmq_ffn_swiglu(self._ctx, gate.data_ptr(), up.data_ptr(), min(gb, ub), _dtype_id(dtype_gate_up),
                                            down.data_ptr(), down.numel() * down.element_size(), _dtype_id(dtype_down),
                                            x.data_ptr(), out.data_ptr(), m, hidden, ffn, 1 if relu_gate else 0,
                                            self._stream())
        else:
            rc = self._lib.gllmq_ffn_swiglu_elem(self._ctx, gate.data_ptr(), up.data_ptr(), min(gb, ub), _dtype_id(dtype_gate_up),
                                                 down.data_ptr(), down.numel() * down.element_size(), _dtype_id(dtype_down),
                                                 x.data_ptr(), out.data_ptr(), m, hidden, ffn, 1 if relu_gate else 0,
                                                 elem, OUT_ACCUMULATE if accumulate else 0, self._stream())
        if rc != OK:
            self._raise(rc, "ffn_swiglu")

    def argmax(self, logits, token, value=None) -> None:
        """Op::Argmax with the semantics of the reference's ``argmax_token``: ``token[r]`` = index of
        the largest non-NaN entry of row ``r`` of the device f32 matrix ``logits`` (a view with a row
        stride is fine), the last of equal maxima, ``ARGMAX_NONE`` when there is none."""
        if not (logits.is_cuda and token.is_cuda and logits.dtype == self._torch.float32 and token.element_size() == 4):
            raise OtherError("argmax: logits must be device f32, token a device 32-bit integer tensor")
        lg = logits if logits.dim() == 2 else logits.reshape(1, -1)
        if lg.stride(1) != 1 and lg.shape[1] > 1:
            raise OtherError("argmax: rows must be contiguous")
        rows, n = lg.shape
        ld = lg.stride(0) if rows > 1 else max(n, 1)
        if token.numel() < rows or (value is not None and value.numel() < rows):
            raise OtherError("argmax: token/value shorter than the number of rows")
        rc = self._lib.gllmq_argmax(self._ctx, lg.data_ptr(), rows, n, ld, token.data_ptr(),
                                    value.data_ptr() if value is not None else None, self._stream())
        if rc != OK:
            self._raise(rc, "argmax")

    def lm_head_argmax(self, weight_blocks, input, quant_type, n: int, k: int, token, logits=None, value=None) -> None:
        """The lm_head matvec of one activation row and the greedy token choice behind it as one
        call: ``token[0]`` as ``argmax`` gives it on ``quantized_matmul``'s logits.  ``logits`` (device
        f32, ``n`` entries) receives them; without it Q6_K / Q8_0 matrices never write them."""
        w, x = weight_blocks, input
        if not (_is_torch(w) and w.is_cuda and x.is_cuda and token.is_cuda and x.dtype == self._torch.float32
                and token.element_size() == 4):
            raise OtherError("lm_head_argmax: device tensors, f32 activations and a 32-bit integer token")
        if not (w.is_contiguous() and x.is_contiguous()) or x.numel() < k or token.numel() < 1:
            raise OtherError("lm_head_argmax: contiguous tensors of at least k activations and one token")
        if logits is not None and not (logits.is_cuda and logits.dtype == self._torch.float32 and logits.is_contiguous()
                                       and logits.numel() >= n):
            raise OtherError("lm_head_argmax: logits must be a contiguous device f32 tensor of n entries")
        if value is not None and not (value.is_cuda and value.dtype == self._torch.float32 and value.numel() >= 1):
            raise OtherError("lm_head_argmax: value must be a device f32 tensor")
        rc = self._lib.gllmq_lm_head_argmax(self._ctx, w.data_ptr(), w.numel() * w.element_size(), x.data_ptr(),
                                            _dtype_id(quant_type), n, k, logits.data_ptr() if logits is not None else None,
                                            token.data_ptr(), value.data_ptr() if value is not None else None,
                                            self._stream())
        if rc != OK:
            self._raise(rc, "lm_head_argmax")

    def moe_route(self, logits, top_k: int, route_expert, route_weight, route_len, capacity_factor: float = 1.25,
                  route_pos=None, expert_counts=None, overflow=None) -> None:
        """ExpertRouteTable::from_gate_logits on device tensors: ``logits`` f32 ``[tokens, experts]``;
        outputs ``route_expert`` (32-bit int) and ``route_weight`` (f32) ``[tokens, top_k]``,
        ``route_len`` ``[tokens]``; optional ``route_pos`` ``[tokens, top_k]``, ``expert_counts``
        ``[experts]``, ``overflow`` ``[1]``.  The reference's default capacity factor is 1.25."""
        tokens, experts = logits.shape
        if logits.dtype != self._torch.float32 or not logits.is_cuda or not logits.is_contiguous():
            raise OtherError("moe_route: logits must be a contiguous device f32 tensor")
        if route_expert.numel() < tokens * top_k or route_weight.numel() < tokens * top_k or route_len.numel() < tokens:
            raise OtherError("moe_route: outputs shorter than tokens * top_k / tokens")
        opt = [t.data_ptr() if t is not None else None for t in (route_pos, expert_counts, overflow)]
        rc = self._lib.gllmq_moe_route(self._ctx, logits.data_ptr(), tokens, experts, top_k, float(capacity_factor),
                                       route_expert.data_ptr(), route_weight.data_ptr(), route_len.data_ptr(),
                                       opt[0], opt[1], opt[2], self._stream())
        if rc != OK:
            self._raise(rc, "moe_route")

    def moe_matvec(self, gate_up, dtype_gate_up, down, dtype_down, x, out, hidden: int, ffn: int,
                   experts: int, route_expert, route_weight, route_len, relu_gate: bool = False,
                   up=None, accumulate: bool = False) -> None:
        """Expert matvec over a route table.  ``gate_up``: per expert ``ffn`` gate rows followed by
        ``ffn`` up rows (one stacked tensor), or, with ``up`` given, the gate rows of all experts
        (``[experts, ffn, hidden]``) with ``up`` holding the up rows the same way (GGUF's layout);
        ``down``: ``[experts, hidden, ffn]``; ``x`` and ``out`` f32, f16 or bf16 (both of one type);
        ``accumulate``: ``out += ...``."""
        tokens, top_k = route_expert.shape
        elem = self._elem_of(x.dtype)
        if elem is None or out.dtype != x.dtype:
            raise OtherError("moe_matvec: x and out must be f32, f16 or bf16, both of one type")
        dgu, ddn = _dtype_id(dtype_gate_up), _dtype_id(dtype_down)
        each = ffn * self._lib.gllmq_row_bytes(dgu, hidden)  # 0 for a dtype the library does not cover
        gbytes = gate_up.numel() * gate_up.element_size()
        if up is None:
            gate_ptr, gate_b, gate_st = gate_up.data_ptr(), max(gbytes - each, 0), 2 * each
            up_ptr, up_b, up_st = gate_up.data_ptr() + each, max(gbytes - each, 0), 2 * each
        else:
            gate_ptr, gate_b, gate_st = gate_up.data_ptr(), gbytes, each
            up_ptr, up_b, up_st = up.data_ptr(), up.numel() * up.element_size(), each
        args = (self._ctx, gate_ptr, gate_b, gate_st, up_ptr, up_b, up_st, dgu,
                down.data_ptr(), down.numel() * down.element_size(), hidden * self._lib.gllmq_row_bytes(ddn, ffn), ddn,
                x.data_ptr(), out.data_ptr(), tokens, hidden, ffn, experts, top_k, route_expert.data_ptr(),
                route_weight.data_ptr(), route_len.data_ptr(), int(relu_gate))
        if elem == ELEM_F32 and not accumulate:
            rc = self._lib.gllmq_moe_matvec(*args, self._stream())
        else:
            rc = self._lib.gllmq_moe_matvec_elem(*args, elem, OUT_ACCUMULATE if accumulate else 0, self._stream())
        if rc != OK:
            self._raise(rc, "moe_matvec")


__all__ = ["HipBackend", "BackendError", "Unimplemented", "HipError", "OtherError", "QuantType",
           "GgmlDType", "block_size", "block_bytes", "row_bytes", "supported", "load_library",
           "EXPORTED_SYMBOLS", "ACT_F32_SPLIT", "ACT_BF16", "LIB_PATH"]
