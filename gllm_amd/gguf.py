"""GGUF files through the library's reader (``gllmq_gguf_*``): tensor table, metadata, and
upload of a tensor's bytes into a device tensor, as the file stores them.

Mirror of the reference's ``GgufReader`` for this path (src/loader/gguf/reader.rs:38-187):
same acceptance rules, shapes handed out outermost-first (reader.rs:593-598)."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

from . import backend

ERR_NAMES = {1: "Io", 2: "InvalidMagic", 3: "UnsupportedVersion", 4: "ParseError", 5: "InvalidMetadata",
             6: "TensorOutOfBounds", 7: "UnknownDType", 8: "Utf8"}


class GgufError(Exception):
    def __init__(self, code: int, message: str):
        super().__init__(f"{ERR_NAMES.get(code, code)}: {message}")
        self.code = code
        self.kind = ERR_NAMES.get(code, str(code))


class _TensorStruct(C.Structure):
    _fields_ = [("name", C.c_char_p), ("ggml_dtype", C.c_uint32), ("n_dims", C.c_uint32),
                ("shape", C.c_uint64 * 4), ("ne", C.c_uint64 * 4), ("offset", C.c_size_t), ("nbytes", C.c_size_t)]


@dataclass(frozen=True)
class TensorInfo:
    index: int
    name: str
    ggml_dtype: int
    shape: tuple  # outermost first
    ne: tuple     # as stored, ne[0] innermost
    offset: int
    nbytes: int


def _declare(L):
    vp, sz = C.c_void_p, C.c_size_t
    L.gllmq_gguf_open.restype = C.c_int
    L.gllmq_gguf_open.argtypes = [C.c_char_p, C.POINTER(vp), C.c_char_p, sz]
    L.gllmq_gguf_parse.restype = C.c_int
    L.gllmq_gguf_parse.argtypes = [vp, sz, C.POINTER(vp), C.c_char_p, sz]
    L.gllmq_gguf_close.restype = None
    L.gllmq_gguf_close.argtypes = [vp]
    L.gllmq_gguf_version.restype = C.c_uint32
    L.gllmq_gguf_version.argtypes = [vp]
    for n in ("tensor_count", "kv_count", "alignment", "data_offset"):
        f = getattr(L, "gllmq_gguf_" + n)
        f.restype, f.argtypes = sz, [vp]
    L.gllmq_gguf_tensor_at.restype = C.c_int
    L.gllmq_gguf_tensor_at.argtypes = [vp, sz, C.POINTER(_TensorStruct)]
    L.gllmq_gguf_find_tensor.restype = C.c_long
    L.gllmq_gguf_find_tensor.argtypes = [vp, C.c_char_p]
    L.gllmq_gguf_tensor_data.restype = vp
    L.gllmq_gguf_tensor_data.argtypes = [vp, sz]
    L.gllmq_gguf_meta_type.restype = C.c_int
    L.gllmq_gguf_meta_type.argtypes = [vp, C.c_char_p]
    L.gllmq_gguf_meta_u64.restype = C.c_int
    L.gllmq_gguf_meta_u64.argtypes = [vp, C.c_char_p, C.POINTER(C.c_uint64)]
    L.gllmq_gguf_meta_i64.restype = C.c_int
    L.gllmq_gguf_meta_i64.argtypes = [vp, C.c_char_p, C.POINTER(C.c_int64)]
    L.gllmq_gguf_meta_f64.restype = C.c_int
    L.gllmq_gguf_meta_f64.argtypes = [vp, C.c_char_p, C.POINTER(C.c_double)]
    L.gllmq_gguf_meta_bool.restype = C.c_int
    L.gllmq_gguf_meta_bool.argtypes = [vp, C.c_char_p, C.POINTER(C.c_int)]
    L.gllmq_gguf_meta_str.restype = vp
    L.gllmq_gguf_meta_str.argtypes = [vp, C.c_char_p, C.POINTER(sz)]
    L.gllmq_gguf_meta_array.restype = C.c_int
    L.gllmq_gguf_meta_array.argtypes = [vp, C.c_char_p, C.POINTER(C.c_uint32), C.POINTER(C.c_uint64)]
    L.gllmq_gguf_meta_array_str.restype = vp
    L.gllmq_gguf_meta_array_str.argtypes = [vp, C.c_char_p, C.c_uint64, C.POINTER(sz)]
    L.gllmq_gguf_layer_count.restype = sz
    L.gllmq_gguf_layer_count.argtypes = [vp]
    L.gllmq_gguf_layer_tensors.restype = sz
    L.gllmq_gguf_layer_tensors.argtypes = [vp, sz, C.POINTER(sz), sz]
    L.gllmq_gguf_layer_tensor.restype = C.c_long
    L.gllmq_gguf_layer_tensor.argtypes = [vp, sz, C.c_char_p]
    L.gllmq_gguf_mixed_quant_groups.restype = sz
    L.gllmq_gguf_mixed_quant_groups.argtypes = [vp, C.POINTER(C.c_uint32), sz]
    L.gllmq_gguf_upload.restype = C.c_int
    L.gllmq_gguf_upload.argtypes = [vp, vp, sz, vp, sz, vp]
    return L


class GgufFile:
    """``GgufFile(path)`` or ``GgufFile(image=bytes)``; raises :class:`GgufError` as the reference's reader would."""

    def __init__(self, path: str | None = None, image: bytes | None = None):
        self._lib = _declare(backend.load_library())
        self._h = C.c_void_p()
        err = C.create_string_buffer(512)
        if path is not None:
            rc = self._lib.gllmq_gguf_open(str(path).encode(), C.byref(self._h), err, len(err))
        else:
            self._image = C.create_string_buffer(bytes(image), len(image))  # kept alive with the reader
            rc = self._lib.gllmq_gguf_parse(self._image, len(image), C.byref(self._h), err, len(err))
        if rc != 0:
            self._h = C.c_void_p()
            raise GgufError(rc, err.value.decode(errors="replace"))

    def close(self) -> None:
        if getattr(self, "_h", None):
            self._lib.gllmq_gguf_close(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    version = property(lambda self: self._lib.gllmq_gguf_version(self._h))
    tensor_count = property(lambda self: self._lib.gllmq_gguf_tensor_count(self._h))
    kv_count = property(lambda self: self._lib.gllmq_gguf_kv_count(self._h))
    alignment = property(lambda self: self._lib.gllmq_gguf_alignment(self._h))
    data_offset = property(lambda self: self._lib.gllmq_gguf_data_offset(self._h))

    def tensor(self, key) -> TensorInfo:
        index = key
        if isinstance(key, str):
            index = self._lib.gllmq_gguf_find_tensor(self._h, key.encode())
            if index < 0:
                raise KeyError(key)
        t = _TensorStruct()
        if self._lib.gllmq_gguf_tensor_at(self._h, index, C.byref(t)) != 0:
            raise IndexError(index)
        return TensorInfo(index, t.name.decode(), t.ggml_dtype, tuple(t.shape[:t.n_dims]), tuple(t.ne[:t.n_dims]),
                          t.offset, t.nbytes)

    def tensors(self):
        return [self.tensor(i) for i in range(self.tensor_count)]

    def tensor_bytes(self, key) -> bytes:
        t = self.tensor(key)
        p = self._lib.gllmq_gguf_tensor_data(self._h, t.index)
        return C.string_at(p, t.nbytes)

    def meta(self, key: str):
        """The value of a metadata key (None if absent); arrays of strings as lists, other arrays as (item_type, count)."""
        k = key.encode()
        ty = self._lib.gllmq_gguf_meta_type(self._h, k)
        if ty < 0:
            return None
        if ty in (0, 2, 4, 10):
            v = C.c_uint64()
            self._lib.gllmq_gguf_meta_u64(self._h, k, C.byref(v))
            return v.value
        if ty in (1, 3, 5, 11):
            v = C.c_int64()
            self._lib.gllmq_gguf_meta_i64(self._h, k, C.byref(v))
            return v.value
        if ty in (6, 12):
            v = C.c_double()
            self._lib.gllmq_gguf_meta_f64(self._h, k, C.byref(v))
            return v.value
        if ty == 7:
            v = C.c_int()
            self._lib.gllmq_gguf_meta_bool(self._h, k, C.byref(v))
            return bool(v.value)
        if ty == 8:
            n = C.c_size_t()
            p = self._lib.gllmq_gguf_meta_str(self._h, k, C.byref(n))
            return C.string_at(p, n.value).decode()
        it, cnt = C.c_uint32(), C.c_uint64()
        self._lib.gllmq_gguf_meta_array(self._h, k, C.byref(it), C.byref(cnt))
        if it.value == 8:
            out = []
            for i in range(cnt.value):
                n = C.c_size_t()
                p = self._lib.gllmq_gguf_meta_array_str(self._h, k, i, C.byref(n))
                out.append(C.string_at(p, n.value).decode())
            return out
        return (it.value, cnt.value)

    def meta_u64(self, key: str):
        """``GgufValue::as_u64`` of the reference: None for absent keys, negative or non-integer values."""
        v = C.c_uint64()
        return v.value if self._lib.gllmq_gguf_meta_u64(self._h, key.encode(), C.byref(v)) else None

    def layer_count(self) -> int:
        """Highest layer with a per-layer weight, plus one, among the layers below the model's declared
        layer count (gllmq_gguf_layer_count)."""
        return int(self._lib.gllmq_gguf_layer_count(self._h))

    def layer_table(self) -> dict:
        """``{layer: {projection: TensorInfo}}`` over the per-layer weights ``blk.{layer}.{projection}.weight``
        (attn_q, attn_k, attn_v, attn_output, ffn_gate, ffn_up, ffn_down, ...): the (layer, projection) ->
        dtype table a host walks to call the kernels with each matrix's own format, as `*_K_M` files
        mix Q4_K / Q5_K with Q6_K from layer to layer (gllmq_gguf_layer_count / gllmq_gguf_layer_tensors)."""
        table: dict = {}
        for layer in range(self._lib.gllmq_gguf_layer_count(self._h)):
            n = self._lib.gllmq_gguf_layer_tensors(self._h, layer, None, 0)
            if n == 0:
                continue
            idx = (C.c_size_t * n)()
            self._lib.gllmq_gguf_layer_tensors(self._h, layer, idx, n)
            table[layer] = {}
            for i in idx:
                t = self.tensor(int(i))
                table[layer][t.name.split(".")[2]] = t
        return table

    def layer_tensor(self, layer: int, projection: str):
        """The weight ``blk.{layer}.{projection}.weight`` or None (gllmq_gguf_layer_tensor)."""
        i = self._lib.gllmq_gguf_layer_tensor(self._h, layer, projection.encode())
        return None if i < 0 else self.tensor(int(i))

    def mixed_quant_groups(self):
        """Layers grouped by their dtype signature (sorted ``(projection, dtype)`` pairs), or None when
        every layer has the same one: what the reference's graph builder detects before it emits
        per-group matmul ops (src/arch/auto_graph_fragments/build_graph.inc.rs:388-470).  Groups come
        in a fixed order, by signature (gllmq_gguf_mixed_quant_groups)."""
        layers = self._lib.gllmq_gguf_layer_count(self._h)
        group_of = (C.c_uint32 * max(layers, 1))()
        count = self._lib.gllmq_gguf_mixed_quant_groups(self._h, group_of, layers)
        if count == 0:
            return None
        table = self.layer_table()
        groups = [[] for _ in range(count)]
        for layer in range(layers):
            if group_of[layer] != 0xFFFFFFFF:
                groups[group_of[layer]].append(layer)
        return [(tuple(sorted((proj, t.ggml_dtype) for proj, t in table[g[0]].items())), g) for g in groups]

    def upload(self, hip: "backend.HipBackend", key, dst) -> TensorInfo:
        """Copies the tensor's bytes, as stored, into the device uint8 tensor ``dst``."""
        t = self.tensor(key)
        rc = self._lib.gllmq_gguf_upload(hip._ctx, self._h, t.index, dst.data_ptr(), dst.numel() * dst.element_size(),
                                         hip._stream())
        if rc != backend.OK:
            hip._raise(rc, "gguf_upload")
        return t
