"""A minimal GGUF v3 writer for the tests, written from the format description
(docs/domain-knowledge/gguf-format-spec.md of the reference: header, key/value metadata,
tensor infos, padding to `general.alignment`, tensor data at aligned offsets).  Every knob a
test needs to produce a malformed file is a parameter."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARR, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q", F64: "<d"}


def _string(s) -> bytes:
    b = s if isinstance(s, bytes) else s.encode()
    return struct.pack("<Q", len(b)) + b


def _value(ty, v) -> bytes:
    if ty == STR:
        return _string(v)
    if ty == ARR:
        item_type, items = v
        return struct.pack("<IQ", item_type, len(items)) + b"".join(_value(item_type, x) for x in items)
    return struct.pack(_FMT.get(ty, "<I"), v)  # an id outside the table (malformed-file tests) is written as 4 bytes


def build(metadata, tensors, version=3, magic=0x46554747, alignment=None, tensor_count=None, truncate=None,
          offsets=None) -> bytes:
    """metadata: list of (key, type, value); tensors: list of (name, ne (innermost first), ggml_dtype, data bytes).
    `alignment`: what the data is laid out with (default: the metadata's general.alignment or 32);
    `offsets`: relative data offsets to write instead of the computed ones."""
    al = alignment
    if al is None:
        al = next((v for k, t, v in metadata if k == "general.alignment" and t in (U32, U64)), 32) or 32
    head = struct.pack("<IIQQ", magic, version, len(tensors) if tensor_count is None else tensor_count, len(metadata))
    for k, t, v in metadata:
        head += _string(k) + struct.pack("<I", t) + _value(t, v)
    rel, pos = [], 0
    for name, ne, dt, data in tensors:
        rel.append(pos)
        pos += len(data)
        pos += (-pos) % al
    placed = list(rel)  # where the data really goes; `offsets` only changes what the infos claim
    if offsets is not None:
        rel = list(offsets)
    for (name, ne, dt, data), off in zip(tensors, rel):
        head += _string(name) + struct.pack("<I", len(ne)) + b"".join(struct.pack("<Q", d) for d in ne)
        head += struct.pack("<IQ", dt, off)
    head += b"\0" * ((-len(head)) % al)
    body = bytearray(max([0] + [off + len(t[3]) for t, off in zip(tensors, placed)]))
    for (name, ne, dt, data), off in zip(tensors, placed):
        body[off:off + len(data)] = bytes(data)
    out = head + bytes(body)
    return out if truncate is None else out[:truncate]


def f32_tensor(name, array):
    a = np.ascontiguousarray(array, np.float32)
    return (name, list(reversed(a.shape)), 0, a.tobytes())
