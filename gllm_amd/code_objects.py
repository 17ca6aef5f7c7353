"""Reads the metadata that the compiler leaves in the library's gfx950 code objects
(``csrc/build/kernels_*.hsaco``): per kernel its registers, LDS, and the bytes of scratch (spilled
registers) per lane.  The AMDGPU metadata is a msgpack map in an ELF note (owner "AMDGPU", type 32);
nothing is executed or disassembled.

    python -m gllm_amd.code_objects            # a table of all kernels
"""
from __future__ import annotations

import glob
import os
import struct

HERE = os.path.dirname(os.path.abspath(__file__))
BUILD = os.path.join(HERE, "csrc", "build")
NT_AMDGPU_METADATA = 32


def _device_image(blob: bytes) -> bytes:
    """The gfx950 ELF image inside a clang offload bundle (what `hipcc --genco` writes), or the
    blob itself when it already is an ELF image."""
    magic = b"__CLANG_OFFLOAD_BUNDLE__"
    if not blob.startswith(magic):
        return blob
    count, = struct.unpack_from("<Q", blob, len(magic))
    at = len(magic) + 8
    for _ in range(count):
        offset, size, idlen = struct.unpack_from("<QQQ", blob, at)
        at += 24
        ident = blob[at:at + idlen].decode()
        at += idlen
        if "amdgcn" in ident and size:
            return blob[offset:offset + size]
    raise ValueError("no device image in the offload bundle")


def _notes(blob: bytes):
    """(owner, type, descriptor) of every note of a little-endian ELF64 image."""
    if blob[:4] != b"\x7fELF" or blob[4] != 2 or blob[5] != 1:
        raise ValueError("not a little-endian ELF64 image")
    shoff, = struct.unpack_from("<Q", blob, 0x28)
    shentsize, shnum = struct.unpack_from("<HH", blob, 0x3A)
    for i in range(shnum):
        base = shoff + i * shentsize
        sh_type, = struct.unpack_from("<I", blob, base + 4)
        if sh_type != 7:  # SHT_NOTE
            continue
        offset, size = struct.unpack_from("<QQ", blob, base + 0x18)
        at, end = offset, offset + size
        while at + 12 <= end:
            namesz, descsz, ntype = struct.unpack_from("<III", blob, at)
            at += 12
            owner = blob[at:at + namesz].rstrip(b"\0").decode()
            at += (namesz + 3) & ~3
            desc = blob[at:at + descsz]
            at += (descsz + 3) & ~3
            yield owner, ntype, desc


def kernels_of(path: str) -> list[dict]:
    """One dict per kernel of the code object: name, vgprs, agprs, sgprs, lds_bytes (static),
    scratch_bytes (per lane), vgpr_spills, sgpr_spills, max_threads."""
    import msgpack
    with open(path, "rb") as f:
        blob = _device_image(f.read())
    out = []
    for owner, ntype, desc in _notes(blob):
        if owner != "AMDGPU" or ntype != NT_AMDGPU_METADATA:
            continue
        meta = msgpack.unpackb(desc, raw=False, strict_map_key=False)
        for k in meta.get("amdhsa.kernels", []):
            out.append({
                "name": k[".name"],
                "vgprs": k.get(".vgpr_count", 0),
                "agprs": k.get(".agpr_count", 0),
                "sgprs": k.get(".sgpr_count", 0),
                "lds_bytes": k.get(".group_segment_fixed_size", 0),
                "scratch_bytes": k.get(".private_segment_fixed_size", 0),
                "vgpr_spills": k.get(".vgpr_spill_count", 0),
                "sgpr_spills": k.get(".sgpr_spill_count", 0),
                "max_threads": k.get(".max_flat_workgroup_size", 0),
            })
    return out


def all_kernels(build_dir: str = BUILD) -> dict[str, dict]:
    """name -> resources over every built code object of the library."""
    found: dict[str, dict] = {}
    for path in sorted(glob.glob(os.path.join(build_dir, "kernels_*.hsaco"))):
        for k in kernels_of(path):
            k["unit"] = os.path.basename(path)[len("kernels_"):-len(".hsaco")]
            found[k["name"]] = k
    return found


if __name__ == "__main__":
    rows = all_kernels()
    print(f"{'kernel':44s} {'unit':12s} vgprs agprs sgprs scratch threads")
    for name, k in sorted(rows.items()):
        print(f"{name:44s} {k['unit']:12s} {k['vgprs']:5d} {k['agprs']:5d} {k['sgprs']:5d} {k['scratch_bytes']:7d} {k['max_threads']:7d}")
