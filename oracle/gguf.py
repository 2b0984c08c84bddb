"""GGUF directory parser -- CPU restatement, test infrastructure only.

Follows rust/crates/lev-gguf/src/lib.rs of the reference (bounds :11-19, block
layouts :94-112, values :137-176, parse :407-486) with the two extra checks of
the Swift reader that the MoE binding relies on (duplicate tensor names and zero
dimensions, Sources/LeviathanCore/GGUF.swift:232-247, 141-174).  Only tests use
it: the C++ reader in leviathan_amd/host/ is checked against its dump.
"""
from __future__ import annotations

import struct

MAX_KV = 1 << 16
MAX_TENSORS = 1 << 20
MAX_STRING = 1 << 24
MAX_DIMS = 8
KEPT_ARRAY_LEN = 64
DEFAULT_ALIGNMENT = 32

# (elements per block, bytes per block), lev-gguf/src/lib.rs:94-112
BLOCK_LAYOUT = {
    0: (1, 4), 1: (1, 2), 30: (1, 2),
    2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 9: (32, 36),
    10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 15: (256, 292),
}
SCALAR = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<B", 10: "<Q", 11: "<q", 12: "<d"}
U64_MAX = (1 << 64) - 1


class GgufError(ValueError):
    pass


class _Cursor:
    def __init__(self, data: bytes):
        self.data, self.pos = data, 0

    def take(self, n: int) -> bytes:
        if n < 0 or self.pos + n > len(self.data):
            raise GgufError("truncated")
        b = self.data[self.pos:self.pos + n]
        self.pos += n
        return b

    def u32(self) -> int:
        return struct.unpack("<I", self.take(4))[0]

    def u64(self) -> int:
        return struct.unpack("<Q", self.take(8))[0]

    def string(self) -> bytes:
        n = self.u64()
        if n > MAX_STRING:
            raise GgufError(f"string length {n} exceeds {MAX_STRING}")
        raw = self.take(n)
        try:
            raw.decode("utf-8")
        except UnicodeDecodeError:
            raise GgufError("string is not valid utf-8")
        return raw

    def scalar(self, ty: int):
        if ty == 8:
            return self.string()
        if ty not in SCALAR:
            raise GgufError(f"unsupported value type {ty}")
        fmt = SCALAR[ty]
        raw = self.take(struct.calcsize(fmt))
        if ty in (6, 12):                      # floats are compared by their bits
            return int.from_bytes(raw, "little")
        v = struct.unpack(fmt, raw)[0]
        return int(v != 0) if ty == 7 else v


def byte_size(ty: int, dims) -> int | None:
    """TensorInfo::byte_size, lib.rs:187-201 (None: unknown type, overflow, partial block)."""
    if ty not in BLOCK_LAYOUT:
        return None
    n = 1
    for d in dims:
        n *= d
        if n > U64_MAX:
            return None
    elems, nbytes = BLOCK_LAYOUT[ty]
    if n % elems:
        return None
    size = n // elems * nbytes
    return size if size <= U64_MAX else None


def parse(data: bytes, file_len: int | None = None) -> dict:
    """lev-gguf parse(): header, metadata, tensor directory; no weight bytes are read."""
    file_len = len(data) if file_len is None else file_len
    c = _Cursor(data)
    if c.take(4) != b"GGUF":
        raise GgufError("missing GGUF magic")
    version = c.u32()
    if not 2 <= version <= 3:
        raise GgufError(f"unsupported version {version}")
    tensor_count, kv_count = c.u64(), c.u64()
    if tensor_count > MAX_TENSORS:
        raise GgufError("tensor count")
    if kv_count > MAX_KV:
        raise GgufError("metadata count")
    metadata, skipped = {}, {}
    for _ in range(kv_count):
        key = c.string()
        ty = c.u32()
        elements_at = c.pos + 12
        if ty != 9:
            value = (ty, c.scalar(ty))
        else:
            et, n = c.u32(), c.u64()
            if et == 9:
                raise GgufError("nested arrays are not supported")
            if n <= KEPT_ARRAY_LEN:
                value = (9, (et, n, [c.scalar(et) for _ in range(n)]))
            else:
                if et == 8:
                    for _ in range(n):
                        c.string()
                else:
                    if et not in SCALAR:
                        raise GgufError(f"unsupported array element type {et}")
                    total = n * struct.calcsize(SCALAR[et])
                    if total > U64_MAX:
                        raise GgufError("array byte length overflows")
                    c.take(total)
                value = (9, (et, n, None))
                skipped[key] = (et, n, elements_at)
        if key in metadata:
            raise GgufError("duplicate metadata key")
        metadata[key] = value
    tensors, names = [], set()
    for _ in range(tensor_count):
        name = c.string()
        nd = c.u32()
        if nd == 0 or nd > MAX_DIMS:
            raise GgufError("bad dimension count")
        dims = [c.u64() for _ in range(nd)]
        ty, off = c.u32(), c.u64()
        if name in names:
            raise GgufError("duplicate tensor name")
        names.add(name)
        tensors.append({"name": name, "dims": dims, "type": ty, "offset": off})
    alignment = DEFAULT_ALIGNMENT
    if b"general.alignment" in metadata:
        ty, v = metadata[b"general.alignment"]
        ok = ty in (0, 1, 2, 3, 4, 5, 10, 11) and v > 0 and (v & (v - 1)) == 0
        if not ok:
            raise GgufError("general.alignment is not a positive power of two")
        alignment = v
    data_offset = -(-c.pos // alignment) * alignment
    if data_offset > file_len:
        raise GgufError("tensor data section starts past end of file")
    for t in tensors:
        size = byte_size(t["type"], t["dims"])
        if size is None:
            raise GgufError(f"tensor {t['name']!r}: unsupported or inconsistent size")
        if any(d == 0 for d in t["dims"]):
            raise GgufError("zero dimension")
        if t["offset"] % alignment:
            raise GgufError("offset not aligned")
        end = data_offset + t["offset"] + size
        if end > U64_MAX or end > file_len:
            raise GgufError("extent exceeds file length")
        t["size"] = size
    return {"version": version, "alignment": alignment, "data_offset": data_offset, "file_len": file_len,
            "metadata": metadata, "tensors": tensors, "skipped": skipped}


def _repr(ty: int, v) -> str:
    if ty == 8:
        return v.hex() or "-"
    if ty == 9:
        et, n, vals = v
        body = "skipped" if vals is None else " ".join(_repr(et, x) for x in vals)
        return f"[{et} {n} {body}]".replace(" ]", "]")
    return str(v)


def dump(g: dict) -> str:
    """Canonical text form of a parsed directory; the C++ reader prints the same."""
    out = [f"version {g['version']}", f"alignment {g['alignment']}", f"data_offset {g['data_offset']}",
           f"file_len {g['file_len']}"]
    for key in sorted(g["metadata"]):
        ty, v = g["metadata"][key]
        out.append(f"kv {key.hex()} {ty} {_repr(ty, v)}")
    for key in sorted(g["skipped"]):
        et, n, at = g["skipped"][key]
        out.append(f"skipped {key.hex()} {et} {n} {at}")
    for t in g["tensors"]:
        dims = ",".join(str(d) for d in t["dims"])
        out.append(f"tensor {t['name'].hex()} {t['type']} {dims} {t['offset']} {t['size']}")
    return "\n".join(out) + "\n"
