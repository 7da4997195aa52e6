"""CPU restatement of the reference's tolerant GGUF header reader.  TEST INFRASTRUCTURE:
only tests, the smoke check and the benchmark's CPU leg may import this module.

Follows src/gguf_ext.rs: limits :33-59, value reader :293-398, read_header :400-480,
type_size_bytes :483-512, architecture :148-152.  Pinned by the reference's own parser
tests (src/gguf_ext.rs:515-949), restated byte for byte in tests/test_gguf.py.
"""
from __future__ import annotations

import struct

MAGIC = 0x46554747
DEFAULT_ALIGNMENT = 32
MAX_COUNT = 1 << 24
MAX_STRING_LENGTH = 1 << 24
MAX_ARRAY_ELEMENTS = 1 << 24
MAX_VALUE_DEPTH = 64


class GgufError(ValueError):
    pass


def _bad(msg: str) -> GgufError:            # src/gguf_ext.rs:289-291
    return GgufError(f"GGUF header: {msg}")


def type_size_bytes(dtype: int, elems: int):
    """src/gguf_ext.rs:483-512."""
    table = {0: (1, 4), 1: (1, 2), 30: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34),
             9: (32, 36), 10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210),
             15: (256, 292), 26: (1, 4), 16: (256, 66), 39: (32, 17)}
    if dtype not in table:
        return None
    blck, nbytes = table[dtype]
    if elems % blck:
        return None
    return elems // blck * nbytes


class _Rdr:
    def __init__(self, data: bytes):
        self.d, self.pos, self.version = data, 0, 0

    def take(self, n: int) -> bytes:
        if self.pos + n > len(self.d):
            raise _bad("failed to fill whole buffer")
        out = self.d[self.pos:self.pos + n]
        self.pos += n
        return out

    def u32(self) -> int:
        return struct.unpack("<I", self.take(4))[0]

    def u64(self) -> int:
        return struct.unpack("<Q", self.take(8))[0]

    def len(self) -> int:                       # :310-316
        return self.u32() if self.version == 1 else self.u64()

    def string(self) -> str:                    # :317-351
        n = self.len()
        if n > MAX_STRING_LENGTH:
            raise _bad(f"string of {n} bytes exceeds max {MAX_STRING_LENGTH}")
        left = len(self.d) - self.pos
        if n > left:
            raise _bad(f"string of {n} bytes exceeds the {left} bytes remaining in the stream")
        raw = self.take(n).rstrip(b"\0")
        return raw.decode("utf-8", errors="replace")

    def value(self, ty: int, depth: int):       # :353-397
        if depth > MAX_VALUE_DEPTH:
            raise _bad(f"value nesting depth exceeds max {MAX_VALUE_DEPTH}")
        fmt = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 10: "<Q", 11: "<q", 12: "<d"}
        if ty in fmt:
            return (ty, struct.unpack(fmt[ty], self.take(struct.calcsize(fmt[ty])))[0])
        if ty == 7:
            return (7, self.take(1)[0] != 0)
        if ty == 8:
            return (8, self.string())
        if ty == 9:
            elem = self.u32()
            n = self.len()
            if n > MAX_ARRAY_ELEMENTS:
                raise _bad(f"array of {n} elements exceeds max {MAX_ARRAY_ELEMENTS}")
            return (9, [self.value(elem, depth + 1) for _ in range(n)])
        raise _bad(f"unknown metadata value type {ty}")


def read_header(data: bytes) -> dict:
    """{"version", "metadata": {key: (type, value)}, "tensors": {name: (dtype, dims, offset)},
    "tensor_data_offset"}; dims are reversed into row-major order (:444-447)."""
    rd = _Rdr(data)
    if rd.u32() != MAGIC:
        raise _bad("not a GGUF file (bad magic)")
    version = rd.u32()
    if not 1 <= version <= 3:
        raise _bad(f"unsupported GGUF version {version}")
    rd.version = version
    tensor_count, kv_count = rd.len(), rd.len()
    if tensor_count > MAX_COUNT or kv_count > MAX_COUNT:
        raise _bad("implausible tensor/metadata count")
    metadata = {}
    for _ in range(kv_count):
        key = rd.string()
        ty = rd.u32()
        metadata[key] = rd.value(ty, 0)
    tensors = {}
    for _ in range(tensor_count):
        name = rd.string()
        n_dims = rd.u32()
        if n_dims > 8:
            raise _bad(f"tensor `{name}` claims {n_dims} dimensions")
        dims = [rd.len() for _ in range(n_dims)][::-1]
        dtype = rd.u32()
        offset = rd.u64()
        tensors[name] = (dtype, dims, offset)
    alignment = DEFAULT_ALIGNMENT               # :456-468
    if "general.alignment" in metadata:
        ty, v = metadata["general.alignment"]
        if ty in (0, 2, 4) or (ty in (1, 3, 5) and v >= 0):
            alignment = v
    if alignment == 0 or alignment & (alignment - 1):
        raise _bad(f"invalid general.alignment {alignment}")
    tdo = (rd.pos + alignment - 1) // alignment * alignment
    return {"version": version, "metadata": metadata, "tensors": tensors, "tensor_data_offset": tdo}


def architecture(header: dict):
    v = header["metadata"].get("general.architecture")
    return v[1] if v and v[0] == 8 else None
