"""Writer of GGUF files for the synthetic models of the harness.

The container as its readers expect it (reference reader: src/gguf_ext.rs:400-480):
magic "GGUF", version, tensor count, metadata count (u64 from version 2 on), the
metadata pairs, the tensor directory (name, dimensions fastest first, raw type id,
offset from the start of the data section), padding to general.alignment (32 when
absent), then each tensor's bytes at its aligned offset.
"""
from __future__ import annotations

import struct

import numpy as np

MAGIC = 0x46554747
# value type ids of the container
U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_SCALAR_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q",
               I64: "<q", F64: "<d"}


class Value:
    """A metadata value with an explicit container type; `elem` is the element type of an array."""

    def __init__(self, vtype: int, value, elem: "int | None" = None):
        self.vtype, self.value, self.elem = vtype, value, elem


def u32(v): return Value(U32, v)
def f32(v): return Value(F32, v)
def boolean(v): return Value(BOOL, v)
def string(v): return Value(STRING, v)
def array(elem, items): return Value(ARRAY, items, elem)


def _len(n: int, version: int) -> bytes:
    return struct.pack("<I", n) if version == 1 else struct.pack("<Q", n)


def _string(s, version: int) -> bytes:
    raw = s if isinstance(s, bytes) else s.encode()
    return _len(len(raw), version) + raw


def _payload(vtype: int, value, elem, version: int) -> bytes:
    if vtype == STRING:
        return _string(value, version)
    if vtype == ARRAY:
        out = struct.pack("<I", elem) + _len(len(value), version)
        for item in value:
            if isinstance(item, Value):          # nested array: the item carries its own element type
                out += _payload(item.vtype, item.value, item.elem, version)
            else:
                out += _payload(elem, item, None, version)
        return out
    return struct.pack(_SCALAR_FMT[vtype], value)


def header_bytes(metadata: dict, directory: list, version: int = 3) -> bytes:
    """directory: [(name, dims in row-major order, raw type id, offset)]."""
    out = struct.pack("<II", MAGIC, version) + _len(len(directory), version) + _len(len(metadata), version)
    for key, v in metadata.items():
        out += _string(key, version) + struct.pack("<I", v.vtype) + _payload(v.vtype, v.value, v.elem, version)
    for name, dims, dtype, offset in directory:
        out += _string(name, version) + struct.pack("<I", len(dims))
        for d in reversed(dims):
            out += _len(d, version)
        out += struct.pack("<IQ", dtype, offset)
    return out


def write_gguf(path: str, metadata: dict, tensors: list, alignment: "int | None" = None, version: int = 3) -> dict:
    """tensors: [(name, raw type id, dims in row-major order, bytes-like)].  Returns
    {name: absolute file offset}."""
    md = dict(metadata)
    if alignment is not None:
        md["general.alignment"] = u32(alignment)
    align = alignment or 32
    directory, blobs, off = [], [], 0
    for name, dtype, dims, data in tensors:
        raw = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
        directory.append((name, list(dims), dtype, off))
        blobs.append((off, raw))
        off = (off + raw.size + align - 1) // align * align
    head = header_bytes(md, directory, version)
    data_start = (len(head) + align - 1) // align * align
    where = {}
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * (data_start - len(head)))
        for (name, *_), (o, raw) in zip(directory, blobs):
            f.seek(data_start + o)
            f.write(raw.tobytes())
            where[name] = data_start + o
        end = data_start + off
        if f.tell() < end:
            f.seek(end - 1)
            f.write(b"\0")
    return where


def qwen3_metadata(cfg: dict, with_key_length: bool = True, with_ffn: bool = True, with_norm_topk=None) -> dict:
    """The `qwen3.*` keys a dense Qwen3 file carries, or with n_expert in the configuration the
    `qwen3moe.*` keys of a mixture-of-experts one (read by the loader at
    reference: src/quantized_qwen3_moe.rs:90-147).  with_norm_topk: True / False writes
    attention.norm_topk_prob, None leaves it out (the loader then takes true)."""
    a = "qwen3moe" if cfg.get("n_expert") else "qwen3"
    md = {"general.architecture": string(a), "general.name": string("synthetic-" + a),
          a + ".block_count": u32(cfg["n_layer"]), a + ".embedding_length": u32(cfg["hidden"]),
          a + ".attention.head_count": u32(cfg["n_head"]), a + ".attention.head_count_kv": u32(cfg["n_kv_head"]),
          a + ".context_length": u32(cfg.get("context_length", cfg["n_ctx"])),
          a + ".attention.layer_norm_rms_epsilon": f32(cfg["rms_eps"]), a + ".rope.freq_base": f32(cfg["rope_theta"])}
    if with_key_length:
        md[a + ".attention.key_length"] = u32(cfg["head_dim"])
        md[a + ".attention.value_length"] = u32(cfg["head_dim"])
    if cfg.get("n_expert"):
        md[a + ".expert_count"] = u32(cfg["n_expert"])
        md[a + ".expert_used_count"] = u32(cfg["n_expert_used"])
        md[a + ".expert_feed_forward_length"] = u32(cfg["expert_ffn"])
        if with_norm_topk is not None:
            md[a + ".attention.norm_topk_prob"] = boolean(bool(with_norm_topk))
    elif with_ffn:
        md[a + ".feed_forward_length"] = u32(cfg["ffn"])
    return md


def write_qwen3(path: str, cfg: dict, tensors, plan, **kw) -> dict:
    """tensors: iterable of (name, qtype, data) as qwen3_tensors yields; plan: qwen3_tensor_plan
    of the same configuration (for the shapes)."""
    from .model import gguf_dims
    shapes = {name: gguf_dims(cfg, name, n, k) for name, _, n, k in plan}
    items = [(name, qt, shapes[name], data) for name, qt, data in tensors]
    md_kw = {k: kw.pop(k) for k in ("with_key_length", "with_ffn", "with_norm_topk") if k in kw}
    return write_gguf(path, qwen3_metadata(cfg, **md_kw), items, **kw)
