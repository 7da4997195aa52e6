"""Random-weight Qwen3 decoder tensors in the block types a Q4_K_M GGUF holds.

There is no network for checkpoints, so the end-to-end harness runs on seeded
normal weights of the real architecture and tensor-type mix: everything Q4_K
except the output head and, on the layers llama.cpp's Q4_K_M recipe gives more
bits (first and last eighth, and every third in between), attn_v and ffn_down
in Q6_K.  Norm weights are f32 around 1.
"""
from __future__ import annotations

import zlib

import numpy as np

from . import normal, normal_quantized

Q4_K, Q6_K, F32 = 12, 14, 0


def more_bits(layer: int, n_layer: int) -> bool:
    return layer < n_layer // 8 or layer >= 7 * n_layer // 8 or (layer - n_layer // 8) % 3 == 2


def qwen3_tensor_plan(cfg: dict, mix: str = "q4_k_m"):
    """[(name, qtype, n, k)] for every tensor of the model; k == 0 marks an f32 vector."""
    h, d, ffn = cfg["hidden"], cfg["head_dim"], cfg["ffn"]
    qd, kd, L = cfg["n_head"] * d, cfg["n_kv_head"] * d, cfg["n_layer"]
    base = Q4_K if mix in ("q4_k_m", "q4_k") else int(mix)
    plan = [("token_embd.weight", base, cfg["vocab"], h), ("output_norm.weight", F32, h, 0),
            ("output.weight", Q6_K if mix == "q4_k_m" else base, cfg["vocab"], h)]
    for l in range(L):
        hi = Q6_K if (mix == "q4_k_m" and more_bits(l, L)) else base
        p = f"blk.{l}."
        plan += [(p + "attn_norm.weight", F32, h, 0), (p + "attn_q.weight", base, qd, h),
                 (p + "attn_k.weight", base, kd, h), (p + "attn_v.weight", hi, kd, h),
                 (p + "attn_q_norm.weight", F32, d, 0), (p + "attn_k_norm.weight", F32, d, 0),
                 (p + "attn_output.weight", base, h, qd), (p + "ffn_norm.weight", F32, h, 0),
                 (p + "ffn_gate.weight", base, ffn, h), (p + "ffn_up.weight", base, ffn, h),
                 (p + "ffn_down.weight", hi, h, ffn)]
    return plan


def qwen3_tensors(cfg: dict, seed: int, mix: str = "q4_k_m", share_layers: bool = False):
    """Yields (name, qtype, data).  With share_layers the bytes of a tensor are drawn once
    per (role, type, shape) and repeated on every layer, which keeps generating an
    8B-parameter model to seconds; each layer still gets its own copy in HBM."""
    cache: dict = {}
    for i, (name, qt, n, k) in enumerate(qwen3_tensor_plan(cfg, mix)):
        role = name.split(".", 2)[-1] if name.startswith("blk.") else name
        key = (role, qt, n, k) if share_layers else (name,)
        if key not in cache:
            s = seed * 1000003 + (zlib.crc32(role.encode()) % 1000 if share_layers else i)
            if k == 0:
                cache[key] = normal(s, (n,), 0.1, 1.0)
            else:
                cache[key] = normal_quantized(qt, s, n * k, float(1.0 / np.sqrt(k)))
        yield name, qt, cache[key]
