"""Random-weight Qwen3 decoder tensors in the block types a Q4_K_M GGUF holds.

There is no network for checkpoints, so the end-to-end harness runs on seeded
normal weights of the real architecture and tensor-type mix, drawn N(0, 1/sqrt(k))
for a matrix of k columns so that every product keeps its input's scale through
all layers (at N(0, 0.02), 1.3 to 2.2 times that, the 36-layer model's logits
differ from the CPU restatement's by up to 1.7e-3 of max(|ref|, 1): the 15-bit
fixed point of the activations compounds past the 1e-3 a single product is held
to; the bytes read are the same either way): everything
Q4_K except the output head (Q6_K) and, on the layers llama.cpp's Q4_K_M recipe
gives more bits (first and last eighth, and every third in between), ffn_down in
Q6_K and attn_v in Q6_K or, on every other of those layers, Q8_0 (the three block
types a Q4_K / Q6_K / Q8_0 file mixes).  Norm weights are f32 around 1.
"""
from __future__ import annotations

import zlib

import numpy as np

from . import normal, normal_quantized

Q4_K, Q6_K, Q8_0, F32 = 12, 14, 8, 0


def more_bits(layer: int, n_layer: int) -> bool:
    return layer < n_layer // 8 or layer >= 7 * n_layer // 8 or (layer - n_layer // 8) % 3 == 2


def qwen3_tensor_plan(cfg: dict, mix: str = "q4_k_m"):
    """[(name, qtype, n, k)] for every tensor of the model; k == 0 marks an f32 vector.  With n_expert in
    the configuration the feed-forward tensors are those of a qwen3moe file: the f32 router
    ffn_gate_inp of n_expert * hidden values and the stacked ffn_{gate,up,down}_exps, expert after expert."""
    h, d, ffn = cfg["hidden"], cfg["head_dim"], cfg.get("ffn", 0)
    E, eff = cfg.get("n_expert", 0), cfg.get("expert_ffn", 0)
    qd, kd, L = cfg["n_head"] * d, cfg["n_kv_head"] * d, cfg["n_layer"]
    base = Q4_K if mix in ("q4_k_m", "q4_k") else int(mix)
    plan = [("token_embd.weight", base, cfg["vocab"], h), ("output_norm.weight", F32, h, 0),
            ("output.weight", Q6_K if mix == "q4_k_m" else base, cfg["vocab"], h)]
    for l in range(L):
        hi = Q6_K if (mix == "q4_k_m" and more_bits(l, L)) else base
        hi_v = Q8_0 if (hi == Q6_K and l % 2 == 1) else hi
        p = f"blk.{l}."
        plan += [(p + "attn_norm.weight", F32, h, 0), (p + "attn_q.weight", base, qd, h),
                 (p + "attn_k.weight", base, kd, h), (p + "attn_v.weight", hi_v, kd, h),
                 (p + "attn_q_norm.weight", F32, d, 0), (p + "attn_k_norm.weight", F32, d, 0),
                 (p + "attn_output.weight", base, h, qd), (p + "ffn_norm.weight", F32, h, 0)]
        if E:
            plan += [(p + "ffn_gate_inp.weight", F32, E * h, 0), (p + "ffn_gate_exps.weight", base, E * eff, h),
                     (p + "ffn_up_exps.weight", base, E * eff, h), (p + "ffn_down_exps.weight", hi, E * h, eff)]
        else:
            plan += [(p + "ffn_gate.weight", base, ffn, h), (p + "ffn_up.weight", base, ffn, h),
                     (p + "ffn_down.weight", hi, h, ffn)]
    return plan


def gguf_dims(cfg: dict, name: str, n: int, k: int) -> list:
    """The shape a GGUF directory gives the tensor, slowest dimension first: [n] for vectors, [n, k] for
    matrices, [n_expert, hidden] for the router and [n_expert, out, in] for stacked experts."""
    E = cfg.get("n_expert", 0)
    if name.endswith(".ffn_gate_inp.weight"):
        return [E, n // E]
    if name.endswith("_exps.weight"):
        return [E, n // E, k]
    return [n] if k == 0 else [n, k]


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
            if name.endswith(".ffn_gate_inp.weight"):   # router rows: logits of standard deviation ~1 on a normed row
                cache[key] = normal(s, (n,), float(1.0 / np.sqrt(cfg["hidden"])), 0.0)
            elif k == 0:
                cache[key] = normal(s, (n,), 0.1, 1.0)
            else:
                cache[key] = normal_quantized(qt, s, n * k, float(1.0 / np.sqrt(k)))
        yield name, qt, cache[key]
