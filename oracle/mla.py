"""CPU restatement of the reference's multi-head latent attention (DeepSeek-V2 /
V3 / Kimi-K2 `deepseek2` graphs).  TEST INFRASTRUCTURE (see oracle/__init__.py).

Follows src/quantized_deepseek2.rs: the YaRN-aware rotary tables (:226-345), the
Q projection, plain or low-rank (:357-371), the combined KV up-projection and
its reconstruction from the pre-split tensors (:405-420, :931-958) and
`Attention::forward` in its unabsorbed form with the per-head K/V cache kept
transposed and appended per call (:422-499); the causal mask is the model's
(:875-889: a mask for more than one token, none for a single one).

RMSNorm, softmax, the interleaved rotary op (`rope_i`), cos/sin and the f32
attention matmuls are third-party candle ops: their formulas are public, their
ulp-level rounding order is not pinned by anything in the reference, so
comparisons against this file use a relative bound.

What pins this file (tests/test_mla_oracle.py): closed forms of the YaRN helpers,
the rotation as a complex multiplication (sign and pairing), the reference's own
invariants (cache shapes :1184-1209, prefill == incremental :1213-1256) and a
textbook per-head, per-query attention written with explicit loops in float64.
"""
from __future__ import annotations

import math

import numpy as np

from . import dequantize, matmul_t
from .qwen3 import rmsnorm

f32 = np.float32


def yarn_get_mscale(scale: float, mscale: float) -> float:
    """0.1 * mscale * ln(scale) + 1 for scale > 1, else 1 (:230-236), in f32."""
    if scale <= 1.0:
        return 1.0
    return float(f32(f32(f32(0.1) * f32(mscale)) * f32(np.log(f32(scale))) + f32(1.0)))


def yarn_find_correction_dim(num_rot: float, dim: int, base: float, max_pos: int) -> float:
    """(:314-317)"""
    return float(f32(f32(dim) * f32(np.log(f32(f32(max_pos) / f32(f32(num_rot) * f32(2.0) * f32(np.pi))))))
                 / f32(f32(2.0) * f32(np.log(f32(base)))))


def yarn_correction_range(low_rot: float, high_rot: float, dim: int, base: float, max_pos: int):
    """(:319-329)"""
    low = math.floor(yarn_find_correction_dim(low_rot, dim, base, max_pos))
    high = math.ceil(yarn_find_correction_dim(high_rot, dim, base, max_pos))
    return max(float(low), 0.0), min(float(high), float(dim) - 1.0)


def yarn_linear_ramp(lo: float, hi: float, dim: int) -> np.ndarray:
    """(:331-339)"""
    if abs(lo - hi) < float(np.finfo(f32).eps):
        hi += 0.001
    lo, hi = f32(lo), f32(hi)
    return np.clip((np.arange(dim, dtype=f32) - lo) / (hi - lo), f32(0), f32(1)).astype(f32)


def softmax_scale(cfg: dict) -> float:
    """1/sqrt(q_head_dim), times mscale^2 under YaRN (:186-192), in f64 as there."""
    s = 1.0 / math.sqrt(cfg["qk_nope"] + cfg["qk_rope"])
    y = cfg.get("yarn")
    if y:
        m = yarn_get_mscale(y["factor"], y["mscale_all_dim"])
        s *= m * m
    return s


def rope_tables(cfg: dict):
    """cos, sin of shape [context_length, qk_rope / 2], scaled by the YaRN mscale (:246-301)."""
    dim, theta = cfg["qk_rope"], f32(cfg["rope_theta"])
    max_seq = max(cfg["context_length"], 1)
    extra = (f32(1) / np.power(theta, np.arange(0, dim, 2, dtype=f32) / f32(dim), dtype=f32)).astype(f32)
    y = cfg.get("yarn")
    if not y:
        inv, mscale = extra, 1.0
    else:
        half = dim // 2
        inter = (f32(1) / (f32(y["factor"]) * np.power(theta, np.arange(0, dim, 2, dtype=f32) / f32(dim), dtype=f32))).astype(f32)
        lo, hi = yarn_correction_range(32.0, 1.0, dim, float(theta), y["orig_context_length"])
        ramp = yarn_linear_ramp(lo, hi, half)
        mask = (f32(1) - ramp).astype(f32)
        inv = (inter * (f32(1) - mask) + extra * mask).astype(f32)
        mscale = yarn_get_mscale(y["factor"], y["mscale_all_dim"])
    freqs = (np.arange(max_seq, dtype=f32)[:, None] * inv[None, :]).astype(f32)
    return (np.cos(freqs, dtype=f32) * f32(mscale)).astype(f32), (np.sin(freqs, dtype=f32) * f32(mscale)).astype(f32)


def rope_interleaved(v: np.ndarray, cos: np.ndarray, sin: np.ndarray, offset: int) -> np.ndarray:
    """v: [T, heads, d]; rotates the neighbouring pairs (2i, 2i + 1) of token t by row
    offset + t of the tables (candle's `rope_i`, the llama.cpp NORM type; :302-311)."""
    T = v.shape[0]
    c, s = cos[offset:offset + T, None, :], sin[offset:offset + T, None, :]
    a, b = v[..., 0::2], v[..., 1::2]
    out = np.empty_like(v, dtype=f32)
    out[..., 0::2] = a * c - b * s
    out[..., 1::2] = a * s + b * c
    return out


def fold_kv_b(k_b: np.ndarray, v_b: np.ndarray, cfg: dict) -> np.ndarray:
    """The combined [n_head * (qk_nope + v_head_dim), kv_lora_rank] up-projection from the
    pre-split tensors k_b [n_head, kv_lora_rank, qk_nope] and v_b [n_head, v_head_dim,
    kv_lora_rank] (:931-958)."""
    h, lkv, npe, vh = cfg["n_head"], cfg["kv_lora_rank"], cfg["qk_nope"], cfg["v_head_dim"]
    k_b, v_b = np.asarray(k_b, f32).reshape(h, lkv, npe), np.asarray(v_b, f32).reshape(h, vh, lkv)
    return np.concatenate([np.concatenate([k_b[i].T, v_b[i]], axis=0) for i in range(h)], axis=0)


def softmax_last(x: np.ndarray) -> np.ndarray:
    m = x.max(axis=-1, keepdims=True)
    e = np.exp((x - m).astype(f32), dtype=f32)
    return (e / e.sum(axis=-1, keepdims=True, dtype=f32)).astype(f32)


class MlaOracle:
    """cfg: n_embd, n_head, q_lora_rank (0 for the plain projection), kv_lora_rank, qk_nope,
    qk_rope, v_head_dim, rms_eps, rope_theta, context_length, yarn (None or a dict with factor,
    orig_context_length, mscale_all_dim).  tensors: name -> (qtype, blocks) for the matrices
    ("q" or "q_a" and "q_b", "kv_a_mqa", "kv_b", "o"; qtype 0 holds a dense f32 matrix) and
    f32 vectors for "q_a_norm" and "kv_a_norm"."""

    def __init__(self, cfg: dict, tensors: dict, *, avx2: bool = True):
        self.c, self.t, self.avx2 = cfg, tensors, avx2
        self.cos, self.sin = rope_tables(cfg)
        self.scale = softmax_scale(cfg)
        self.k_cache = self.v_cache = None  # [n_head, q_head_dim, seq], [n_head, v_head_dim, seq]

    def reset(self) -> None:
        self.k_cache = self.v_cache = None

    def mm(self, name: str, x: np.ndarray, n: int) -> np.ndarray:
        qt, w = self.t[name]
        x = np.ascontiguousarray(x, f32)
        if qt == 0:
            return (x @ np.asarray(w, f32).reshape(n, x.shape[1]).T).astype(f32)
        return matmul_t(qt, (x.shape[0], x.shape[1], n), x, w, avx2=self.avx2)

    def forward(self, x: np.ndarray, offset: int, masked: bool | None = None) -> np.ndarray:
        """x: [T, n_embd] -> [T, n_embd]; appends T tokens to the cache."""
        c = self.c
        T, nh, lkv, npe, r, vh = x.shape[0], c["n_head"], c["kv_lora_rank"], c["qk_nope"], c["qk_rope"], c["v_head_dim"]
        qd = npe + r
        if c.get("q_lora_rank"):
            qa = rmsnorm(self.mm("q_a", x, c["q_lora_rank"]), self.t["q_a_norm"], c["rms_eps"])
            q = self.mm("q_b", qa, nh * qd)
        else:
            q = self.mm("q", x, nh * qd)
        q = q.reshape(T, nh, qd)
        comp = self.mm("kv_a_mqa", x, lkv + r)
        kv_cmpr, k_pe = comp[:, :lkv], comp[:, lkv:].reshape(T, 1, r)
        q_pe = rope_interleaved(q[..., npe:], self.cos, self.sin, offset)
        k_pe = rope_interleaved(k_pe, self.cos, self.sin, offset)
        q = np.concatenate([q[..., :npe], q_pe], axis=-1)
        kv = self.mm("kv_b", rmsnorm(kv_cmpr, self.t["kv_a_norm"], c["rms_eps"]), nh * (npe + vh)).reshape(T, nh, npe + vh)
        k_new = np.concatenate([kv[..., :npe], np.broadcast_to(k_pe, (T, nh, r))], axis=-1)  # [T, nh, qd]
        k_new, v_new = k_new.transpose(1, 2, 0), kv[..., npe:].transpose(1, 2, 0)            # [nh, dim, T]
        if self.k_cache is None:
            self.k_cache, self.v_cache = np.ascontiguousarray(k_new), np.ascontiguousarray(v_new)
        else:
            self.k_cache = np.concatenate([self.k_cache, k_new], axis=2)
            self.v_cache = np.concatenate([self.v_cache, v_new], axis=2)
        scores = (np.matmul(q.transpose(1, 0, 2), self.k_cache).astype(f32) * f32(self.scale)).astype(f32)  # [nh, T, total]
        if masked if masked is not None else T > 1:
            total = scores.shape[-1]
            j, i = np.arange(total)[None, :], np.arange(T)[:, None]
            scores = np.where(j > i + offset, f32(-np.inf), scores)
        probs = softmax_last(scores)
        ctx = np.matmul(self.v_cache, probs.transpose(0, 2, 1)).astype(f32)  # [nh, vh, T]
        ctx = ctx.transpose(2, 0, 1).reshape(T, nh * vh)
        return self.mm("o", ctx, c["n_embd"])


def dense(qtype: int, blocks, n: int, k: int) -> np.ndarray:
    """The matrix a tensor entry stands for, as f32 [n, k]."""
    if qtype == 0:
        return np.asarray(blocks, f32).reshape(n, k)
    return dequantize(qtype, blocks).reshape(n, k)
