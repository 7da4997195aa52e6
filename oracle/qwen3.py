"""CPU restatement of the reference's Qwen3 decoder graph, dense or with
mixture-of-experts feed-forward blocks, on top of the oracle matmul.  TEST INFRASTRUCTURE (see oracle/__init__.py).

Layer structure follows src/embedding.rs:297-396 (pre-norm residual blocks,
per-head Q/K RMSNorm before RoPE, half-split rotary pairs, grouped-query
attention, SwiGLU MLP); KV cache, causal mask and last-token logits follow
src/quantized_qwen3_moe.rs:366-386,776-826; with n_expert in the configuration
every layer's feed-forward block is the mixture of experts of :404-528, 806-812
(oracle/moe.py).  RMSNorm, softmax, silu, the f32
attention matmuls and cos/sin are third-party candle ops: their formulas are
public, their ulp-level rounding order is not pinned by anything in the
reference, so comparisons against this file use a relative bound on the logits
and exact agreement of the greedy token only where the top-2 margin exceeds it.
"""
from __future__ import annotations

import time

import numpy as np

from . import dequantize, matmul_t
from .moe import MoeOracle, silu

f32 = np.float32


def rmsnorm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    x = x.astype(f32)
    ms = (x * x).sum(axis=-1, keepdims=True, dtype=f32) / f32(x.shape[-1])
    return (x / np.sqrt(ms + f32(eps), dtype=f32) * w.astype(f32)).astype(f32)


def rope_half_split(v: np.ndarray, pos0: int, theta: float) -> np.ndarray:
    """v: [T, heads, d]; rotates pairs (i, i + d/2) by (pos0 + t) * theta^(-2i/d)
    (src/quantized_qwen3_moe.rs:237-262; closed form checked in its test :867-895)."""
    T, _, d = v.shape
    half = d // 2
    inv = (f32(1) / np.power(f32(theta), np.arange(0, d, 2, dtype=f32) / f32(d), dtype=f32)).astype(f32)
    ang = (np.arange(pos0, pos0 + T, dtype=f32)[:, None] * inv[None, :]).astype(f32)
    c, s = np.cos(ang, dtype=f32)[:, None, :], np.sin(ang, dtype=f32)[:, None, :]
    a, b = v[..., :half], v[..., half:]
    return np.concatenate([a * c - b * s, a * s + b * c], axis=-1).astype(f32)


def gqa_attention(q: np.ndarray, K: np.ndarray, V: np.ndarray, pos: int) -> np.ndarray:
    """softmax(q K^T / sqrt(d) + causal mask) V per query head; q: [T, n_head, d] for the tokens at
    positions pos .. pos + T - 1, K and V: [pos + T, n_kv_head, d], the whole cache.  Query head h reads
    KV head h // (n_head / n_kv_head): repeat_kv lays the copies of a KV head side by side
    (src/quantized_qwen3_moe.rs:267-278, :366-381); token t sees keys 0 .. pos + t (mask :776-789)."""
    T, nh, d = q.shape
    rep = nh // K.shape[1]
    att = np.empty((T, nh, d), f32)
    for hq in range(nh):
        kv = hq // rep
        sc = (q[:, hq, :] @ K[:, kv, :].T).astype(f32) / f32(np.sqrt(f32(d)))
        mask = np.arange(K.shape[0])[None, :] > (pos + np.arange(T))[:, None]
        sc = np.where(mask, f32(-np.inf), sc)
        e = np.exp(sc - sc.max(axis=-1, keepdims=True), dtype=f32)
        pr = (e / e.sum(axis=-1, keepdims=True, dtype=f32)).astype(f32)
        att[:, hq, :] = pr @ V[:, kv, :]
    return att


class Qwen3Oracle:
    """cfg: dict with n_layer, hidden, n_head, n_kv_head, head_dim, ffn, vocab, rms_eps,
    rope_theta; a mixture-of-experts model adds n_expert, n_expert_used, expert_ffn and
    norm_topk_prob (default True).  tensors: name -> (qtype, data) with qtype 0 for f32
    vectors and the router."""

    def __init__(self, cfg: dict, tensors: dict, *, avx2: bool = True, threads: int = 0):
        self.c, self.t, self.avx2, self.threads = cfg, tensors, avx2, threads
        self._moe: dict = {}
        self.reset()

    def reset(self) -> None:
        self.k = [None] * self.c["n_layer"]
        self.v = [None] * self.c["n_layer"]
        self.n_past = 0
        self.mm_seconds = 0.0   # time spent inside the C matmul kernels (the rest is this numpy graph)

    def mm(self, name: str, x: np.ndarray, n: int) -> np.ndarray:
        qt, blocks = self.t[name]
        m, k = x.shape
        t0 = time.perf_counter()
        y = matmul_t(qt, (m, k, n), np.ascontiguousarray(x, f32), blocks, avx2=self.avx2, threads=self.threads)
        self.mm_seconds += time.perf_counter() - t0
        return y

    def moe(self, l: int) -> MoeOracle:
        """The layer's expert block from its four tensors (src/quantized_qwen3_moe.rs:653-675)."""
        if l not in self._moe:
            c, p = self.c, f"blk.{l}."
            as_bytes = lambda name: np.frombuffer(bytes(self.t[name][1]), np.uint8) if not isinstance(
                self.t[name][1], np.ndarray) else self.t[name][1].view(np.uint8).ravel()
            qg, qu, qd = (self.t[p + f"ffn_{r}_exps.weight"][0] for r in ("gate", "up", "down"))
            assert qg == qu
            router = np.asarray(self.t[p + "ffn_gate_inp.weight"][1], f32).reshape(c["n_expert"], c["hidden"])
            self._moe[l] = MoeOracle(qg, c["hidden"], c["expert_ffn"], c["n_expert"], c["n_expert_used"], router,
                                     as_bytes(p + "ffn_gate_exps.weight"), as_bytes(p + "ffn_up_exps.weight"),
                                     as_bytes(p + "ffn_down_exps.weight"), gating="softmax",
                                     norm_topk=bool(c.get("norm_topk_prob", True)), avx2=self.avx2, qtype_down=qd)
        return self._moe[l]

    def vec(self, name: str) -> np.ndarray:
        return np.asarray(self.t[name][1], f32)

    def embed(self, tokens) -> np.ndarray:
        qt, blocks = self.t["token_embd.weight"]
        h = self.c["hidden"]
        from . import block_geometry
        be, bb = block_geometry(qt)
        row = h // be * bb
        raw = np.frombuffer(bytes(blocks), np.uint8) if not isinstance(blocks, np.ndarray) else blocks.view(np.uint8).ravel()
        return np.stack([dequantize(qt, raw[t * row:(t + 1) * row]) for t in tokens]).astype(f32)

    def forward(self, tokens, pos: int) -> np.ndarray:
        c = self.c
        assert pos == self.n_past
        T, h, nh, nkv, d = len(tokens), c["hidden"], c["n_head"], c["n_kv_head"], c["head_dim"]
        x = self.embed(tokens)
        for l in range(c["n_layer"]):
            p = f"blk.{l}"
            hn = rmsnorm(x, self.vec(p + ".attn_norm.weight"), c["rms_eps"])
            q = self.mm(p + ".attn_q.weight", hn, nh * d).reshape(T, nh, d)
            k = self.mm(p + ".attn_k.weight", hn, nkv * d).reshape(T, nkv, d)
            v = self.mm(p + ".attn_v.weight", hn, nkv * d).reshape(T, nkv, d)
            q = rope_half_split(rmsnorm(q, self.vec(p + ".attn_q_norm.weight"), c["rms_eps"]), pos, c["rope_theta"])
            k = rope_half_split(rmsnorm(k, self.vec(p + ".attn_k_norm.weight"), c["rms_eps"]), pos, c["rope_theta"])
            self.k[l] = k if self.k[l] is None else np.concatenate([self.k[l], k], axis=0)
            self.v[l] = v if self.v[l] is None else np.concatenate([self.v[l], v], axis=0)
            att = gqa_attention(q, self.k[l], self.v[l], pos)
            x = (x + self.mm(p + ".attn_output.weight", att.reshape(T, nh * d), h)).astype(f32)
            hn = rmsnorm(x, self.vec(p + ".ffn_norm.weight"), c["rms_eps"])
            if c.get("n_expert"):
                x = (x + self.moe(l).forward(hn)).astype(f32)
                continue
            g = self.mm(p + ".ffn_gate.weight", hn, c["ffn"])
            u = self.mm(p + ".ffn_up.weight", hn, c["ffn"])
            x = (x + self.mm(p + ".ffn_down.weight", (silu(g) * u).astype(f32), h)).astype(f32)
        self.n_past = pos + T
        last = rmsnorm(x[-1:], self.vec("output_norm.weight"), c["rms_eps"])
        head = "output.weight" if "output.weight" in self.t else "token_embd.weight"
        return self.mm(head, last, c["vocab"])[0]


def greedy(logits: np.ndarray) -> int:
    """Last index of the maximum (Iterator::max_by keeps the last of equals, src/engine.rs:2371-2378)."""
    m = logits.max()
    return int(np.flatnonzero(logits == m)[-1])
