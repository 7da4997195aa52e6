"""CPU restatement of the reference's mixture-of-experts blocks on top of the
oracle matmul.  TEST INFRASTRUCTURE (see oracle/__init__.py).

route / dispatch follow src/quantized_qwen3_moe.rs:412-528 and
src/quantized_deepseek2.rs:522-685; the f32 router matmul, softmax, sigmoid and
argsort there are third-party candle ops whose ulp-level behaviour and tie
order are not pinned by anything in the reference, so comparisons against this
file use the reference's own MoE tolerances (1e-4 abs on tiny layers) and a
relative bound on real shapes.
"""
from __future__ import annotations

import numpy as np

from . import matmul_t

F16_EPS_CLAMP = np.float32(6.103515625e-5)  # src/quantized_qwen3_moe.rs:432


def silu(x):
    x = x.astype(np.float32)
    return (x / (np.float32(1) + np.exp(-x, dtype=np.float32))).astype(np.float32)


def topk_indices(v: np.ndarray, k: int) -> np.ndarray:
    """First k of a descending argsort; equal values ordered by index."""
    return np.argsort(-v, axis=-1, kind="stable")[..., :k]


class MoeOracle:
    def __init__(self, qtype, h, inter, n_expert, k_used, router_w, gate, up, down, *, gating="softmax",
                 norm_topk=True, weights_scale=0.0, n_group=1, topk_group=1, router_bias=None, shared=None,
                 avx2=False, swiglu_clamp=0.0, swiglu_clamp_shared=0.0, qtype_down=None):
        self.qtype, self.h, self.inter, self.E, self.k = qtype, h, inter, n_expert, k_used
        self.qtype_down = qtype if qtype_down is None else qtype_down   # ffn_down_exps may hold more bits
        self.router_w = np.asarray(router_w, np.float32)          # [E, h]
        self.gate, self.up, self.down = gate, up, down            # stacked block bytes
        self.gating, self.norm_topk, self.scale = gating, norm_topk, np.float32(weights_scale)
        self.n_group, self.topk_group = n_group, topk_group
        self.bias = None if router_bias is None else np.asarray(router_bias, np.float32)
        self.shared = shared                                      # (qtype, inter_s, gate, up, down) or None
        self.avx2 = avx2
        self.clamp, self.clamp_shared = np.float32(swiglu_clamp), np.float32(swiglu_clamp_shared)

    @staticmethod
    def clamped(g, u, c):
        """src/quantized_deepseek4.rs:445-462: gate to (-inf, c], up to [-c, c] when c > 0."""
        if c > 0:
            g, u = np.minimum(g, c), np.clip(u, -c, c)
        return g, u

    # -- routing (src/quantized_qwen3_moe.rs:424-436, src/quantized_deepseek2.rs:527-551) ----
    def route(self, x2: np.ndarray):
        logits = (x2.astype(np.float32) @ self.router_w.T).astype(np.float32)
        if self.gating == "sigmoid":
            probs = (np.float32(1) / (np.float32(1) + np.exp(-logits, dtype=np.float32))).astype(np.float32)
        else:
            e = np.exp(logits - logits.max(axis=-1, keepdims=True), dtype=np.float32)
            probs = (e / e.sum(axis=-1, keepdims=True, dtype=np.float32)).astype(np.float32)
        sel = probs if self.bias is None else (probs + self.bias[None, :]).astype(np.float32)
        sel = self.group_limit(sel)
        idx = topk_indices(sel, self.k)
        w = np.take_along_axis(probs, idx, axis=-1)
        if self.norm_topk:
            denom = np.maximum(w.sum(axis=-1, keepdims=True, dtype=np.float32), F16_EPS_CLAMP)
            w = (w / denom).astype(np.float32)
        if self.scale != 0.0 and self.scale != 1.0:
            w = (w * self.scale).astype(np.float32)
        return idx.astype(np.uint32), w.astype(np.float32)

    # -- src/quantized_deepseek2.rs:563-597 ---------------------------------------------------
    def group_limit(self, sel: np.ndarray) -> np.ndarray:
        if self.n_group <= 1:
            return sel
        t = sel.shape[0]
        per = self.E // self.n_group
        grouped = sel.reshape(t, self.n_group, per)
        if self.gating == "sigmoid":
            score = np.sort(grouped, axis=-1)[..., ::-1][..., :2].sum(axis=-1, dtype=np.float32)
        else:
            score = grouped.max(axis=-1)
        gidx = topk_indices(score, self.topk_group)
        mask = np.zeros((t, self.n_group), np.float32)
        np.put_along_axis(mask, gidx, np.float32(1), axis=-1)
        penalty = (np.repeat(mask, per, axis=1) * np.float32(1e30) + np.float32(-1e30)).astype(np.float32)
        return (sel + penalty).astype(np.float32)

    # -- experts ---------------------------------------------------------------------------------
    def _slice(self, blocks, e):
        per = blocks.size // self.E
        return blocks[e * per:(e + 1) * per]

    def mlp(self, e: int, x: np.ndarray) -> np.ndarray:
        """down(silu(gate x) * (up x)) (src/quantized_qwen3_moe.rs:397-401)."""
        m = x.shape[0]
        g = matmul_t(self.qtype, (m, self.h, self.inter), x, self._slice(self.gate, e), avx2=self.avx2)
        u = matmul_t(self.qtype, (m, self.h, self.inter), x, self._slice(self.up, e), avx2=self.avx2)
        g, u = self.clamped(g, u, self.clamp)
        hid = (silu(g) * u).astype(np.float32)
        return matmul_t(self.qtype_down, (m, self.inter, self.h), hid, self._slice(self.down, e), avx2=self.avx2).copy()

    def shared_mlp(self, x: np.ndarray) -> np.ndarray:
        qt, si, g, u, d = self.shared
        m = x.shape[0]
        gg = matmul_t(qt, (m, self.h, si), x, g, avx2=self.avx2)
        uu = matmul_t(qt, (m, self.h, si), x, u, avx2=self.avx2)
        gg, uu = self.clamped(gg, uu, self.clamp_shared)
        hid = (silu(gg) * uu).astype(np.float32)
        return matmul_t(qt, (m, si, self.h), hid, d, avx2=self.avx2).copy()

    def dispatch_decode(self, x2, idx, w):
        """src/quantized_qwen3_moe.rs:504-520: k expert MLPs over the one row, stack, scale, sum."""
        outs = np.stack([self.mlp(int(e), x2) for e in idx[0]], axis=0)       # [k, 1, h]
        return (outs * w.reshape(self.k, 1, 1)).sum(axis=0, dtype=np.float32)   # [1, h]

    def dispatch_bucketed(self, x2, idx, w):
        """src/quantized_qwen3_moe.rs:444-498: bucket (token, weight) by expert, batched MLP, index_add."""
        t = x2.shape[0]
        y = np.zeros((t, self.h), np.float32)
        for e in range(self.E):
            tok, slot = np.nonzero(idx == e)
            if tok.size == 0:
                continue
            out = self.mlp(e, np.ascontiguousarray(x2[tok]))
            np.add.at(y, tok, (out * w[tok, slot][:, None]).astype(np.float32))
        return y

    def forward(self, x2: np.ndarray, force_bucketed: bool = False) -> np.ndarray:
        x2 = np.ascontiguousarray(x2, np.float32)
        idx, w = self.route(x2)
        if x2.shape[0] == 1 and not force_bucketed:
            y = self.dispatch_decode(x2, idx, w)
        else:
            y = self.dispatch_bucketed(x2, idx, w)
        if self.shared is not None:
            y = (y + self.shared_mlp(x2)).astype(np.float32)
        return y
