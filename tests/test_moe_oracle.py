"""Invariants the reference's own MoE unit tests check, on the CPU oracle
(reference: src/quantized_qwen3_moe.rs:897-928, src/quantized_deepseek2.rs:1259-1310)."""
import numpy as np
import pytest

import oracle
from oracle.moe import MoeOracle
from joshua_amd import synth


def tiny(qtype=oracle.Q8_0, h=256, inter=64, E=8, k=2, seed=1, **kw):
    rw = synth.normal(seed, (E, h))
    gate = synth.normal_quantized(qtype, seed + 1, E * inter * h, 0.05)
    up = synth.normal_quantized(qtype, seed + 2, E * inter * h, 0.05)
    down = synth.normal_quantized(qtype, seed + 3, E * h * inter, 0.05)
    return MoeOracle(qtype, h, inter, E, k, rw, gate, up, down, **kw)


def test_routing_weights_sum_to_one_under_norm():
    moe = tiny(norm_topk=True)
    _, w = moe.route(synth.normal(9, (3, 256)))
    assert np.all(np.abs(w.sum(axis=1) - 1.0) < 1e-4)


def test_routing_picks_descending_top_k_of_softmax():
    moe = tiny(norm_topk=False, k=3)
    x = synth.normal(10, (5, 256))
    idx, w = moe.route(x)
    logits = x @ moe.router_w.T
    p = np.exp(logits - logits.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    for t in range(5):
        order = np.argsort(-p[t])[:3]
        assert list(idx[t]) == list(order)
        assert np.allclose(w[t], p[t][order], rtol=1e-5)


def test_prefill_bucketing_matches_decode_path():
    moe = tiny()
    row = synth.normal(11, (1, 256))
    two = np.concatenate([row, row], axis=0)
    out2 = moe.forward(two)
    out1 = moe.forward(row)
    assert np.all(np.abs(out2[1] - out1[0]) < 1e-4)
    assert np.all(np.abs(out2[0] - out1[0]) < 1e-4)


def test_group_limit_keeps_only_the_best_groups():
    moe = tiny(E=16, k=4, gating="sigmoid", n_group=4, topk_group=2, norm_topk=True, weights_scale=2.5,
               router_bias=np.linspace(-0.1, 0.1, 16, dtype=np.float32))
    x = synth.normal(12, (6, 256))
    idx, w = moe.route(x)
    probs = 1.0 / (1.0 + np.exp(-(x @ moe.router_w.T)))
    sel = probs + moe.bias
    for t in range(6):
        score = np.sort(sel[t].reshape(4, 4), axis=1)[:, -2:].sum(1)
        kept = set(np.argsort(-score)[:2])
        assert {int(e) // 4 for e in idx[t]} <= kept
        assert abs(w[t].sum() - 2.5) < 1e-4          # normalised, then scaled
        # weights come from the unbiased probabilities
        assert np.allclose(w[t] / 2.5, probs[t][idx[t]] / probs[t][idx[t]].sum(), rtol=1e-4)


def test_shared_expert_is_added_for_every_token():
    base = tiny(seed=5)
    sg = synth.normal_quantized(oracle.Q8_0, 50, 96 * 256, 0.05)
    su = synth.normal_quantized(oracle.Q8_0, 51, 96 * 256, 0.05)
    sd = synth.normal_quantized(oracle.Q8_0, 52, 256 * 96, 0.05)
    withs = tiny(seed=5, shared=(oracle.Q8_0, 96, sg, su, sd))
    x = synth.normal(13, (2, 256))
    diff = withs.forward(x) - base.forward(x)
    assert np.allclose(diff, withs.shared_mlp(x), atol=1e-5)


def test_silu_by_value():
    """x / (1 + exp(-x)) at points whose values are known: fails for sigmoid alone, for x * sigmoid(-x),
    for gelu."""
    from oracle.moe import silu
    got = silu(np.array([0.0, 1.0, -1.0, 20.0, -20.0], np.float32))
    assert got[0] == 0.0
    assert got[1] == pytest.approx(0.7310585786, rel=1e-6)
    assert got[2] == pytest.approx(-0.2689414214, rel=1e-6)
    assert got[3] == pytest.approx(20.0, rel=1e-6) and abs(got[4]) < 1e-7


def test_expert_mlp_is_down_of_silu_gate_times_up():
    """One expert's MLP against float64 over the decoded weights, down (silu(gate x) * (up x))
    (src/quantized_qwen3_moe.rs:397-401).  gate and up hold different bytes, so applying the activation to
    up instead of gate, or dropping it, fails; so does reading another expert's slice."""
    from scipy.special import expit
    h, inter, E = 256, 64, 4
    moe = tiny(h=h, inter=inter, E=E, seed=21)
    x = synth.normal(22, (3, h))
    for e in (0, 3):
        def dec(blocks, n, k):
            per = blocks.size // E
            return oracle.dequantize(moe.qtype, blocks[e * per:(e + 1) * per]).reshape(n, k).astype(np.float64)
        g, u = x.astype(np.float64) @ dec(moe.gate, inter, h).T, x.astype(np.float64) @ dec(moe.up, inter, h).T
        want = (g * expit(g) * u) @ dec(moe.down, h, inter).T
        got = moe.mlp(e, x)
        assert np.abs(got - want).max() <= 1e-4 * max(np.abs(want).max(), 1.0)
        swapped = (u * expit(u) * g) @ dec(moe.down, h, inter).T
        assert np.abs(swapped - want).max() > 1e-2 * np.abs(want).max()      # the check can tell them apart


def test_decode_dispatch_is_the_weighted_sum_of_the_selected_experts():
    """y = sum_s w_s mlp(e_s, x) over the router's k picks (src/quantized_qwen3_moe.rs:504-520)."""
    moe = tiny(E=8, k=3, seed=31)
    x = synth.normal(32, (1, 256))
    idx, w = moe.route(x)
    want = sum(float(w[0, s]) * moe.mlp(int(idx[0, s]), x).astype(np.float64) for s in range(3))
    assert np.allclose(moe.forward(x), want, rtol=1e-5, atol=1e-6)
