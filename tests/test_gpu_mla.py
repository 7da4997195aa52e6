"""Multi-head latent attention on the GPU (absorbed form, latent cache) against the numpy
restatement of the reference's unabsorbed Attention::forward (oracle/mla.py), through the C ABI.
Bound: |gpu - ref| <= 1e-3 * max(|ref|, 1) on the block's output."""
import numpy as np
import pytest

import oracle
from oracle import mla as om
from joshua_amd import capi, synth
from joshua_amd.synth import normal

pytestmark = pytest.mark.gpu


def close(got, want, tol=1e-3):
    """Element by element, the bound of the other parity tests."""
    return bool(np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1.0)))


def quantized(qtype, seed, n, k, scale=1.0):
    """Random weights as blocks of `qtype` (n rows of k)."""
    w = (normal(seed, (n, k)) * np.float32(scale)).astype(np.float32)
    return synth.quantize(qtype, w)


def build(c, qtype=capi.Q8_0, seed=100, dense_kv_b=False):
    """Oracle tensors and the device object over the same blocks."""
    nh, lkv, npe, r, vh, h = c["n_head"], c["kv_lora_rank"], c["qk_nope"], c["qk_rope"], c["v_head_dim"], c["n_embd"]
    qd = npe + r
    shapes = {"kv_a_mqa": (lkv + r, h), "kv_b": (nh * (npe + vh), lkv), "o": (h, nh * vh)}
    if c["q_lora_rank"]:
        shapes.update(q_a=(c["q_lora_rank"], h), q_b=(nh * qd, c["q_lora_rank"]))
    else:
        shapes["q"] = (nh * qd, h)
    t, w = {}, {}
    for i, (name, (n, k)) in enumerate(sorted(shapes.items())):
        if name == "kv_b" and dense_kv_b:
            t[name] = (0, (normal(seed + i, (n, k)) / np.float32(np.sqrt(k))).astype(np.float32))
            continue
        blocks = quantized(qtype, seed + i, n, k, 1.0 / np.sqrt(k))
        t[name] = (qtype, blocks)
        w[name] = capi.Weight.upload(qtype, blocks, n, k)
    t["kv_a_norm"] = (1.0 + 0.1 * normal(seed + 20, (lkv,))).astype(np.float32)
    if c["q_lora_rank"]:
        t["q_a_norm"] = (1.0 + 0.1 * normal(seed + 21, (c["q_lora_rank"],))).astype(np.float32)
    y = c.get("yarn")
    cfg = capi.MlaConfig(n_embd=h, n_head=nh, q_lora_rank=c["q_lora_rank"], kv_lora_rank=lkv, qk_nope_head_dim=npe,
                         qk_rope_head_dim=r, v_head_dim=vh, n_ctx=c["context_length"], rms_eps=c["rms_eps"],
                         rope_theta=c["rope_theta"], yarn_factor=y["factor"] if y else 0.0,
                         yarn_mscale_all_dim=y["mscale_all_dim"] if y else 0.0,
                         yarn_orig_context_length=y["orig_context_length"] if y else 0)
    q = (w["q_a"], t["q_a_norm"], w["q_b"]) if c["q_lora_rank"] else w["q"]
    dev = capi.Mla(cfg, q, w["kv_a_mqa"], t["kv_a_norm"], t["kv_b"][1] if dense_kv_b else w["kv_b"], w["o"])
    return om.MlaOracle(c, t), dev


def cfg(**over):
    c = dict(n_embd=256, n_head=4, q_lora_rank=0, kv_lora_rank=64, qk_nope=32, qk_rope=16, v_head_dim=32,
             rms_eps=1e-6, rope_theta=10000.0, context_length=128, yarn=None)
    c.update(over)
    return c


CASES = {
    "plain_q": cfg(),
    "lora_q": cfg(q_lora_rank=96),
    "yarn": cfg(q_lora_rank=64, yarn=dict(factor=40.0, orig_context_length=64, mscale_all_dim=1.0)),
    "odd_dims": cfg(n_head=3, kv_lora_rank=96, qk_nope=24, qk_rope=6, v_head_dim=32),   # ragged latent, one head a workgroup
    "two_heads": cfg(n_head=6, kv_lora_rank=160, qk_nope=64, qk_rope=32, v_head_dim=48),
    "v3_heads": cfg(n_embd=512, n_head=16, q_lora_rank=128, kv_lora_rank=512, qk_nope=128, qk_rope=64, v_head_dim=128,
                    context_length=160),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_prefill_then_decode_matches_the_reference_graph(name):
    c = CASES[name]
    ref, dev = build(c)
    x = normal(7, (21, c["n_embd"]))
    assert close(dev.forward(x[:17], 0), ref.forward(x[:17], 0))   # prefill (causal mask)
    assert dev.cached_tokens == 17
    for p in range(17, 21):                                         # token by token
        assert close(dev.forward(x[p:p + 1], p), ref.forward(x[p:p + 1], p))
    assert dev.cached_tokens == 21


def test_prefill_equals_incremental():
    """src/quantized_deepseek2.rs:1213-1256 on the device, with its bound on the outputs."""
    c = CASES["lora_q"]
    _, a = build(c)
    _, b = build(c)
    x = normal(8, (9, c["n_embd"]))
    whole = a.forward(x, 0)
    steps = np.concatenate([b.forward(x[i:i + 1], i) for i in range(9)])
    assert np.abs(whole - steps).max() < 1e-5 * max(1.0, np.abs(whole).max())


def test_long_context_is_split_over_workgroups():
    """Enough cached tokens that a decode step splits its context (32 tokens a split or more) and the
    partial softmax results merge; scores spread over a wide range."""
    c = cfg(n_head=8, kv_lora_rank=128, qk_nope=32, qk_rope=32, v_head_dim=64, context_length=700)
    ref, dev = build(c, seed=300)
    x = normal(9, (650, c["n_embd"])) * np.float32(3.0)
    assert close(dev.forward(x[:600], 0), ref.forward(x[:600], 0))
    for p in (600, 601):
        assert close(dev.forward(x[p:p + 1], p), ref.forward(x[p:p + 1], p))
    assert close(dev.forward(x[602:650], 602), ref.forward(x[602:650], 602))  # a second prefill chunk at an offset


def test_matrix_core_attention_for_the_deepseek_geometry():
    """512 latent + 64 rope elements and heads in groups of 32 run on the f32 matrix cores: tiles of 32
    tokens, several tiles a workgroup in the prefill, several context splits in the decode steps, a
    ragged last tile."""
    c = cfg(n_embd=256, n_head=64, kv_lora_rank=512, qk_nope=32, qk_rope=64, v_head_dim=32, context_length=260)
    ref, dev = build(c, seed=700)
    x = normal(14, (250, c["n_embd"])) * np.float32(2.0)
    assert close(dev.forward(x[:150], 0), ref.forward(x[:150], 0))
    for p in (150, 151, 152):
        assert close(dev.forward(x[p:p + 1], p), ref.forward(x[p:p + 1], p))
    assert close(dev.forward(x[153:250], 153), ref.forward(x[153:250], 153))


def test_dense_kv_b_and_other_formats():
    c = cfg(kv_lora_rank=256, n_embd=256, v_head_dim=64)
    for qtype in (capi.Q4_K, capi.Q6_K):
        ref, dev = build(c, qtype=qtype, seed=400 + qtype)
        x = normal(10, (5, c["n_embd"]))
        assert close(dev.forward(x, 0), ref.forward(x, 0))
    ref, dev = build(cfg(), dense_kv_b=True, seed=500)
    x = normal(11, (6, 256))
    assert close(dev.forward(x, 0), ref.forward(x, 0))
    # the latent width of the reference's own tiny attention (src/quantized_deepseek2.rs:1102-1125)
    c = cfg(n_embd=32, n_head=2, kv_lora_rank=6, qk_nope=4, qk_rope=4, v_head_dim=16)
    ref, dev = build(c, dense_kv_b=True, seed=600)
    x = normal(12, (4, 32))
    assert close(dev.forward(x[:3], 0), ref.forward(x[:3], 0))
    assert close(dev.forward(x[3:], 3), ref.forward(x[3:], 3))


def test_reset_and_position_checks():
    c = CASES["plain_q"]
    ref, dev = build(c)
    x = normal(12, (4, c["n_embd"]))
    first = dev.forward(x, 0)
    with pytest.raises(capi.JoshuaHipError, match="tokens are cached"):
        dev.forward(x[:1], 0)
    dev.reset()
    assert dev.cached_tokens == 0
    assert np.array_equal(dev.forward(x, 0), first)
    with pytest.raises(capi.JoshuaHipError, match="exceed the context"):
        dev.forward(normal(13, (c["context_length"], c["n_embd"])), 4)


def test_create_rejects_wrong_shapes():
    c = CASES["plain_q"]
    blocks = quantized(capi.Q8_0, 1, 64, 256)
    w = capi.Weight.upload(capi.Q8_0, blocks, 64, 256)
    mc = capi.MlaConfig(n_embd=256, n_head=4, q_lora_rank=0, kv_lora_rank=64, qk_nope_head_dim=32, qk_rope_head_dim=16,
                        v_head_dim=32, n_ctx=16, rms_eps=1e-6, rope_theta=1e4)
    with pytest.raises(capi.JoshuaHipError, match="attn_q is"):
        capi.Mla(mc, w, w, np.ones(64, np.float32), w, w)
