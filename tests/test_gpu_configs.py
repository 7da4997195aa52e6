"""The benchmark configurations at their own shapes, through the C ABI against the CPU oracle:
the DeepSeek-V3-shaped expert layer (h 7168, 2048 wide experts, 256 routed + 1 shared, top-8) in
IQ2_XXS and MXFP4, the Qwen3-30B-A3B-shaped layer with all 128 experts at batch 1 and 64, the
14336 x 4096 Q4_K product with 512 activation rows, and single-token steps of a decoder with
Qwen3-8B's layer and vocabulary sizes.  Experts hold distinct bytes (joshua_amd.synth.experts).
Tolerance: |gpu - ref| <= 1e-3 * max(|ref|, 1), the reference's own form (src/kquant_dot.rs:853)."""
import numpy as np
import pytest

import oracle
from oracle import qwen3 as oq
from oracle.moe import MoeOracle
from joshua_amd import capi, synth
from joshua_amd.synth.experts import RolledExperts
from joshua_amd.synth.model import qwen3_tensors

pytestmark = pytest.mark.gpu

TOL = 1e-3


def close(got, want, tol=TOL):
    err = np.abs(got - want) / np.maximum(np.abs(want), 1.0)
    return bool(np.all(err <= tol)), float(err.max())


def moe_layer(qtype, h, inter, n_expert, k_used, seed, shared, gating):
    """(device layer, oracle) over rolled expert stacks: the device holds the whole stack, the oracle builds
    the experts the router picks."""
    import torch
    dev = torch.device("cuda:0")
    stacks, weights = [], []
    for i, (rows, cols) in enumerate(((inter, h), (inter, h), (h, inter))):
        tmpl = synth.normal_quantized(qtype, seed + i, rows * cols, 0.02)
        st = RolledExperts(qtype, tmpl, n_expert)
        d = st.device_stack(torch, dev)
        weights.append(capi.Weight.upload_device(qtype, d.data_ptr(), d.numel(), n_expert * rows, cols))
        del d
        stacks.append(st)
    shared_o = shared_w = None
    if shared:
        sb = [synth.normal_quantized(qtype, seed + 10 + i, inter * h, 0.02) for i in range(3)]
        shared_o = (qtype, inter, sb[0], sb[1], sb[2])
        shared_w = (capi.Weight.upload(qtype, sb[0], inter, h), capi.Weight.upload(qtype, sb[1], inter, h),
                    capi.Weight.upload(qtype, sb[2], h, inter))
    router = synth.normal(seed + 20, (n_expert, h), 0.02)
    ora = MoeOracle(qtype, h, inter, n_expert, k_used, router, stacks[0], stacks[1], stacks[2], gating=gating,
                    norm_topk=True, shared=shared_o, avx2=oracle.have_avx2())
    cfg = capi.MoeConfig(n_expert, k_used, h, inter, 1 if gating == "sigmoid" else 0, 1, 0.0, 1, 1, 0.0, 0.0)
    layer = capi.Moe(cfg, router, weights[0], weights[1], weights[2], shared=shared_w)
    return layer, ora


@pytest.mark.parametrize("qtype", [capi.IQ2_XXS, capi.MXFP4])
def test_deepseek_v3_shaped_expert_layer(qtype):
    """h = 7168: IQ2_XXS rows of 1848 bytes (8-byte aligned only) and MXFP4 rows of 3808 bytes, 2048-wide
    experts, 256 routed experts + 1 shared, top-8, sigmoid gating (src/quantized_deepseek2.rs:520-559; expert
    slices src/quantized_deepseek4.rs:2306-2331).  One token (the decode path: the matrix-core expert kernels)
    and three tokens (27 pairs, still one group a pair)."""
    layer, ora = moe_layer(qtype, 7168, 2048, 256, 8, 500 + qtype, shared=True, gating="sigmoid")
    for tokens in (1, 3):
        x = synth.normal(520 + tokens, (tokens, 7168))
        ids, _ = layer.route(x)
        assert np.array_equal(ids, ora.route(x)[0])
        ok, e = close(layer.forward(x), ora.forward(x))
        assert ok, f"{capi.TYPE_NAMES[qtype]} tokens={tokens}: {e}"
    layer.close()


@pytest.mark.parametrize("qtype,tokens,expert_dot8,kernel", [
    (capi.IQ2_XXS, 150, True, "moe_expert_dot8"), (capi.MXFP4, 90, True, "moe_expert_dot8"),
    (capi.IQ2_XXS, 30, True, "moe_expert_dot8"), (capi.IQ2_XXS, 5, True, "moe_down_mfma"),
    (capi.IQ2_XXS, 150, False, "moe_gemm_i8_few"), (capi.MXFP4, 90, False, "moe_gemm_i8_few"),
    (capi.IQ2_XXS, 48, False, "moe_down_mfma")])
def test_deepseek_v3_shaped_expert_layer_over_a_prompt(monkeypatch, qtype, tokens, expert_dot8, kernel):
    """The same layer over a prompt, at the layer's own row lengths: gate and up of 7168 columns (28 super-blocks,
    224 units of 32: seven a lane), down of 2048.  150 tokens of IQ2_XXS (1200 routed pairs over 256 experts and the
    shared expert's 150), 90 of MXFP4 and 30 of IQ2_XXS (240 pairs, fewer than experts): bucketed by expert, an
    expert's rows decoded once into registers and its pairs streamed past them.  5 tokens: one group a pair.
    With that kernel switched off: the grouped int8 GEMM, and at 48 tokens still one group a pair (a pair's rows cost
    less to read again than an expert's to unpack for a tile of 32 rows)."""
    if expert_dot8:
        monkeypatch.delenv("JQ_MOE_EXPERT_DOT8_UPTO_PAIRS_PER_EXPERT", raising=False)
    else:
        monkeypatch.setenv("JQ_MOE_EXPERT_DOT8_UPTO_PAIRS_PER_EXPERT", "0")
    layer, ora = moe_layer(qtype, 7168, 2048, 256, 8, 500 + qtype, shared=True, gating="sigmoid")
    x = synth.normal(530 + tokens, (tokens, 7168))
    got = layer.forward(x)
    assert capi.last_kernel() == kernel
    ok, e = close(got, ora.forward(x))
    assert ok, f"{capi.TYPE_NAMES[qtype]} tokens={tokens}: {e}"
    layer.close()


@pytest.mark.parametrize("tokens", [1, 64])
def test_qwen3_30b_a3b_shaped_layer_with_all_128_experts(tokens):
    """h 2048, 128 experts of 768, top-8, Q4_K (src/quantized_qwen3_moe.rs:404-520): batch 1 takes the
    per-pair decode kernels, batch 64 the grouped kernel over the ~126 experts hit."""
    layer, ora = moe_layer(capi.Q4_K, 2048, 768, 128, 8, 540, shared=False, gating="softmax")
    x = synth.normal(541 + tokens, (tokens, 2048))
    ids, _ = layer.route(x)
    assert np.array_equal(ids, ora.route(x)[0])
    if tokens == 64:
        assert len(np.unique(ids)) > 100
    ok, e = close(layer.forward(x), ora.forward(x))
    assert ok, f"tokens={tokens}: {e}"
    layer.close()


def test_q4k_prefill_gemm_at_the_headline_shape():
    """Q4_K 14336 x 4096 with 512 activation rows: 256 tiles of 256 x 112 on the int8 matrix cores.  The oracle multiplies a
    sample of 1536 weight rows (the first and last 128-row tiles, and rows spread over the rest) by all 512
    activation rows; the device result is checked at those columns."""
    import torch
    n, k, m = 14336, 4096, 512
    blocks = synth.normal_quantized(capi.Q4_K, 102, n * k, 0.02)
    lhs = synth.normal(202, (m, k))
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    x = torch.from_numpy(lhs).cuda()
    y = torch.full((m, n), float("nan"), device="cuda")
    w.matmul_t_dev(m, x.data_ptr(), x.numel(), y.data_ptr(), y.numel(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert capi.last_kernel() == "q4k_gemm_i8"
    got = y.cpu().numpy()
    assert np.all(np.isfinite(got))
    rows = np.unique(np.concatenate([np.arange(128), np.arange(n - 128, n), np.arange(128, n - 128, 11)[:1280]]))
    sub = blocks.reshape(n, -1)[rows].reshape(-1)
    want = oracle.matmul_t(capi.Q4_K, (m, k, rows.size), lhs, sub, avx2=oracle.have_avx2())
    ok, e = close(got[:, rows], want)
    assert ok, e


def test_single_token_steps_at_qwen3_8b_layer_sizes():
    """Two layers with Qwen3-8B's widths (hidden 4096, 32 query / 8 KV heads of 128, feed-forward 12288,
    vocabulary 151936) in the Q4_K_M mix: an 8-token prefill, then teacher-forced single-token steps, which
    run the fused launches (residual + norm + q|k|v over 6144 rows, + gate|up + SwiGLU over 24576 rows) and
    the 151936-row Q6_K head at their real shapes."""
    cfg = dict(n_layer=2, hidden=4096, n_head=32, n_kv_head=8, head_dim=128, ffn=12288, vocab=151936, n_ctx=32,
               rms_eps=1e-6, rope_theta=1e6)
    tensors = {n: (qt, d) for n, qt, d in qwen3_tensors(cfg, 7, "q4_k_m")}
    c = capi.Qwen3Config(cfg["n_layer"], cfg["hidden"], cfg["n_head"], cfg["n_kv_head"], cfg["head_dim"], cfg["ffn"],
                         cfg["vocab"], cfg["n_ctx"], cfg["rms_eps"], cfg["rope_theta"])
    m = capi.Qwen3(c)
    for name, (qt, d) in tensors.items():
        m.set_tensor(name, qt, d)
    o = oq.Qwen3Oracle(cfg, tensors, avx2=oracle.have_avx2())
    prompt = [int(t) for t in synth.uniform_u32(31, 8, cfg["vocab"])]
    ok, e = close(m.forward(prompt, 0), o.forward(prompt, 0))
    assert ok, f"prefill: {e}"
    pos = len(prompt)
    for t in (5, 151935, 70000):
        got, ref = m.forward([t], pos), o.forward([t], pos)
        ok, e = close(got, ref)
        assert ok, f"pos {pos}: {e}"
        top2 = np.sort(ref)[-2:]
        if top2[1] - top2[0] > 2e-3 * max(abs(top2[1]), 1.0):
            assert m.greedy() == oq.greedy(ref)
        pos += 1
    m.close()


def test_mla_at_deepseek_v3_size():
    """Multi-head latent attention with DeepSeek-V3's dimensions (7168 wide, 128 heads, query rank 1536,
    latent 512 + 64 rope, YaRN factor 40; src/quantized_deepseek2.rs:357-499): a 200-token prefill in two
    chunks, then single-token steps, absorbed device form against the reference's unabsorbed form."""
    from tests.test_gpu_mla import build, cfg, close as mla_close
    c = cfg(n_embd=7168, n_head=128, q_lora_rank=1536, kv_lora_rank=512, qk_nope=128, qk_rope=64, v_head_dim=128,
            context_length=256, yarn=dict(factor=40.0, orig_context_length=4096, mscale_all_dim=1.0))
    ref, dev = build(c, qtype=capi.Q4_K, seed=900)
    x = synth.normal(901, (204, c["n_embd"]))
    assert mla_close(dev.forward(x[:128], 0), ref.forward(x[:128], 0))
    assert mla_close(dev.forward(x[128:200], 128), ref.forward(x[128:200], 128))
    for p in range(200, 204):
        assert mla_close(dev.forward(x[p:p + 1], p), ref.forward(x[p:p + 1], p))


def test_group_limited_routing_at_deepseek_v3_size():
    """256 experts in 8 groups, 4 groups kept, top-8, sigmoid scores with a selection bias, weights scaled
    by 2.5 (src/quantized_deepseek2.rs:527-597): ids and weights of 33 tokens against the oracle."""
    h, E = 7168, 256
    router = synth.normal(910, (E, h), 0.02)
    bias = synth.normal(911, (E,), 0.01)
    tiny = synth.normal_quantized(capi.Q8_0, 912, E * 32 * h, 0.02)      # experts are not exercised here
    down = synth.normal_quantized(capi.Q8_0, 913, E * h * 32, 0.02)
    ora = MoeOracle(capi.Q8_0, h, 32, E, 8, router, tiny, tiny, down, gating="sigmoid", norm_topk=True,
                    weights_scale=2.5, n_group=8, topk_group=4, router_bias=bias)
    cfg_ = capi.MoeConfig(E, 8, h, 32, 1, 1, 2.5, 8, 4, 0.0, 0.0)
    g = capi.Weight.upload(capi.Q8_0, tiny, E * 32, h)
    d = capi.Weight.upload(capi.Q8_0, down, E * h, 32)
    layer = capi.Moe(cfg_, router, g, g, d, router_bias=bias)
    x = synth.normal(914, (33, h))
    ids, w = layer.route(x)
    oid, ow = ora.route(x)
    assert np.array_equal(ids, oid)
    assert np.allclose(w, ow, rtol=2e-5, atol=1e-7)
    for t in range(33):                      # the picks really sit in 4 of the 8 groups
        assert len({int(e) // 32 for e in ids[t]}) <= 4
    layer.close()
