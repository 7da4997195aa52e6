"""A Qwen3-MoE model (general.architecture = qwen3moe) behind the joshua_npu_* plugin symbols and
jq_qwen3_*: a small synthetic GGUF with stacked expert tensors, against the numpy graph over the oracle
matmul and the oracle's expert block on the same tensors (reference: src/quantized_qwen3_moe.rs:100-147
configuration, :556-675 expert tensors, :700-830 graph)."""
import numpy as np
import pytest

import oracle
from oracle import qwen3 as oq
from joshua_amd import capi, synth
from joshua_amd.synth import gguf as gw
from joshua_amd.synth.model import gguf_dims, qwen3_tensor_plan, qwen3_tensors

pytestmark = pytest.mark.gpu

CFG = dict(n_layer=3, hidden=512, n_head=4, n_kv_head=2, head_dim=64, ffn=0, vocab=768, n_ctx=48,
           rms_eps=1e-6, rope_theta=1e6, n_expert=8, n_expert_used=2, expert_ffn=256)


def close(got, ref, tol=1e-3):
    return bool(np.all(np.abs(got - ref) <= tol * np.maximum(np.abs(ref), 1.0)))


def write_model(path, cfg, seed, mix="q4_k_m", **kw):
    tensors = {n: (qt, d) for n, qt, d in qwen3_tensors(cfg, seed, mix)}
    gw.write_qwen3(str(path), cfg, [(n, qt, d) for n, (qt, d) in tensors.items()], qwen3_tensor_plan(cfg, mix), **kw)
    return tensors


def test_plugin_serves_a_qwen3moe_gguf(tmp_path):
    """Teacher-forced logits of a prompt and of single-token steps; a prompt fed at once and fed token by
    token end in the same logits."""
    path = tmp_path / "moe.gguf"
    tensors = write_model(path, CFG, 61)
    o = oq.Qwen3Oracle(CFG, tensors, avx2=oracle.have_avx2())
    p = capi.NpuPlugin(str(path), CFG["n_ctx"])
    assert p.rc == 0 and p.vocab == CFG["vocab"], capi.last_error()
    prompt = [3, 700, 41, 41, 256, 9, 88, 511, 2, 640, 77]
    rc, got = p.forward(prompt, 0)
    assert rc == 0 and close(got, o.forward(prompt, 0)), capi.last_error()
    pos = len(prompt)
    for t in [5, 123, 767]:
        rc, got = p.forward([t], pos)
        assert rc == 0 and close(got, o.forward([t], pos))
        pos += 1
    last = got
    assert p.forward([1], pos + 1)[0] == -3            # the position contract holds as for the dense model
    # incremental: the same 14 tokens one at a time
    assert p.reset() == 0
    for i, t in enumerate(prompt + [5, 123, 767]):
        rc, got = p.forward([t], i)
        assert rc == 0
    assert close(got, last, 2e-3)
    p.close()


def test_single_token_steps_with_2048_wide_rows(tmp_path):
    """hidden = 2048 (Qwen3-30B-A3B's): a single-token step runs the attention block's norm inside the q|k launch and the
    expert block's norm inside the router launch; steps of several tokens run them as launches of their own."""
    cfg = dict(CFG, n_layer=3, hidden=2048, n_head=4, n_kv_head=2, head_dim=128, vocab=512, n_ctx=40, n_expert=16,
               n_expert_used=4, expert_ffn=256)
    path = tmp_path / "moe2048.gguf"
    tensors = write_model(path, cfg, 67)
    o = oq.Qwen3Oracle(cfg, tensors, avx2=oracle.have_avx2())
    p = capi.NpuPlugin(str(path), cfg["n_ctx"])
    assert p.rc == 0, capi.last_error()
    prompt = [3, 500, 41, 41, 256, 9, 88]
    rc, got = p.forward(prompt, 0)
    assert rc == 0 and close(got, o.forward(prompt, 0)), capi.last_error()
    pos = len(prompt)
    for step in ([5], [123], [7, 8, 9], [511], [0]):
        rc, got = p.forward(step, pos)
        assert rc == 0 and close(got, o.forward(step, pos)), f"pos {pos}"
        pos += len(step)
    p.close()


def test_configuration_of_a_qwen3moe_file(tmp_path):
    """The expert keys land in the configuration; attention.norm_topk_prob defaults to true when the file
    leaves it out and is honoured when false (reference: src/quantized_qwen3_moe.rs:119-134)."""
    cfg = dict(CFG, n_layer=1, n_expert=4, n_expert_used=3, n_ctx=16)
    toks = [11, 12, 700, 5]
    for with_norm, expect in ((None, 1), (True, 1), (False, 0)):
        path = tmp_path / f"n{with_norm}.gguf"
        tensors = write_model(path, cfg, 62, mix="q4_k", with_norm_topk=with_norm)
        m = capi.Qwen3.from_gguf(str(path), 0)
        c = m.cfg
        assert (c.n_expert, c.n_expert_used, c.expert_ffn, c.norm_topk_prob, c.ffn, c.n_ctx) == (4, 3, 256, expect, 0, 16)
        o = oq.Qwen3Oracle(dict(cfg, norm_topk_prob=bool(expect)), tensors, avx2=oracle.have_avx2())
        assert close(m.forward(toks, 0), o.forward(toks, 0))
        assert close(m.forward([9], 4), o.forward([9], 4))
        m.close()
    # the two routings differ on this input, so the flag is seen to matter
    a = oq.Qwen3Oracle(dict(cfg, norm_topk_prob=True), tensors).forward(toks, 0)
    b = oq.Qwen3Oracle(dict(cfg, norm_topk_prob=False), tensors).forward(toks, 0)
    assert not close(a, b)


def test_tensor_by_tensor_with_an_f16_router_and_a_replaced_expert_stack():
    """jq_qwen3_create + jq_qwen3_set_tensor: the router as F16, one layer's gate and up stacks in Q8_0
    beside Q4_K; replacing a layer's expert tensor after a step rebuilds that layer."""
    cfg = dict(CFG, n_layer=2, n_ctx=16)
    tensors = {n: (qt, d) for n, qt, d in qwen3_tensors(cfg, 63, "q4_k")}
    E, h, eff = cfg["n_expert"], cfg["hidden"], cfg["expert_ffn"]
    tensors["blk.1.ffn_gate_exps.weight"] = (capi.Q8_0, synth.normal_quantized(capi.Q8_0, 64, E * eff * h, h ** -0.5))
    tensors["blk.1.ffn_up_exps.weight"] = (capi.Q8_0, synth.normal_quantized(capi.Q8_0, 65, E * eff * h, h ** -0.5))
    r16 = np.asarray(tensors["blk.0.ffn_gate_inp.weight"][1], np.float32).astype(np.float16)
    as_oracle = dict(tensors, **{"blk.0.ffn_gate_inp.weight": (0, r16.astype(np.float32))})
    c = capi.Qwen3Config(cfg["n_layer"], h, cfg["n_head"], cfg["n_kv_head"], cfg["head_dim"], 0, cfg["vocab"], cfg["n_ctx"],
                         cfg["rms_eps"], cfg["rope_theta"], E, cfg["n_expert_used"], eff, 1)
    m = capi.Qwen3(c)
    for name, (qt, data) in tensors.items():
        if name == "blk.0.ffn_gate_inp.weight":
            m.set_tensor(name, 1, r16)
        else:
            m.set_tensor(name, qt, data)
    o = oq.Qwen3Oracle(cfg, as_oracle, avx2=oracle.have_avx2())
    toks = [1, 2, 3, 400, 5]
    assert close(m.forward(toks, 0), o.forward(toks, 0))
    assert close(m.forward([6], 5), o.forward([6], 5))
    new_down = synth.normal_quantized(capi.Q4_K, 66, E * h * eff, eff ** -0.5)
    m.set_tensor("blk.0.ffn_down_exps.weight", capi.Q4_K, new_down)
    o2 = oq.Qwen3Oracle(cfg, dict(as_oracle, **{"blk.0.ffn_down_exps.weight": (capi.Q4_K, new_down)}), avx2=oracle.have_avx2())
    m.reset()
    assert close(m.forward(toks, 0), o2.forward(toks, 0))
    with pytest.raises(capi.JoshuaHipError, match="must be F32 or F16"):
        m.set_tensor("blk.0.ffn_gate_inp.weight", 0, np.zeros(3, np.float32))
    m.close()
    bad = capi.Qwen3Config(1, 256, 2, 1, 64, 0, 256, 8, 1e-6, 1e4, 4, 5, 128, 1)
    with pytest.raises(capi.JoshuaHipError, match=r"expert_used_count 5 must be in 1..=expert_count 4"):
        capi.Qwen3(bad)


def test_load_failures_of_a_qwen3moe_file(tmp_path):
    cfg = dict(CFG, n_layer=1, n_ctx=16)
    plan = qwen3_tensor_plan(cfg, "q4_k")
    tensors = {n: (qt, d) for n, qt, d in qwen3_tensors(cfg, 67, "q4_k")}
    shapes = {n: gguf_dims(cfg, n, r, k) for n, _, r, k in plan}

    def attempt(name, items, md=None, expect=""):
        path = str(tmp_path / name)
        gw.write_gguf(path, md or gw.qwen3_metadata(cfg), [(n, qt, sh or shapes[n], d) for n, qt, sh, d in items])
        p = capi.NpuPlugin(path, 16)
        assert p.rc == -2 and expect in capi.last_error(), capi.last_error()

    full = [(n, qt, None, d) for n, (qt, d) in tensors.items()]
    attempt("no_router.gguf", [t for t in full if t[0] != "blk.0.ffn_gate_inp.weight"],
            expect="qwen3moe: missing tensor `blk.0.ffn_gate_inp.weight`")
    attempt("no_down.gguf", [t for t in full if t[0] != "blk.0.ffn_down_exps.weight"],
            expect="missing tensor `blk.0.ffn_down_exps.weight`")
    E, h, eff = cfg["n_expert"], cfg["hidden"], cfg["expert_ffn"]
    flat = [(n, qt, [E * eff, h] if n == "blk.0.ffn_up_exps.weight" else None, d) for n, qt, _, d in full]
    attempt("flat.gguf", flat, expect="expected expert tensor `blk.0.ffn_up_exps.weight` shaped [n_expert, out, in]")
    md = gw.qwen3_metadata(cfg)
    md.pop("qwen3moe.expert_used_count")
    attempt("nokey.gguf", full, md=md, expect="missing GGUF metadata key `qwen3moe.expert_used_count`")
    attempt("toomany.gguf", full, md=gw.qwen3_metadata(dict(cfg, n_expert_used=9)),
            expect="expert_used_count 9 must be in 1..=expert_count 8")
