"""GGUF files on the device: a dense Qwen3 model written by our writer, loaded through the
joshua_npu_* plugin symbols and through jq_qwen3_load_gguf, against the numpy graph over the
oracle matmul on the same tensors; single tensors and expert stacks uploaded from the mapping."""
import numpy as np
import pytest

import oracle
from oracle import qwen3 as oq
from joshua_amd import capi, synth
from joshua_amd.synth import gguf as gw
from joshua_amd.synth.model import qwen3_tensor_plan, qwen3_tensors

pytestmark = pytest.mark.gpu

CFG = dict(n_layer=3, hidden=512, n_head=4, n_kv_head=2, head_dim=64, ffn=1024, vocab=768, n_ctx=40,
           rms_eps=1e-6, rope_theta=1e6)


def close(got, ref, tol=1e-3):
    return bool(np.all(np.abs(got - ref) <= tol * np.maximum(np.abs(ref), 1.0)))


def write_model(path, cfg, seed, mix="q4_k_m", drop=(), **kw):
    tensors = {n: (qt, d) for n, qt, d in qwen3_tensors(cfg, seed, mix)}
    items = [(n, qt, d) for n, (qt, d) in tensors.items() if n not in drop]
    gw.write_qwen3(str(path), cfg, items, qwen3_tensor_plan(cfg, mix), **kw)
    return tensors


def test_plugin_serves_a_gguf_model(tmp_path):
    path = tmp_path / "m.gguf"
    tensors = write_model(path, CFG, 41)
    o = oq.Qwen3Oracle(CFG, tensors, avx2=oracle.have_avx2())
    p = capi.NpuPlugin(str(path), CFG["n_ctx"])
    assert p.rc == 0 and p.vocab == CFG["vocab"], capi.last_error()
    prompt = [3, 700, 41, 41, 256, 9, 88, 511, 2, 640, 77]
    rc, got = p.forward(prompt, 0)
    assert rc == 0 and close(got, o.forward(prompt, 0))
    pos = len(prompt)
    for t in [5, 123, 767]:
        rc, got = p.forward([t], pos)
        assert rc == 0 and close(got, o.forward([t], pos))
        pos += 1
    # the position contract: pos must be the number of tokens fed so far; the context is n_ctx tokens
    assert p.forward([1], pos + 1)[0] == -3 and p.forward([1], 0)[0] == -3
    assert p.forward([1] * (CFG["n_ctx"] - pos + 1), pos)[0] == -4
    assert p.forward([CFG["vocab"]], pos)[0] == -5 and "out of range" in capi.last_error()
    rc, again = p.forward([9], pos)          # the refused calls fed nothing
    assert rc == 0 and close(again, o.forward([9], pos))
    # reset, then the same prompt gives the same logits
    assert p.reset() == 0
    rc, second = p.forward(prompt, 0)
    o2 = oq.Qwen3Oracle(CFG, tensors, avx2=oracle.have_avx2())
    assert rc == 0 and close(second, o2.forward(prompt, 0))
    p.close()


def test_tied_embeddings_and_metadata_fallbacks(tmp_path):
    """No output.weight: the embedding matrix is the output head (reference:
    src/quantized_qwen3_moe.rs:739-743).  No attention.key_length: head_dim = embedding_length /
    head_count (:105); no feed_forward_length: read off blk.0.ffn_gate; other alignment."""
    cfg = dict(CFG, head_dim=128, n_ctx=24)          # 512 / 4 heads
    path = tmp_path / "tied.gguf"
    tensors = write_model(path, cfg, 43, mix="q4_k", drop=("output.weight",), with_key_length=False, with_ffn=False,
                          alignment=64)
    tied = dict(tensors, **{"output.weight": tensors["token_embd.weight"]})
    o = oq.Qwen3Oracle(cfg, tied, avx2=oracle.have_avx2())
    m = capi.Qwen3.from_gguf(str(path), cfg["n_ctx"])
    c = m.cfg
    assert (c.n_layer, c.hidden, c.n_head, c.n_kv_head, c.head_dim, c.ffn, c.vocab, c.n_ctx) == \
        (3, 512, 4, 2, 128, 1024, 768, 24)
    assert c.rms_eps == np.float32(1e-6) and c.rope_theta == np.float32(1e6)
    toks = [11, 12, 700, 5]
    assert close(m.forward(toks, 0), o.forward(toks, 0))
    assert close(m.forward([8], 4), o.forward([8], 4))
    m.close()
    # n_ctx = 0 takes the file's context_length
    m = capi.Qwen3.from_gguf(str(path), 0)
    assert m.cfg.n_ctx == 24
    m.close()


def test_load_failures_name_the_problem(tmp_path):
    plan = qwen3_tensor_plan(CFG)
    tensors = {n: (qt, d) for n, qt, d in qwen3_tensors(CFG, 44)}

    def attempt(name, items, md=None, expect=""):
        path = str(tmp_path / name)
        shapes = {n: ([r] if k == 0 else [r, k]) for n, _, r, k in plan}
        gw.write_gguf(path, md or gw.qwen3_metadata(CFG), [(n, qt, shapes.get(n, sh), d) for n, qt, sh, d in items])
        p = capi.NpuPlugin(path, 16)
        assert p.rc == -2 and expect in capi.last_error(), capi.last_error()

    full = [(n, qt, None, d) for n, (qt, d) in tensors.items()]
    attempt("missing.gguf", [t for t in full if t[0] != "blk.1.ffn_up.weight"], expect="missing tensor `blk.1.ffn_up.weight`")
    f16 = [(n, 1, None, np.zeros(CFG["hidden"] * CFG["hidden"], np.float16)) if n == "blk.0.attn_q.weight" else (n, qt, s, d)
           for n, qt, s, d in full]
    attempt("f16.gguf", f16, expect="unsupported tensor type id 1")
    bad_head = gw.qwen3_metadata(dict(CFG, n_kv_head=3))
    attempt("heads.gguf", full, md=bad_head, expect="must be a multiple of head_count_kv")
    wrong = gw.qwen3_metadata(dict(CFG, hidden=768))
    attempt("shape.gguf", full, md=wrong, expect="does not have the shape")


def test_upload_from_the_mapping(tmp_path):
    """One matrix, and a stack of experts as one weight whose slices are views
    (reference: src/mmap_tensor.rs:520-565, src/quantized_qwen3_moe.rs:596-631)."""
    n, k, E = 48, 512, 5
    mat = synth.normal_quantized(capi.Q6_K, 5, n * k, 0.05)
    stack = synth.normal_quantized(capi.MXFP4, 6, E * n * k, 0.05)
    path = str(tmp_path / "w.gguf")
    gw.write_gguf(path, {}, [("a.weight", capi.Q6_K, [n, k], mat), ("blk.0.ffn_gate_exps.weight", capi.MXFP4, [E, n, k], stack),
                             ("v", 0, [k], np.ones(k, np.float32))])
    g = capi.Gguf.open(path)
    x = synth.normal(7, (3, k))
    w = g.upload("a.weight")
    assert (w.dtype, w.n, w.k) == (capi.Q6_K, n, k)
    assert close(w.matmul_t(3, x), oracle.matmul_t(capi.Q6_K, (3, k, n), x, mat))
    s = g.upload("blk.0.ffn_gate_exps.weight")
    assert (s.dtype, s.n, s.k) == (capi.MXFP4, E * n, k)
    per = s.nbytes // E
    for e in (0, 3, 4):
        got = s.view(e * per, n, k).matmul_t(3, x)
        assert close(got, oracle.matmul_t(capi.MXFP4, (3, k, n), x, stack[e * per:(e + 1) * per]))
    with pytest.raises(capi.JoshuaHipError, match="a matrix needs 2"):
        g.upload("v")
    with pytest.raises(capi.JoshuaHipError, match="no tensor"):
        g.upload("absent")
    g.close()
    assert close(w.matmul_t(3, x), oracle.matmul_t(capi.Q6_K, (3, k, n), x, mat))     # the copy in HBM outlives the file


def test_model_file_with_the_other_block_formats(tmp_path):
    """A model whose matrices use Q5_K, Q5_0, Q5_1, Q4_0, Q4_1 and Q3_K beside Q4_K and Q6_K, as the
    K-quant mixes other than Q4_K_M hold."""
    plan = qwen3_tensor_plan(CFG)
    shapes = {n: (r, k) for n, _, r, k in plan}
    tensors = {n: (qt, d) for n, qt, d in qwen3_tensors(CFG, 47)}
    swap = {"attn_q": capi.Q5_K, "attn_k": capi.Q5_0, "attn_output": capi.Q5_1, "ffn_gate": capi.Q4_1, "ffn_up": capi.Q3_K,
            "ffn_down": capi.Q5_K}
    for name in list(tensors):
        role = name.split(".")[2] if name.startswith("blk.") else name.split(".")[0]
        qt = swap.get(role, capi.Q4_0 if role == "token_embd" else None)
        if qt is not None:
            r, k = shapes[name]
            tensors[name] = (qt, synth.random_blocks(qt, 48 + len(name), r * k))
    path = str(tmp_path / "mixed.gguf")
    gw.write_qwen3(path, CFG, [(n, qt, d) for n, (qt, d) in tensors.items()], plan)
    o = oq.Qwen3Oracle(CFG, tensors, avx2=oracle.have_avx2())
    p = capi.NpuPlugin(path, CFG["n_ctx"])
    assert p.rc == 0, capi.last_error()
    prompt = [3, 700, 41, 41, 256, 9, 88]
    rc, got = p.forward(prompt, 0)
    assert rc == 0 and close(got, o.forward(prompt, 0))
    for i, t in enumerate([5, 123]):
        rc, got = p.forward([t], len(prompt) + i)
        assert rc == 0 and close(got, o.forward([t], len(prompt) + i))
    p.close()
