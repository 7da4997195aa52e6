"""End-to-end dense Qwen3 decode on the device against the numpy graph over the
oracle matmul: teacher-forced logits after a prefill and on every decode step,
the KV-cache position contract, and the greedy pick's tie order."""
import numpy as np
import pytest

import oracle
from oracle import qwen3 as oq
from joshua_amd import capi
from joshua_amd.synth.model import qwen3_tensors

pytestmark = pytest.mark.gpu

CFG = dict(n_layer=3, hidden=512, n_head=4, n_kv_head=2, head_dim=64, ffn=1024, vocab=768, n_ctx=48,
           rms_eps=1e-6, rope_theta=1e6)


def make(cfg, seed, mix="q4_k_m", override=None):
    tensors = {n: (qt, d) for n, qt, d in qwen3_tensors(cfg, seed, mix)}
    if override:
        tensors.update(override)
    c = capi.Qwen3Config(cfg["n_layer"], cfg["hidden"], cfg["n_head"], cfg["n_kv_head"], cfg["head_dim"], cfg["ffn"],
                         cfg["vocab"], cfg["n_ctx"], cfg["rms_eps"], cfg["rope_theta"])
    m = capi.Qwen3(c)
    for n, (qt, d) in tensors.items():
        m.set_tensor(n, qt, d)
    return m, oq.Qwen3Oracle(cfg, tensors, avx2=oracle.have_avx2())


def close(got, ref, tol=1e-3):
    # the bound the reference's acceptance uses for f32 results: |gpu - ref| <= tol * max(|ref|, 1)
    err = np.abs(got - ref) / np.maximum(np.abs(ref), 1.0)
    return float(err.max()) <= tol, float(err.max())


@pytest.mark.parametrize("mix", ["q4_k_m", "8"])
def test_teacher_forced_logits(mix):
    m, o = make(CFG, 21, mix)
    prompt = [3, 700, 41, 41, 256, 9, 88, 511, 2, 640, 77]
    got, ref = m.forward(prompt, 0), o.forward(prompt, 0)
    ok, e = close(got, ref)
    assert ok, f"prefill: {e}"
    pos = len(prompt)
    for t in [5, 123, 767, 0, 350, 12]:
        got, ref = m.forward([t], pos), o.forward([t], pos)
        ok, e = close(got, ref)
        assert ok, f"pos {pos}: {e}"
        g = m.greedy()
        top2 = np.sort(ref)[-2:]
        if top2[1] - top2[0] > 2e-3 * max(abs(top2[1]), 1.0):
            assert g == oq.greedy(ref)
        assert got[g] == got.max()
        pos += 1


@pytest.mark.parametrize("mix", ["q4_k_m", "q4_k"])
def test_single_token_steps_with_4096_wide_rows(mix):
    """hidden = 4096: a single-token step runs residual add + RMSNorm + q|k(|v) and + gate|up as
    one launch each ("q4_k": every matrix Q4_K, v inside the fused launch; "q4_k_m": some layers keep
    attn_v as Q6_K, a launch of its own over the normalised row the fused kernel leaves behind)."""
    cfg = dict(CFG, n_layer=4, hidden=4096, n_head=4, n_kv_head=2, head_dim=128, ffn=1024, vocab=512, n_ctx=32)
    m, o = make(cfg, 29, mix)
    prompt = [3, 500, 41, 41, 256, 9]
    ok, e = close(m.forward(prompt, 0), o.forward(prompt, 0))
    assert ok, f"prefill: {e}"
    pos = len(prompt)
    for t in [5, 123, 511, 0, 350]:
        ok, e = close(m.forward([t], pos), o.forward([t], pos))
        assert ok, f"pos {pos}: {e}"
        pos += 1


@pytest.mark.parametrize("mix", ["q4_k_m", "q4_k"])
def test_single_token_steps_with_2048_wide_rows(mix):
    """hidden = 2048: residual add + RMSNorm + q|k(|v) of a single-token step are one launch of the kernel
    that takes a tile of 16 rows a workgroup; gate, up and the rest run as launches of their own."""
    cfg = dict(CFG, n_layer=4, hidden=2048, n_head=4, n_kv_head=2, head_dim=128, ffn=768, vocab=512, n_ctx=32)
    m, o = make(cfg, 37, mix)
    prompt = [3, 500, 41, 41, 256, 9]
    ok, e = close(m.forward(prompt, 0), o.forward(prompt, 0))
    assert ok, f"prefill: {e}"
    pos = len(prompt)
    for t in [5, 123, 511, 0, 350]:
        ok, e = close(m.forward([t], pos), o.forward([t], pos))
        assert ok, f"pos {pos}: {e}"
        pos += 1


def test_single_token_steps_with_attn_v_of_another_format_in_the_qk_launch():
    """hidden = 4096 and 2560 rows of q|k: on the layers that keep attn_v as Q6_K or Q8_0 (four of these eight, two of
    each) its tiles run in the launch of residual add + RMSNorm + q|k, behind the workgroups of the Q4_K product."""
    cfg = dict(CFG, n_layer=8, hidden=4096, n_head=16, n_kv_head=4, head_dim=128, ffn=512, vocab=512, n_ctx=32)
    m, o = make(cfg, 39, "q4_k_m")
    kinds = {o.t[f"blk.{l}.attn_v.weight"][0] for l in range(8)}
    assert {capi.Q6_K, capi.Q8_0} <= kinds
    prompt = [3, 500, 41, 41, 256, 9]
    ok, e = close(m.forward(prompt, 0), o.forward(prompt, 0))
    assert ok, f"prefill: {e}"
    pos = len(prompt)
    for t in [5, 123, 511, 0]:
        ok, e = close(m.forward([t], pos), o.forward([t], pos))
        assert ok, f"pos {pos}: {e}"
        pos += 1


def test_single_token_steps_over_one_to_eighteen_key_chunks():
    """32 heads of 128, four KV heads: single-token steps whose split attention covers one, two, three, five and
    eighteen chunks of 64 keys, between prefill chunks of 61 to 830 tokens."""
    cfg = dict(CFG, n_layer=2, hidden=512, n_head=32, n_kv_head=4, head_dim=128, ffn=512, vocab=512, n_ctx=1120)
    m, o = make(cfg, 41, "q4_k")
    rng = np.random.default_rng(17)
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], size=1110)]
    pos = 0
    for step in (1, 1, 61, 1, 1, 1, 64, 1, 130, 1, 1, 830, 1, 1):   # single-token steps at 1, 2, 64..66, 131, 262, 1093.. cached tokens
        chunk = toks[pos:pos + step]
        ok, e = close(m.forward(chunk, pos), o.forward(chunk, pos))
        assert ok, f"pos {pos} +{step}: {e}"
        pos += step


def test_paired_gate_up_rows_serve_prefill_and_replacement():
    """With 4096-wide Q4_K rows the gate and up matrices are stored with alternating rows (the
    single-token launch applies SwiGLU itself); multi-token steps read them as strided views, and a
    replaced part sends the layer back to separate launches."""
    cfg = dict(CFG, n_layer=2, hidden=4096, n_head=4, n_kv_head=2, head_dim=128, ffn=512, vocab=512, n_ctx=40)
    m, o = make(cfg, 31, "q4_k")
    toks = [7, 400, 41, 300, 256, 9, 12, 13, 14, 15, 16, 17, 18, 19, 20, 21, 22, 23, 24, 25]
    ok, e = close(m.forward(toks[:1], 0), o.forward(toks[:1], 0))      # fuses on the first single-token step
    assert ok, e
    ok, e = close(m.forward(toks[1:4], 1), o.forward(toks[1:4], 1))    # 3 rows: views under the few-row kernel
    assert ok, e
    ok, e = close(m.forward(toks[4:], 4), o.forward(toks[4:], 4))      # 16 rows
    assert ok, e
    m.reset(), o.reset()
    ok, e = close(m.forward(toks + toks, 0), o.forward(toks + toks, 0))  # 40 rows: views under the GEMM
    assert ok, e
    name = "blk.1.ffn_up.weight"
    tensors = {n: (qt, d) for n, qt, d in qwen3_tensors(cfg, 31, "q4_k")}
    tensors[name] = {n: (qt, d) for n, qt, d in qwen3_tensors(cfg, 99, "q4_k")}[name]
    m.set_tensor(name, *tensors[name])
    o2 = oq.Qwen3Oracle(cfg, tensors, avx2=oracle.have_avx2())
    m.reset()
    ok, e = close(m.forward([5], 0), o2.forward([5], 0))
    assert ok, e
    ok, e = close(m.forward([6], 1), o2.forward([6], 1))
    assert ok, e


def test_prefill_in_two_chunks_matches_one():
    m, o = make(CFG, 22)
    toks = list(range(10, 30))
    ref = o.forward(toks, 0)
    m.forward(toks[:13], 0)
    got = m.forward(toks[13:], 13)
    ok, e = close(got, ref)
    assert ok, e


@pytest.mark.parametrize("n_head,n_kv", [(4, 1), (4, 2), (2, 2)])
def test_prefill_in_chunks_with_head_size_128(n_head, n_kv):
    """Chunks of more than 8 tokens at a position past 0: the tiled attention with keys already in the
    cache, token counts that leave the last tile part empty, and a chunk that starts inside a key tile."""
    cfg = dict(CFG, n_ctx=96, n_layer=2, head_dim=128, n_head=n_head, n_kv_head=n_kv)
    m, o = make(cfg, 27)
    rng = np.random.default_rng(4)
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], size=90)]
    pos = 0
    for step in (21, 16, 37, 9):
        chunk = toks[pos:pos + step]
        ok, e = close(m.forward(chunk, pos), o.forward(chunk, pos))
        assert ok, f"pos {pos} +{step}: {e}"
        pos += step


@pytest.mark.parametrize("mix", ["q4_k_m", "q4_k"])
def test_prefill_of_many_tokens_with_4096_wide_rows(mix):
    """80 and 70 tokens a step at hidden = 4096: q|k(|v) as one product read through row strides, gate|up as
    one product over the paired matrix, SwiGLU applied by the down projection's activation preparation
    (Q4_K and, in the q4_k_m mix, Q6_K down projections on the int8 GEMM), then single-token steps."""
    cfg = dict(CFG, n_layer=2, hidden=4096, n_head=4, n_kv_head=2, head_dim=128, ffn=1024, vocab=512, n_ctx=192)
    m, o = make(cfg, 35, mix)
    rng = np.random.default_rng(15)
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], size=153)]
    pos = 0
    for step in (80, 70, 1, 1, 1):
        chunk = toks[pos:pos + step]
        ok, e = close(m.forward(chunk, pos), o.forward(chunk, pos))
        assert ok, f"pos {pos} +{step}: {e}"
        pos += step


@pytest.mark.parametrize("n_head,n_kv", [(4, 1), (4, 2), (2, 2), (8, 1)])
def test_long_prefill_chunks_split_their_keys_between_two_sets_of_waves(n_head, n_kv):
    """From 128 keys on the tiled attention gives the key tiles of even and odd number to two sets of waves
    and merges their running softmax states (up to four query heads a KV head; eight keep one set): a chunk
    from position 0, chunks that start inside a key tile, an odd number of key tiles, a last tile part empty."""
    cfg = dict(CFG, n_ctx=400, n_layer=2, head_dim=128, n_head=n_head, n_kv_head=n_kv)
    m, o = make(cfg, 33)
    rng = np.random.default_rng(14)
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], size=390)]
    pos = 0
    for step in (137, 150, 9, 94):
        chunk = toks[pos:pos + step]
        ok, e = close(m.forward(chunk, pos), o.forward(chunk, pos))
        assert ok, f"pos {pos} +{step}: {e}"
        pos += step


@pytest.mark.parametrize("head_dim,n_head,n_kv", [(64, 4, 2), (128, 4, 1), (256, 2, 2), (192, 4, 2), (128, 8, 1),
                                                  (128, 2, 2), (128, 4, 2)])
def test_decode_over_several_key_chunks(head_dim, n_head, n_kv):
    """A cache longer than one 64-key chunk of the split attention kernel, entered both by a
    long prefill and by short multi-token steps; head sizes with and without a split kernel.  The
    multi-token steps with head size 128 run the tiled matrix-core attention, with 8, 4, 2 and 1 query
    heads a KV head, token counts that do not fill a tile and keys already in the cache."""
    cfg = dict(CFG, n_ctx=224, n_layer=2, head_dim=head_dim, n_head=n_head, n_kv_head=n_kv)
    m, o = make(cfg, 26)
    rng = np.random.default_rng(3)
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], size=190)]
    ok, e = close(m.forward(toks[:150], 0), o.forward(toks[:150], 0))
    assert ok, f"prefill: {e}"
    pos = 150
    for step in (1, 5, 8, 1, 3, 1, 1):
        chunk = toks[pos:pos + step]
        ok, e = close(m.forward(chunk, pos), o.forward(chunk, pos))
        assert ok, f"pos {pos} +{step}: {e}"
        pos += step


def test_replacing_a_tensor_after_decoding_takes_effect():
    """Single-token steps run q|k|v and gate|up as fused launches; a tensor set afterwards must win."""
    tensors = {n: (qt, d) for n, qt, d in qwen3_tensors(CFG, 27)}
    m, o = make(CFG, 27)
    m.forward([5, 6, 7], 0)
    m.forward([8], 3)                       # builds the fused copies
    other = {n: (qt, d) for n, qt, d in qwen3_tensors(CFG, 28)}
    for name in ("blk.1.attn_k.weight", "blk.2.ffn_up.weight"):
        tensors[name] = other[name]
        m.set_tensor(name, *other[name])
    o2 = oq.Qwen3Oracle(CFG, tensors, avx2=oracle.have_avx2())
    m.reset()
    ref = o2.forward([5, 6, 7], 0)
    ok, e = close(m.forward([5, 6, 7], 0), ref)
    assert ok, e
    ok, e = close(m.forward([8], 3), o2.forward([8], 3))
    assert ok, e


def test_position_contract_and_reset():
    m, _ = make(CFG, 23)
    a = m.forward([1, 2, 3], 0)
    with pytest.raises(capi.JoshuaHipError, match="does not match"):
        m.forward([4], 5)
    with pytest.raises(capi.JoshuaHipError, match="exceed the context"):
        m.forward(list(range(46)), 3)
    with pytest.raises(capi.JoshuaHipError, match="out of range"):
        m.forward([768], 3)
    with pytest.raises(capi.JoshuaHipError, match="at least one token"):
        m.forward([], 3)
    m.reset()
    b = m.forward([1, 2, 3], 0)
    assert np.array_equal(a, b)


def test_missing_tensor_is_reported():
    c = capi.Qwen3Config(1, 256, 2, 1, 64, 256, 256, 8, 1e-6, 1e4)
    m = capi.Qwen3(c)
    with pytest.raises(capi.JoshuaHipError, match="missing tensor"):
        m.forward([1], 0)
    with pytest.raises(capi.JoshuaHipError, match="unknown tensor"):
        m.set_tensor("blk.0.nope.weight", 0, np.zeros(4, np.float32))
    with pytest.raises(capi.JoshuaHipError, match="expected"):
        m.set_tensor("output_norm.weight", 0, np.zeros(4, np.float32))


def test_greedy_returns_last_index_of_equal_logits():
    # every row of the head identical -> all logits equal -> the last index wins
    from joshua_amd.synth import normal, quantize
    row = normal(5, (1, CFG["hidden"]), 0.05)
    head = quantize(8, np.repeat(row, CFG["vocab"], axis=0))
    m, _ = make(CFG, 24, override={"output.weight": (8, head)})
    logits = m.forward([1, 2], 0)
    assert np.all(logits == logits[0])
    assert m.greedy() == CFG["vocab"] - 1


def test_tied_embeddings_when_no_output_head():
    tensors = {n: (qt, d) for n, qt, d in qwen3_tensors(CFG, 25)}
    del tensors["output.weight"]
    c = capi.Qwen3Config(CFG["n_layer"], CFG["hidden"], CFG["n_head"], CFG["n_kv_head"], CFG["head_dim"], CFG["ffn"],
                         CFG["vocab"], CFG["n_ctx"], CFG["rms_eps"], CFG["rope_theta"])
    m = capi.Qwen3(c)
    for n, (qt, d) in tensors.items():
        m.set_tensor(n, qt, d)
    o = oq.Qwen3Oracle(CFG, tensors, avx2=oracle.have_avx2())
    ok, e = close(m.forward([9, 8, 7], 0), o.forward([9, 8, 7], 0))
    assert ok, e


FALLBACK_CHILD = r"""
import sys, numpy as np
sys.path.insert(0, %r)
from tests.test_gpu_qwen3 import CFG, make, close
cfg = dict(CFG, n_layer=2, hidden=4096, n_head=4, n_kv_head=2, head_dim=128, ffn=512, vocab=512, n_ctx=32)
m, o = make(cfg, 33, "q4_k")
pos = 0
for chunk in ([3, 500, 41], [7], [9], [256, 12]):
    ok, e = close(m.forward(chunk, pos), o.forward(chunk, pos))
    assert ok, (pos, e)
    pos += len(chunk)
print("fallback ok")
"""


@pytest.mark.parametrize("env", [{"JQ_Q4K_DOT4": "0"}, {"JQ_NO_FUSED_NORM": "1"}, {"JQ_NO_PAIRED_GATE_UP": "1"}])
def test_single_token_steps_without_the_fused_launches(env):
    """The switches are read when the library first dispatches, so each runs in a child process: without
    the v_dot4 kernel the row-paired gate|up matrix goes through the plain product and a pairwise
    SwiGLU; without the fused norm the pieces run as launches of their own; without pairing gate and up
    are laid one after the other."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, "-c", FALLBACK_CHILD % root], env=dict(os.environ, **env), capture_output=True,
                         text=True, timeout=110)
    assert res.returncode == 0 and "fallback ok" in res.stdout, res.stdout + res.stderr


def test_short_step_across_a_key_chunk_boundary_after_a_longer_context():
    """A step of 2..8 tokens whose first tokens end before a 64-key chunk that its last tokens reach:
    those tokens have no sums for that chunk, and the buffer of partial sums still holds an earlier,
    longer context's values (laid out for more chunks, so its -inf markers sit where sums are read now).
    The merge must leave such chunks out; weighting them by zero turns inf into NaN."""
    cfg = dict(CFG, n_ctx=224, n_layer=2)
    m, o = make(cfg, 35)
    rng = np.random.default_rng(6)
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], size=200)]
    m.forward(toks[:124], 0)
    m.forward(toks[124:132], 124)           # 3 chunks; tokens 0..3 stop at key 127 and skip the third
    m.forward(toks[132:196], 132)
    m.forward(toks[196:198], 196)           # 4 chunks: 196 keys for token 0 ... stride of the buffer changes
    m.reset()
    got, ref = m.forward(toks[:60], 0), o.forward(toks[:60], 0)
    ok, e = close(got, ref)
    assert ok, f"prefill: {e}"
    for pos, step in ((60, 8), (68, 1), (69, 3)):     # 60 + 8 crosses key 64; tokens 0..3 skip chunk 1
        chunk = toks[pos:pos + step]
        got, ref = m.forward(chunk, pos), o.forward(chunk, pos)
        assert np.all(np.isfinite(got)), f"pos {pos} +{step}: non-finite logits"
        ok, e = close(got, ref)
        assert ok, f"pos {pos} +{step}: {e}"


def test_long_context_with_five_query_heads_a_kv_head():
    """5 query heads a KV head take the one-row-per-workgroup attention for steps of more than 8 tokens;
    its scores go by in chunks, so a context of more than 16384 keys (64 KB of scores a row) works.
    Prefill in chunks of 2048 up to 16384 tokens, then a 16-token step whose rows see up to 16400 keys."""
    cfg = dict(n_layer=1, hidden=256, n_head=5, n_kv_head=1, head_dim=64, ffn=256, vocab=256, n_ctx=16400 + 16,
               rms_eps=1e-6, rope_theta=1e6)
    m, o = make(cfg, 36, "8")            # Q8_0: blocks of 32 fit the 320-wide attention output
    rng = np.random.default_rng(7)
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], size=16400)]
    pos = 0
    while pos < 16384:
        m.forward_only(toks[pos:pos + 2048], pos)
        o.forward(toks[pos:pos + 2048], pos)
        pos += 2048
    got, ref = m.forward(toks[pos:pos + 16], pos), o.forward(toks[pos:pos + 16], pos)
    ok, e = close(got, ref)
    assert ok, e
