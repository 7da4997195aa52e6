"""The numpy multi-head latent attention used as the checker, pinned by what the mathematics
fixes and by the reference's own invariants (src/quantized_deepseek2.rs:1184-1256): closed forms
of the YaRN helpers, the rotation as a complex multiplication, cache shapes, prefill ==
token-by-token decoding, and a textbook attention written with explicit loops in float64."""
import math

import numpy as np
import pytest

from oracle import mla as om
from joshua_amd.synth import normal


def tiny_cfg(**over):
    """The reference's tiny attention (:1102-1125): n_head 2, kv_lora_rank 6, 4 + 4 + 4 head dims, n_embd 8."""
    c = dict(n_embd=8, n_head=2, q_lora_rank=0, kv_lora_rank=6, qk_nope=4, qk_rope=4, v_head_dim=4,
             rms_eps=1e-5, rope_theta=10000.0, context_length=4096, yarn=None)
    c.update(over)
    return c


def tiny_tensors(c, seed=1):
    qd = c["qk_nope"] + c["qk_rope"]
    t = {
        "kv_a_mqa": (0, normal(seed + 1, (c["kv_lora_rank"] + c["qk_rope"], c["n_embd"]))),
        "kv_a_norm": normal(seed + 2, (c["kv_lora_rank"],)),
        "kv_b": (0, normal(seed + 3, (c["n_head"] * (c["qk_nope"] + c["v_head_dim"]), c["kv_lora_rank"]))),
        "o": (0, normal(seed + 4, (c["n_embd"], c["n_head"] * c["v_head_dim"]))),
    }
    if c["q_lora_rank"]:
        t["q_a"] = (0, normal(seed + 5, (c["q_lora_rank"], c["n_embd"])))
        t["q_a_norm"] = normal(seed + 6, (c["q_lora_rank"],))
        t["q_b"] = (0, normal(seed + 7, (c["n_head"] * qd, c["q_lora_rank"])))
    else:
        t["q"] = (0, normal(seed, (c["n_head"] * qd, c["n_embd"])))
    return t


def test_yarn_mscale_closed_forms():
    assert om.yarn_get_mscale(1.0, 5.0) == 1.0
    assert om.yarn_get_mscale(0.5, 5.0) == 1.0
    assert om.yarn_get_mscale(40.0, 1.0) == pytest.approx(0.1 * math.log(40.0) + 1.0, rel=1e-6)
    assert om.yarn_get_mscale(math.e, 10.0) == pytest.approx(2.0, rel=1e-6)


def test_yarn_correction_dim_is_where_a_pair_makes_num_rot_turns():
    """Pair i turns max_pos * base^(-2i/dim) / (2 pi) times over max_pos positions; the correction
    dimension for num_rot is the 2i/2 at which that equals num_rot."""
    dim, base, max_pos = 64, 10000.0, 4096
    for num_rot in (1.0, 32.0):
        d = om.yarn_find_correction_dim(num_rot, dim, base, max_pos)
        turns = max_pos * base ** (-2.0 * d / dim) / (2.0 * math.pi)
        assert turns == pytest.approx(num_rot, rel=1e-4)
    lo, hi = om.yarn_correction_range(32.0, 1.0, dim, base, max_pos)
    assert (lo, hi) == (math.floor(om.yarn_find_correction_dim(32.0, dim, base, max_pos)),
                        math.ceil(om.yarn_find_correction_dim(1.0, dim, base, max_pos)))
    assert om.yarn_correction_range(1e9, 1e-9, 8, 10000.0, 4096) == (0.0, 7.0)  # clamped to [0, dim - 1]


def test_yarn_ramp():
    r = om.yarn_linear_ramp(2.0, 6.0, 8)
    assert np.allclose(r, [0, 0, 0, 0.25, 0.5, 0.75, 1, 1])
    r = om.yarn_linear_ramp(3.0, 3.0, 6)  # equal ends: the upper one moves by 0.001
    assert np.array_equal(r[:4], [0, 0, 0, 0]) and np.array_equal(r[4:], [1, 1])


def test_rope_tables_without_and_with_yarn():
    c = tiny_cfg(qk_rope=8, context_length=64)
    cos, sin = om.rope_tables(c)
    assert cos.shape == (64, 4)
    for t, i in ((0, 0), (5, 1), (63, 3)):
        ang = t * 10000.0 ** (-2 * i / 8)
        assert cos[t, i] == pytest.approx(math.cos(ang), abs=2e-5) and sin[t, i] == pytest.approx(math.sin(ang), abs=2e-5)
    # factor 1: interpolated and extrapolated frequencies coincide, mscale is 1
    c1 = dict(c, yarn=dict(factor=1.0, orig_context_length=32, mscale_all_dim=1.0))
    cos1, sin1 = om.rope_tables(c1)
    assert np.allclose(cos1, cos, atol=1e-6) and np.allclose(sin1, sin, atol=1e-6)
    # factor 4: pairs below the ramp keep their frequency, pairs above it turn 4 times slower, and
    # the tables carry the mscale
    c4 = dict(tiny_cfg(qk_rope=64, context_length=128), yarn=dict(factor=4.0, orig_context_length=4096, mscale_all_dim=1.0))
    cos4, sin4 = om.rope_tables(c4)
    m = 0.1 * math.log(4.0) + 1.0
    lo, hi = om.yarn_correction_range(32.0, 1.0, 64, 10000.0, 4096)
    t = 17
    i = 0  # below `lo`: ramp 0, extrapolated
    assert lo >= 1
    assert cos4[t, i] == pytest.approx(m * math.cos(t * 1.0), abs=1e-4)
    i = 31  # above `hi`: ramp 1, interpolated
    assert hi <= 30
    assert sin4[t, i] == pytest.approx(m * math.sin(t * 10000.0 ** (-2 * i / 64) / 4.0), abs=1e-5)
    assert om.softmax_scale(c4) == pytest.approx(m * m / math.sqrt(c4["qk_nope"] + 64), rel=1e-6)
    assert om.softmax_scale(c) == pytest.approx(1 / math.sqrt(12), rel=1e-12)


def test_rope_interleaved_is_a_complex_rotation_of_neighbouring_pairs():
    c = tiny_cfg(qk_rope=8, context_length=64)
    cos, sin = om.rope_tables(c)
    v = normal(3, (5, 2, 8)).astype(np.float32)
    assert np.array_equal(om.rope_interleaved(v[:1], cos, sin, 0), v[:1])  # position 0
    r = om.rope_interleaved(v, cos, sin, 7)
    z = v[..., 0::2].astype(np.complex128) + 1j * v[..., 1::2]
    ang = (7 + np.arange(5))[:, None, None] * 10000.0 ** (-2 * np.arange(4) / 8)[None, None, :]
    zr = z * np.exp(1j * ang)
    assert np.allclose(r[..., 0::2], zr.real, atol=1e-4) and np.allclose(r[..., 1::2], zr.imag, atol=1e-4)
    # scores depend on the distance only
    q, k = v[:1, :1], v[1:2, :1]
    s1 = float(om.rope_interleaved(q, cos, sin, 9)[0, 0] @ om.rope_interleaved(k, cos, sin, 4)[0, 0])
    s2 = float(om.rope_interleaved(q, cos, sin, 25)[0, 0] @ om.rope_interleaved(k, cos, sin, 20)[0, 0])
    assert s1 == pytest.approx(s2, abs=1e-4)


def test_cache_holds_per_head_keys_and_values_transposed():
    """src/quantized_deepseek2.rs:1184-1209"""
    c = tiny_cfg()
    a = om.MlaOracle(c, tiny_tensors(c))
    a.forward(normal(20, (3, 8)), 0, masked=False)
    assert a.k_cache.shape == (2, 8, 3) and a.v_cache.shape == (2, 4, 3)
    a.forward(normal(21, (1, 8)), 3)
    assert a.k_cache.shape == (2, 8, 4) and a.v_cache.shape == (2, 4, 4)


@pytest.mark.parametrize("q_lora_rank", [0, 5])
def test_prefill_matches_incremental(q_lora_rank):
    """src/quantized_deepseek2.rs:1213-1256, with its bounds."""
    c = tiny_cfg(q_lora_rank=q_lora_rank)
    t = tiny_tensors(c)
    xs = normal(22, (3, 8))
    a, b = om.MlaOracle(c, t), om.MlaOracle(c, t)
    out_prefill = a.forward(xs, 0)
    out_inc = np.concatenate([b.forward(xs[i:i + 1], i) for i in range(3)])
    assert np.abs(a.k_cache - b.k_cache).max() < 1e-6 and np.abs(a.v_cache - b.v_cache).max() < 1e-6
    assert np.abs(out_prefill - out_inc).max() < 1e-5 * max(1.0, np.abs(out_prefill).max())


def textbook(c, t, x, yarn_tables):
    """Causal attention of every query over every earlier token, head by head, in float64."""
    cos, sin = yarn_tables
    nh, lkv, npe, r, vh = c["n_head"], c["kv_lora_rank"], c["qk_nope"], c["qk_rope"], c["v_head_dim"]
    qd = npe + r
    W = {k: np.asarray(v[1], np.float64) for k, v in t.items() if isinstance(v, tuple)}
    T = x.shape[0]

    def norm(v, w):
        return v / math.sqrt(float(np.mean(v * v)) + c["rms_eps"]) * np.asarray(w, np.float64)

    def rot(v, p):
        out = np.empty_like(v)
        for i in range(len(v) // 2):
            out[2 * i] = v[2 * i] * cos[p, i] - v[2 * i + 1] * sin[p, i]
            out[2 * i + 1] = v[2 * i] * sin[p, i] + v[2 * i + 1] * cos[p, i]
        return out

    keys, vals, out = [], [], np.zeros((T, c["n_embd"]))
    for p in range(T):
        xp = x[p].astype(np.float64)
        q = W["q_b"] @ norm(W["q_a"] @ xp, t["q_a_norm"]) if c["q_lora_rank"] else W["q"] @ xp
        comp = W["kv_a_mqa"] @ xp
        kv = W["kv_b"] @ norm(comp[:lkv], t["kv_a_norm"])
        k_pe = rot(comp[lkv:], p)
        keys.append([np.concatenate([kv[h * (npe + vh):h * (npe + vh) + npe], k_pe]) for h in range(nh)])
        vals.append([kv[h * (npe + vh) + npe:(h + 1) * (npe + vh)] for h in range(nh)])
        ctx = []
        for h in range(nh):
            qh = q[h * qd:(h + 1) * qd]
            qh = np.concatenate([qh[:npe], rot(qh[npe:], p)])
            s = np.array([qh @ keys[j][h] for j in range(p + 1)]) * om.softmax_scale(c)
            e = np.exp(s - s.max())
            pr = e / e.sum()
            ctx.append(sum(pr[j] * vals[j][h] for j in range(p + 1)))
        out[p] = W["o"] @ np.concatenate(ctx)
    return out


@pytest.mark.parametrize("q_lora_rank,yarn", [(0, None), (5, None), (5, dict(factor=40.0, orig_context_length=64, mscale_all_dim=1.0))])
def test_forward_equals_textbook_attention(q_lora_rank, yarn):
    c = tiny_cfg(q_lora_rank=q_lora_rank, yarn=yarn, qk_rope=8, context_length=256)
    t = tiny_tensors(c, seed=40)
    x = normal(41, (6, 8))
    want = textbook(c, t, x, om.rope_tables(c))
    a = om.MlaOracle(c, t)
    got = np.concatenate([a.forward(x[:4], 0), a.forward(x[4:5], 4), a.forward(x[5:], 5)])
    assert np.abs(got - want).max() < 2e-4 * max(1.0, np.abs(want).max())


def test_fold_kv_b_stacks_key_rows_then_value_rows_per_head():
    """src/quantized_deepseek2.rs:931-958"""
    c = tiny_cfg()
    k_b = normal(50, (2, 6, 4))  # [n_head, kv_lora_rank, qk_nope]
    v_b = normal(51, (2, 4, 6))  # [n_head, v_head_dim, kv_lora_rank]
    w = om.fold_kv_b(k_b, v_b, c)
    assert w.shape == (16, 6)
    lat = normal(52, (6,))
    for h in range(2):
        assert np.allclose(w[8 * h:8 * h + 4] @ lat, lat @ k_b[h], atol=1e-5)   # k_nope = latent . k_b
        assert np.allclose(w[8 * h + 4:8 * h + 8] @ lat, v_b[h] @ lat, atol=1e-5)
