"""GPU parity of the MoE layer (router, top-k, grouped expert matmuls, combine)
against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

import oracle
from oracle.moe import MoeOracle
from joshua_amd import capi, synth

pytestmark = pytest.mark.gpu


def build(qtype, h, inter, E, k, seed, sigma=0.02, shared_inter=0, **kw):
    rw = synth.normal(seed, (E, h), sigma=0.02)
    gate = synth.normal_quantized(qtype, seed + 1, E * inter * h, sigma)
    up = synth.normal_quantized(qtype, seed + 2, E * inter * h, sigma)
    down = synth.normal_quantized(qtype, seed + 3, E * h * inter, sigma)
    shared_o = shared_w = None
    if shared_inter:
        sg = synth.normal_quantized(qtype, seed + 4, shared_inter * h, sigma)
        su = synth.normal_quantized(qtype, seed + 5, shared_inter * h, sigma)
        sd = synth.normal_quantized(qtype, seed + 6, h * shared_inter, sigma)
        shared_o = (qtype, shared_inter, sg, su, sd)
        shared_w = (capi.Weight.upload(qtype, sg, shared_inter, h), capi.Weight.upload(qtype, su, shared_inter, h),
                    capi.Weight.upload(qtype, sd, h, shared_inter))
    ora = MoeOracle(qtype, h, inter, E, k, rw, gate, up, down, shared=shared_o, avx2=oracle.have_avx2(), **kw)
    cfg = capi.MoeConfig(E, k, h, inter, 1 if kw.get("gating") == "sigmoid" else 0, 1 if kw.get("norm_topk", True) else 0,
                         float(kw.get("weights_scale", 0.0)), kw.get("n_group", 1), kw.get("topk_group", 1),
                         float(kw.get("swiglu_clamp", 0.0)), float(kw.get("swiglu_clamp_shared", 0.0)))
    dev = capi.Moe(cfg, rw, capi.Weight.upload(qtype, gate, E * inter, h), capi.Weight.upload(qtype, up, E * inter, h),
                   capi.Weight.upload(qtype, down, E * h, inter), router_bias=kw.get("router_bias"), shared=shared_w)
    return ora, dev


def close(got, want, tol=1e-3):
    return np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1.0))


@pytest.mark.parametrize("kw", [
    dict(), dict(norm_topk=False),
    dict(gating="sigmoid", weights_scale=2.5),
    dict(gating="sigmoid", n_group=4, topk_group=2, router_bias=np.linspace(-0.05, 0.05, 32).astype(np.float32)),
    dict(gating="softmax", n_group=8, topk_group=3),
])
def test_route_matches_oracle(kw):
    ora, dev = build(capi.Q8_0, 512, 32, 32, 6, 40, **kw)
    x = synth.normal(41, (9, 512))
    ids, w = dev.route(x)
    oid, ow = ora.route(x)
    assert np.array_equal(ids, oid)
    assert np.allclose(w, ow, rtol=2e-5, atol=1e-7)


@pytest.mark.parametrize("h,E,tokens", [(544, 30, 45), (2080, 9, 33), (1024, 64, 128)])
def test_router_logits_of_many_tokens_are_those_of_few(h, E, tokens):
    """From 32 tokens on the logits come from a kernel that works on 8 experts x 8 tokens a workgroup (an expert
    count and a token count that are not multiples of 8, a row that ends inside a step of 1024 columns); it adds
    the same products in the same order, so ids and weights equal those of calls of 8 tokens bit for bit."""
    ora, dev = build(capi.Q8_0, h, 32, E, 4, 50 + E)
    x = synth.normal(51 + E, (tokens, h))
    ids, w = dev.route(x)
    assert np.array_equal(ids, ora.route(x)[0])
    for t0 in range(0, tokens, 8):
        i8, w8 = dev.route(x[t0:t0 + 8])
        assert np.array_equal(ids[t0:t0 + 8], i8) and np.array_equal(w[t0:t0 + 8], w8)


@pytest.mark.parametrize("tokens", [1, 2, 7, 64])
def test_qwen3moe_shaped_layer_q4k(tokens):
    """Qwen3-30B-A3B layer shape (h 2048, inter 768, top-8) with 16 experts."""
    ora, dev = build(capi.Q4_K, 2048, 768, 16, 8, 60)
    x = synth.normal(61 + tokens, (tokens, 2048))
    assert close(dev.forward(x), ora.forward(x))


def test_decode_and_grouped_dispatch_agree_on_device():
    """reference: src/quantized_qwen3_moe.rs:912-928 (prefill vs decode path, 1e-4)."""
    ora, dev = build(capi.Q4_K, 512, 256, 8, 2, 70)
    row = synth.normal(71, (1, 512))
    many = np.repeat(row, 9, axis=0)              # 18 pairs > 8 experts: grouped path
    one = dev.forward(row)
    assert np.all(np.abs(dev.forward(many) - one) < 1e-4)


@pytest.mark.parametrize("qtype", [capi.IQ2_XXS, capi.MXFP4, capi.Q6_K, capi.Q2_K, capi.Q8_0])
def test_deepseek_style_layer_with_shared_expert(qtype):
    ora, dev = build(qtype, 1024, 512, 16, 4, 80, shared_inter=512, gating="sigmoid", n_group=4, topk_group=2,
                     weights_scale=2.5, router_bias=np.linspace(-0.02, 0.02, 16).astype(np.float32))
    for tokens in (1, 5):
        x = synth.normal(81 + tokens, (tokens, 1024))
        assert close(dev.forward(x), ora.forward(x))


def test_shared_expert_of_another_width_runs_beside_the_groups():
    ora, dev = build(capi.Q4_K, 512, 512, 8, 2, 90, shared_inter=256, gating="sigmoid")
    for tokens in (1, 6):
        x = synth.normal(91 + tokens, (tokens, 512))
        assert close(dev.forward(x), ora.forward(x))


def test_q4k_groups_of_many_tokens_with_the_shared_expert_folded_in():
    """40 tokens: the shared expert's group holds all 40 (three passes of 16 in the grouped MFMA
    kernel), routed groups hold 0 to about 20."""
    ora, dev = build(capi.Q4_K, 1024, 768, 8, 2, 95, shared_inter=768, gating="sigmoid")
    x = synth.normal(96, (40, 1024))
    assert close(dev.forward(x), ora.forward(x))


@pytest.mark.parametrize("h,inter", [(4096, 256), (512, 2560), (256, 3072)])
def test_q4k_grouped_kernels_at_other_row_lengths(h, inter):
    """16-super-block gate/up rows (outside the fused MFMA kernel's reach), and down rows of 10 and
    12 super-blocks (two columns a wave)."""
    ora, dev = build(capi.Q4_K, h, inter, 4, 2, 97 + inter)
    x = synth.normal(98, (19, h))
    assert close(dev.forward(x), ora.forward(x))


@pytest.mark.parametrize("qtype,h,inter", [
    (capi.Q6_K, 768, 256),      # 630-byte rows: no aligned staging, plain kernels; 256-wide down rows: 16 lanes a row
    (capi.IQ2_XXS, 2560, 512),  # 660-byte rows: 4-byte staging
    (capi.IQ2_XXS, 1792, 256),  # 462-byte rows: plain kernels
    (capi.Q8_0, 96, 64),        # 102-byte rows, three blocks a row
    (capi.MXFP4, 160, 96),      # 85-byte rows
])
def test_row_lengths_that_change_the_staging(qtype, h, inter):
    ora, dev = build(qtype, h, inter, 8, 3, 100 + h)
    for tokens in (1, 11):
        x = synth.normal(101 + tokens, (tokens, h))
        assert close(dev.forward(x), ora.forward(x))


@pytest.mark.parametrize("tokens,E,k", [(300, 16, 4), (1000, 16, 4), (1024, 24, 4), (1100, 16, 4), (150, 160, 6),
                                        (500, 200, 8)])   # the last: a rank table of more than 64 KB
def test_many_tokens_are_grouped_by_expert_in_pair_order(tokens, E, k):
    """Pair lists of up to 4096 pairs are grouped by ranks within chunks of 64 pairs (one to four chunks a
    wave, a last chunk part empty, experts nobody picked); longer lists, or more chunks x experts than the
    LDS table holds, by one pass per expert.  A pair out of place would multiply a token by another expert
    or add it to another token's sum."""
    ora, dev = build(capi.Q8_0, 128, 64, E, k, 140 + tokens)
    x = synth.normal(141 + tokens, (tokens, 128))
    ids, _ = dev.route(x)
    assert np.array_equal(ids, ora.route(x)[0])
    assert close(dev.forward(x), ora.forward(x))


@pytest.mark.parametrize("qtype", [capi.Q4_K, capi.MXFP4, capi.IQ2_XXS])
def test_decode_sized_call_over_large_expert_matrices(qtype):
    """One token, expert matrices large enough that the integer-dot kernels take their activations
    from the separate quantisation launch rather than quantising them in every workgroup."""
    ora, dev = build(qtype, 2048, 4352, 2, 1, 120)
    x = synth.normal(121, (1, 2048))
    assert close(dev.forward(x), ora.forward(x))


@pytest.mark.parametrize("qtype,h,inter,E,k,shared_inter,tokens", [
    (capi.Q4_K, 2048, 768, 16, 4, 0, 4),          # 16 rows a workgroup, planes quantised by the workgroup
    (capi.MXFP4, 4096, 512, 16, 4, 512, 2),       # shared expert as a fifth pair
    (capi.IQ2_XXS, 4096, 2048, 8, 4, 2048, 1),    # planes copied from the quantisation launch, shared expert
    (capi.MXFP4, 4128, 2048, 8, 3, 0, 2),         # three pairs a token, two tokens
])
def test_decode_sized_down_projection_with_the_combine_fused(qtype, h, inter, E, k, shared_inter, tokens):
    """Decode-sized calls with 512 workgroups or more in the down projection: one launch walks each
    token's pairs and forms the weighted sum itself."""
    kw = dict(gating="sigmoid", weights_scale=2.5) if shared_inter else {}
    ora, dev = build(qtype, h, inter, E, k, 130 + h, shared_inter=shared_inter, **kw)
    x = synth.normal(131 + tokens, (tokens, h))
    want = ora.forward(x)
    assert close(dev.forward(x), want)
    assert close(dev.forward(x), want)


def test_many_tokens_group_beyond_the_lds_pair_list():
    ora, dev = build(capi.Q8_0, 64, 32, 4, 2, 110)
    x = synth.normal(111, (6200, 64))          # 12400 pairs
    ids, w = dev.route(x)
    oid, ow = ora.route(x)
    assert np.array_equal(ids, oid)
    assert close(dev.forward(x), ora.forward(x))


def test_moe_rejects_mismatched_shapes():
    gate = capi.Weight.upload(capi.Q8_0, synth.normal_quantized(capi.Q8_0, 1, 4 * 32 * 256, 0.02), 4 * 32, 256)
    down = capi.Weight.upload(capi.Q8_0, synth.normal_quantized(capi.Q8_0, 2, 4 * 256 * 32, 0.02), 4 * 256, 32)
    rw = synth.normal(3, (4, 256))
    with pytest.raises(capi.JoshuaHipError):
        capi.Moe(capi.MoeConfig(4, 5, 256, 32, 0, 1, 0.0, 1, 1), rw, gate, gate, down)      # k > E
    with pytest.raises(capi.JoshuaHipError):
        capi.Moe(capi.MoeConfig(4, 2, 256, 64, 0, 1, 0.0, 1, 1), rw, gate, gate, down)      # wrong inter


@pytest.mark.parametrize("qtype,h,inter,tokens,shared_inter", [
    (capi.Q4_K, 512, 256, 1, 0),       # decode-sized call, integer-dot kernel
    (capi.MXFP4, 512, 256, 2, 256),    # the same with a shared expert riding along as a group
    (capi.Q8_0, 512, 256, 1, 0),       # decode-sized call, f32 staged kernel
    (capi.Q4_K, 1024, 256, 40, 256),   # many tokens a group: the MFMA ring kernel, shared expert folded in
    (capi.Q6_K, 512, 256, 24, 0),      # many tokens a group, f32 staged kernel
    (capi.Q4_K, 512, 256, 3, 512),     # a shared expert of another width: launches of its own
])
def test_swiglu_clamp(qtype, h, inter, tokens, shared_inter):
    """Gate clamped from above and up on both sides before the activation, with a limit of its own for
    the shared expert (reference: src/quantized_deepseek4.rs:445-462, :2419-2448); limits low enough to bite."""
    kw = dict(swiglu_clamp=0.02, swiglu_clamp_shared=0.01)
    ora, dev = build(qtype, h, inter, 16, 4, 70, shared_inter=shared_inter, **kw)
    plain, _ = build(qtype, h, inter, 16, 4, 70, shared_inter=shared_inter)
    x = synth.normal(71, (tokens, h))
    want = ora.forward(x)
    assert not close(want, plain.forward(x))          # the limits change the result
    assert close(dev.forward(x), want)


@pytest.mark.parametrize("qtype,lead_blocks", [(capi.Q8_0, 1), (capi.MXFP4, 3), (capi.IQ2_XXS, 1), (capi.Q6_K, 1)])
def test_experts_that_are_views_at_odd_block_offsets(qtype, lead_blocks):
    """Expert stacks that start mid-buffer, a whole number of 34-, 17-, 66- or 210-byte blocks in: their
    first byte is 1- or 2-byte aligned while every row is a multiple of 4 bytes long, so the kernels that load
    rows into LDS four or sixteen bytes at a time must stand aside (one and five tokens: the decode-sized and
    the grouped dispatch)."""
    h, inter, E, k_used, seed = 1024, 512, 8, 2, 300 + qtype
    bb = oracle.block_geometry(qtype)[1]
    lead = lead_blocks * bb
    assert lead % 4 != 0
    parts, views = [], []
    for i, (rows, cols) in enumerate(((inter, h), (inter, h), (h, inter))):
        blocks = synth.normal_quantized(qtype, seed + i, E * rows * cols, 0.02)
        parts.append(blocks)
        buf = np.concatenate([np.zeros(lead, np.uint8), blocks])
        # the parent: one row of whole blocks that spans the buffer; the view: the stack behind the lead
        per_block = oracle.block_geometry(qtype)[0]
        parent = capi.Weight.upload(qtype, buf, 1, buf.size // bb * per_block)
        views.append(parent.view(lead, E * rows, cols))
    rw = synth.normal(seed + 9, (E, h), 0.02)
    ora = MoeOracle(qtype, h, inter, E, k_used, rw, parts[0], parts[1], parts[2], avx2=oracle.have_avx2())
    cfg = capi.MoeConfig(E, k_used, h, inter, 0, 1, 0.0, 1, 1, 0.0, 0.0)
    dev = capi.Moe(cfg, rw, views[0], views[1], views[2])
    for tokens in (1, 5):
        x = synth.normal(seed + 20 + tokens, (tokens, h))
        assert close(dev.forward(x), ora.forward(x)), (capi.TYPE_NAMES[qtype], tokens)
    dev.close()


@pytest.mark.parametrize("tokens", [9, 20, 40])
def test_few_tokens_an_expert_take_the_int8_quads_kernel(tokens):
    """16 experts, top-2: 18 to 80 pairs over 16 experts is at most five a group on average, the range of the
    int8 kernel that multiplies four activation rows an MFMA (one quad, two quads, and groups of more than
    eight rows, which take a second pass over the weights); inter 768 gives its down projection three waves a
    workgroup, hidden 2048 its gate and up eight."""
    ora, dev = build(capi.Q4_K, 2048, 768, 16, 2, 90)
    x = synth.normal(91 + tokens, (tokens, 2048))
    if tokens == 40:
        x[:12] = x[0] + 0.01 * x[:12]                # a dozen tokens that route alike
    ids, _ = dev.route(x)
    counts = np.bincount(ids.reshape(-1), minlength=16)
    if tokens == 40:
        assert counts.max() > 8                      # at least one group needs two passes
    assert close(dev.forward(x), ora.forward(x))


@pytest.mark.parametrize("qtype,h,inter,E,k,tokens,shared_inter,kw,kernel", [
    (capi.Q4_K, 5120, 256, 8, 2, 40, 0, {}, "moe_gemm_i8_mixed"),    # rows too long for the Q4_K grouped kernels
    (capi.IQ2_XXS, 1024, 512, 8, 2, 70, 512, dict(gating="sigmoid", swiglu_clamp=0.02, swiglu_clamp_shared=0.01),
     "moe_gemm_i8_mixed"),                                           # the shared expert's 70 pairs: one tile of 128
    (capi.MXFP4, 512, 768, 16, 4, 33, 0, {}, "moe_gemm_i8_mixed"),
    (capi.Q6_K, 768, 256, 4, 2, 300, 0, {}, "moe_gemm_i8_mixed"),    # about 150 pairs an expert: a tile of 128 and one of 32
    (capi.Q2_K, 512, 256, 4, 2, 300, 0, dict(swiglu_clamp=0.02), "moe_gemm_i8_mixed"),
    (capi.Q8_0, 256, 512, 16, 4, 64, 512, dict(gating="sigmoid", weights_scale=2.5), "moe_gemm_i8_mixed"),
    (capi.MXFP4, 256, 256, 160, 6, 150, 0, {}, "moe_gemm_i8_few"),   # more experts than one pass of the tile plan; under 8 pairs an expert
    (capi.IQ2_XXS, 512, 512, 4, 2, 200, 0, {}, "moe_gemm_i8_mixed"),
    (capi.Q4_K, 512, 256, 4, 2, 300, 256, dict(gating="sigmoid"), "moe_gemm_i8_mixed"),  # 16 pairs an expert or more: ahead of the ring kernel
])
def test_many_tokens_take_the_grouped_int8_gemm(qtype, h, inter, E, k, tokens, shared_inter, kw, kernel):
    """Bucketed calls of the formats with a side of the int8 GEMM: pairs sorted by expert are laid out in row
    groups of 16 that never mix two experts, gate and up run from one preparation of the tokens, the activation
    is applied in place (with the shared expert's own clamp on its rows) and the down projection reads it.  Under 8
    pairs an expert on average: tiles of 32 rows whose waves share the weight rows; more: an expert's pairs in tiles of
    128 rows whose waves share the rows while 80 or more are left, the rest in tiles of 32 (two launches)."""
    ora, dev = build(qtype, h, inter, E, k, 150 + h, shared_inter=shared_inter, **kw)
    x = synth.normal(151 + tokens, (tokens, h))
    want = ora.forward(x)
    got = dev.forward(x)
    assert capi.last_kernel() == kernel
    assert close(got, want)
    assert np.array_equal(got, dev.forward(x))
    few = synth.normal(152, (3, h))                                   # then a decode-sized call on the same layer
    assert close(dev.forward(few), ora.forward(few))


@pytest.mark.parametrize("qtype", [capi.Q4_K, capi.MXFP4])
def test_grouped_int8_gemm_with_pairs_that_fall_unevenly(qtype):
    """260 of 300 tokens route alike: two experts get 260 pairs and more (two tiles of 128 and a tail of tiles of 32),
    the others a few each (tiles of 32 only), and experts without a pair get no tile."""
    ora, dev = build(qtype, 2048, 256, 16, 2, 171)
    x = 0.5 * synth.normal(172, (300, 2048))      # (the magnitude a normed layer gives: the GEMM's fixed point holds 1e-3 there)
    # a token whose second and third expert are well apart, so that its near-copies pick the same two
    logits = x[:40] @ ora.router_w.T
    top3 = np.sort(logits, axis=1)[:, -3:]
    x0 = x[int(np.argmax(top3[:, 1] - top3[:, 0]))].copy()
    x[:260] = x0 + 0.01 * x[:260]
    ids, _ = dev.route(x)
    assert np.array_equal(np.sort(ids, axis=1), np.sort(ora.route(x)[0], axis=1))
    counts = np.bincount(ids.reshape(-1), minlength=16)
    assert counts.max() >= 260 and counts.min() < 16
    got = dev.forward(x)
    assert capi.last_kernel() == "moe_gemm_i8_mixed"
    assert close(got, ora.forward(x))
    assert np.array_equal(got, dev.forward(x))


@pytest.mark.parametrize("qtype,h,inter,E,k,tokens,shared_inter,kw", [
    (capi.IQ2_XXS, 512, 512, 8, 2, 9, 0, {}),                       # 16 units a row: one a lane; 2 pairs an expert
    (capi.MXFP4, 1280, 384, 8, 3, 12, 384, {}),                     # 40 units over 16 lanes: a ragged third unit
    (capi.MXFP4, 4352, 128, 4, 2, 7, 128, dict(swiglu_clamp=0.5, swiglu_clamp_shared=0.25)),  # 136 units: 32 lanes, 5 a lane
    (capi.IQ2_XXS, 8704, 512, 4, 2, 5, 0, {}),                      # 272 units: 64 lanes, 5 a lane, rows of 2244 bytes
    (capi.IQ2_XXS, 1024, 4608, 6, 2, 40, 0, dict(gating="sigmoid")),  # down rows of 144 units; 13 pairs an expert
    (capi.MXFP4, 256, 2944, 5, 1, 30, 0, {}),                       # 2944 rows: 23 units (not a multiple of 4 x 16) in gate
    (capi.Q4_K, 512, 256, 8, 2, 9, 0, {}),                          # Q4_K: an offset a sub-block against the activations' sums
    (capi.Q4_K, 4096, 1536, 8, 2, 24, 1536, dict(swiglu_clamp=0.75, swiglu_clamp_shared=0.5)),  # Qwen3-235B-A22B row lengths
    (capi.Q4_K, 7168, 256, 4, 2, 6, 0, dict(gating="sigmoid")),     # rows of 28 super-blocks: seven units a lane
])
def test_few_pairs_an_expert_stream_past_weights_decoded_once(monkeypatch, qtype, h, inter, E, k, tokens, shared_inter, kw):
    """Bucketed calls of MXFP4, IQ2_XXS and Q4_K experts with few pairs an expert: moe_expert_dot8 keeps an expert's rows as
    int8 words in registers and streams the pairs' activation planes through LDS.  Row lengths that give one to
    eight units a lane on 16, 32 and 64 lanes a row, a last unit past the row's end, groups of one pair and of
    many, the folded shared expert (a group with a pair per token) and the clamped activation."""
    monkeypatch.setenv("JQ_MOE_EXPERT_DOT8_UPTO_PAIRS_PER_EXPERT", "1000")
    ora, dev = build(qtype, h, inter, E, k, 900 + h, shared_inter=shared_inter, **kw)
    x = synth.normal(901 + h, (tokens, h))
    got = dev.forward(x)
    assert capi.last_kernel() == "moe_expert_dot8"
    assert close(got, ora.forward(x))


def _random_expert_layers():
    rng = np.random.default_rng(20251125)
    cases = []
    for seed in range(10):
        qtype = [capi.MXFP4, capi.IQ2_XXS, capi.Q4_K][seed % 3]
        step = 512 if qtype == capi.IQ2_XXS else 256     # IQ2_XXS rows a multiple of 4 bytes: 512 columns
        for _ in range(100):
            h, inter = step * int(rng.integers(1, 17)), step * int(rng.integers(1, 7))
            E = int(rng.integers(2, 13))
            if h * inter * E <= 12 << 20:
                break
        k = int(rng.integers(1, min(E, 4) + 1))
        tokens = int(rng.integers(E // k + 1, 70))       # more pairs than experts
        shared = inter if rng.integers(0, 2) else 0
        cases.append((qtype, h, inter, E, k, tokens, shared, 950 + seed))
    return cases


@pytest.mark.parametrize("qtype,h,inter,E,k,tokens,shared_inter,seed", _random_expert_layers())
def test_expert_kernel_at_seeded_random_layers(monkeypatch, qtype, h, inter, E, k, tokens, shared_inter, seed):
    """moe_expert_dot8 at layer shapes drawn from a fixed seed: row lengths of 8 to 256 units (every lanes-a-row
    and units-a-lane combination comes up), 2 to 12 experts, top-1 to top-4, with and without the folded shared
    expert, against the oracle's layer.  The inputs are scaled so that gate and up results keep a standard
    deviation of about one at every row length, as a layer's normed activations give: unit-variance inputs
    against 8192 columns of weights of 0.02 make them 1.8 and the activations reach 50, where the fixed-point
    planes' error (in proportion to a row's largest magnitude) sits at the tolerance itself (one element of
    253952 at 1.06e-3)."""
    monkeypatch.setenv("JQ_MOE_EXPERT_DOT8_UPTO_PAIRS_PER_EXPERT", "1000")
    ora, dev = build(qtype, h, inter, E, k, seed, shared_inter=shared_inter)
    x = synth.normal(seed + 1, (tokens, h)) * np.float32(min(1.0, 1.0 / (0.02 * np.sqrt(h))))
    got = dev.forward(x)
    assert capi.last_kernel() == "moe_expert_dot8", (h, inter, E, k, tokens)
    assert close(got, ora.forward(x))


@pytest.mark.parametrize("tokens,shared", [(1, False), (3, False), (1, True)])
def test_q4k_experts_with_a_q6k_down_projection(tokens, shared):
    """The mix of a Q4_K_M file's layers with more bits: gate and up in Q4_K, down in Q6_K, rows of 768 (three
    210-byte blocks: 630 bytes, a multiple of neither 4 nor 16).  Decode-sized calls take the matrix-core kernels for
    both; the 16 rows of a down tile are copied as one span, which starts and ends on 16 bytes whatever the row."""
    h, inter, E, k = 2048, 768, 16, 4
    rw = synth.normal(700, (E, h), sigma=0.02)
    gate = synth.normal_quantized(capi.Q4_K, 701, E * inter * h, 0.02)
    up = synth.normal_quantized(capi.Q4_K, 702, E * inter * h, 0.02)
    down = synth.normal_quantized(capi.Q6_K, 703, E * h * inter, 0.02)
    sh_o = sh_w = None
    if shared:   # a shared expert of the same types and shape rides along as one more pair
        sg, su = (synth.normal_quantized(capi.Q4_K, 704 + i, inter * h, 0.02) for i in range(2))
        sd = synth.normal_quantized(capi.Q6_K, 706, h * inter, 0.02)
        sh_w = (capi.Weight.upload(capi.Q4_K, sg, inter, h), capi.Weight.upload(capi.Q4_K, su, inter, h),
                capi.Weight.upload(capi.Q6_K, sd, h, inter))
    ora = MoeOracle(capi.Q4_K, h, inter, E, k, rw, gate, up, down, avx2=oracle.have_avx2(), qtype_down=capi.Q6_K)
    cfg = capi.MoeConfig(E, k, h, inter, 0, 1, 0.0, 1, 1, 0.0, 0.0)
    dev = capi.Moe(cfg, rw, capi.Weight.upload(capi.Q4_K, gate, E * inter, h), capi.Weight.upload(capi.Q4_K, up, E * inter, h),
                   capi.Weight.upload(capi.Q6_K, down, E * h, inter), shared=sh_w)
    x = synth.normal(710 + tokens, (tokens, h))
    got = dev.forward(x)
    assert capi.last_kernel() == "moe_down_mfma"
    want = ora.forward(x)
    if shared:
        sx = np.ascontiguousarray(x, np.float32)
        g = oracle.matmul_t(capi.Q4_K, (tokens, h, inter), sx, sg, avx2=oracle.have_avx2())
        u = oracle.matmul_t(capi.Q4_K, (tokens, h, inter), sx, su, avx2=oracle.have_avx2())
        from oracle.moe import silu
        want = want + oracle.matmul_t(capi.Q6_K, (tokens, inter, h), (silu(g) * u).astype(np.float32), sd, avx2=oracle.have_avx2())
    assert close(got, want)
