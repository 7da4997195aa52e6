"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle on
identical seeded block bytes and activations.  Tolerance for f32 results is the
reference's own form, |gpu - ref| <= 1e-3 * max(|ref|, 1)
(reference: src/kquant_dot.rs:853); decode is compared bit for bit."""
import os

import numpy as np
import pytest

import oracle
from joshua_amd import capi, synth
from tests.test_oracle_matmul import fixture_iq2xxs_rhs, mxfp4_pattern, ref_lhs, ref_weights

pytestmark = pytest.mark.gpu

TOL = 1e-3


def close(got, want):
    return np.all(np.abs(got - want) <= TOL * np.maximum(np.abs(want), 1.0))


def make_blocks(qtype, n, k, seed, sigma=0.02):
    return synth.normal_quantized(qtype, seed, n * k, sigma)


@pytest.mark.parametrize("qtype", capi.ALL_TYPES)
def test_dequantize_bit_exact(qtype):
    n, k = 37, 1024
    blocks = make_blocks(qtype, n, k, 11)
    w = capi.Weight.upload(qtype, blocks, n, k)
    got = w.dequantize()
    want = oracle.dequantize(qtype, blocks).reshape(n, k)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("qtype", capi.ALL_TYPES)
def test_dequantize_random_bytes_bit_exact(qtype):
    """Every byte pattern is a valid block (reference: src/kquant_dot.rs:37-40)."""
    elems, nbytes = capi.block_geometry(qtype)
    n, k = 9, 4 * 256
    rng = np.random.default_rng(qtype)
    raw = rng.integers(0, 256, size=n * (k // elems) * nbytes, dtype=np.uint8)
    blk = raw.reshape(-1, nbytes)
    for off in {capi.Q8_0: (0,), capi.Q2_K: (80, 82), capi.Q4_K: (0, 2), capi.Q6_K: (208,), capi.IQ2_XXS: (0,),
                capi.MXFP4: ()}[qtype]:
        blk[:, off + 1] &= 0x7B  # finite f16 scales
    if qtype == capi.MXFP4:
        blk[:, 0] = np.clip(blk[:, 0], 90, 160)
        blk[::5, 0] = 0xFF
        blk[1::5, 0] = 0
    w = capi.Weight.upload(qtype, raw, n, k)
    got, want = w.dequantize(), oracle.dequantize(qtype, raw).reshape(n, k)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_iq2xxs_golden_vectors_on_gpu(golden_dir):
    blocks = np.fromfile(os.path.join(golden_dir, "iq2xxs_blocks.bin"), dtype=np.uint8)
    want = np.loadtxt(os.path.join(golden_dir, "iq2xxs_ref.txt"))
    got = capi.Weight.upload(capi.IQ2_XXS, blocks, 1, 1024).dequantize().reshape(-1)
    assert np.all(np.abs(got - want) <= 1e-6 * np.maximum(np.abs(want), 1.0))


REF_SHAPES = [  # reference: src/kquant_dot.rs:894-901, src/quant_matmul.rs:499-515
    (capi.Q8_0, 1, 256, 40), (capi.Q8_0, 3, 512, 17), (capi.Q8_0, 5, 128, 9),
    (capi.Q2_K, 1, 256, 40), (capi.Q2_K, 3, 512, 11), (capi.Q2_K, 5, 768, 9),
    (capi.Q4_K, 1, 256, 40), (capi.Q4_K, 3, 512, 13), (capi.Q4_K, 4, 768, 25),
    (capi.Q6_K, 1, 256, 40), (capi.Q6_K, 3, 512, 13), (capi.Q6_K, 7, 768, 10),
]


@pytest.mark.parametrize("qtype,m,k,n", REF_SHAPES)
def test_matmul_reference_test_shapes(qtype, m, k, n):
    blocks = synth.quantize(qtype, ref_weights(n, k))
    lhs = ref_lhs(m, k)
    got = capi.Weight.upload(qtype, blocks, n, k).matmul_t(m, lhs)
    assert close(got, oracle.matmul_t(qtype, (m, k, n), lhs, blocks))


@pytest.mark.parametrize("qtype,m,k,n", [
    (capi.Q2_K, 1, 7680, 2048), (capi.Q4_K, 1, 2048, 7680), (capi.Q8_0, 1, 4096, 4096), (capi.Q8_0, 32, 4096, 4096),
])
def test_matmul_reference_model_shapes(qtype, m, k, n):
    # reference: src/kquant_dot.rs:906-914
    blocks = make_blocks(qtype, n, k, 7)
    lhs = synth.normal(8, (m, k))
    got = capi.Weight.upload(qtype, blocks, n, k).matmul_t(m, lhs)
    assert close(got, oracle.matmul_t(qtype, (m, k, n), lhs, blocks, avx2=True))


@pytest.mark.parametrize("qtype", capi.ALL_TYPES)
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 8, 16, 17])
def test_matmul_small_m_all_formats(qtype, m):
    n, k = 203, 1536
    blocks = make_blocks(qtype, n, k, 100 + qtype)
    lhs = synth.normal(200 + m, (m, k))
    got = capi.Weight.upload(qtype, blocks, n, k).matmul_t(m, lhs)
    assert close(got, oracle.matmul_t(qtype, (m, k, n), lhs, blocks, avx2=True))


@pytest.mark.parametrize("m,k,n", [
    (1, 256, 5), (2, 768, 33), (1, 1280, 16), (3, 5120, 100), (1, 14336, 70), (4, 12288, 48), (16, 2048, 250),
    (5, 16384, 17), (1, 16640, 9),
])
def test_q4k_row_lengths_and_tails(m, k, n):
    """Row lengths that are not a whole number of 4-block units, tiles with
    fewer than 16 rows, and a row length beyond the MFMA kernel's reach."""
    blocks = make_blocks(capi.Q4_K, n, k, 31 + k)
    lhs = synth.normal(32 + m, (m, k))
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(m, lhs)
    assert close(got, oracle.matmul_t(capi.Q4_K, (m, k, n), lhs, blocks, avx2=True))


def test_q4k_activation_scales_span_many_orders():
    """Fixed-point activation groups: rows mixing 1e-6 .. 1e6 magnitudes, zero
    groups and a single nonzero element still meet the f32 tolerance."""
    n, k = 64, 4096
    blocks = make_blocks(capi.Q4_K, n, k, 77)
    rng = np.random.default_rng(5)
    lhs = synth.normal(78, (3, k))
    lhs[0] *= (10.0 ** rng.integers(-6, 7, size=k // 16)).repeat(16).astype(np.float32)
    lhs[1, :] = 0.0
    lhs[1, 1234] = 3.5
    lhs[2, 512:1024] = 0.0
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(3, lhs)
    assert close(got, oracle.matmul_t(capi.Q4_K, (3, k, n), lhs, blocks, avx2=True))


def q4k_integer_case(n, k, seed, group=16, big_value=4161407, small=65535):
    """Q4_K blocks with d = 1, dmin = 0, every sub-block scale 1 and at most 16 nonzero
    nibbles per row; activations are integers whose every 16-element group has maximum
    magnitude 4161407 (the fixed-point range of the MFMA kernel, so its activation scale
    is exactly 1) at a position whose nibble is 0.  Every product and partial sum is an
    integer below 2^24: f32 FMA, integer MFMA and int64 arithmetic must agree exactly."""
    rng = np.random.default_rng(seed)
    q = np.zeros((n, k), np.int64)
    x = rng.integers(-small, small + 1, size=k).astype(np.int64)
    big = np.arange(0, k, group) + int(rng.integers(0, group))     # same slot in every group
    x[big] = big_value * rng.choice([-1, 1], size=k // group)
    free = np.setdiff1d(np.arange(k), big)
    for r in range(n):
        q[r, rng.choice(free, size=16, replace=False)] = rng.integers(1, 16, size=16)
    qb = q.reshape(n, k // 256, 4, 2, 32)                      # chunk c: low nibbles 64c.., high 64c+32..
    packed = (qb[:, :, :, 0, :] | (qb[:, :, :, 1, :] << 4)).astype(np.uint8).reshape(n, k // 256, 128)
    blocks = np.zeros((n, k // 256, 144), np.uint8)
    blocks[:, :, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blocks[:, :, 4:8] = 1                                       # sc_0..3 = 1, m = 0
    blocks[:, :, 12:16] = 1                                     # sc_4..7 = 1 (low 4 bits), m = 0
    blocks[:, :, 16:] = packed
    return blocks.reshape(-1), q, x


@pytest.mark.parametrize("m", [1, 2, 5, 16])
def test_q4k_integer_dot_products_are_bit_exact(m):
    n, k = 160, 2048 if m > 1 else 1792   # (one row over rows of 2048 has a kernel and a test of its own)
    if m <= 2:   # int8 MFMA GEMV: activation range 4161407 per 16-element group
        blocks, q, x = q4k_integer_case(n, k, 90 + m)
    else:        # streaming f16 MFMA kernel: 4193279 per 256-element super-block
        blocks, q, x = q4k_integer_case(n, k, 90 + m, group=256, big_value=4193279, small=4000)
    assert np.array_equal(oracle.dequantize(capi.Q4_K, blocks).reshape(n, k), q.astype(np.float32))
    step = 16 if m <= 2 else 256
    lhs = np.stack([np.roll(x, step * i) for i in range(m)]).astype(np.float32)
    want = (np.stack([np.roll(x, step * i) for i in range(m)]) @ q.T)
    assert np.abs(want).max() < 2 ** 24
    ref = oracle.matmul_t(capi.Q4_K, (m, k, n), lhs, blocks, avx2=oracle.have_avx2())
    assert np.array_equal(ref, want.astype(np.float32))
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(m, lhs)
    assert np.array_equal(got, want.astype(np.float32))


@pytest.mark.parametrize("m,k,n", [(16, 4096, 32768 + 5), (3, 768, 32800), (7, 1280, 33000), (4, 256, 32768)])
def test_q4k_few_rows_against_a_very_long_matrix(m, k, n):
    """From 32768 weight rows on, 3 to 16 activation rows take the LDS-ring MFMA kernel; rows of 16, 3,
    5 and 1 super-blocks change how its waves share the copying of a tile."""
    blocks = make_blocks(capi.Q4_K, n, k, 23)
    lhs = synth.normal(24 + m, (m, k))
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(m, lhs)
    assert close(got, oracle.matmul_t(capi.Q4_K, (m, k, n), lhs, blocks, avx2=oracle.have_avx2()))


def test_q4k_ring_kernel_integer_dot_products_are_bit_exact():
    n, k, m = 32768 + 16, 512, 5
    blocks, q, x = q4k_integer_case(n, k, 77, group=256, big_value=4193279, small=4000)
    lhs = np.stack([np.roll(x, 256 * i) for i in range(m)])
    want = lhs @ q.T
    assert np.abs(want).max() < 2 ** 24
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(m, lhs.astype(np.float32))
    assert np.array_equal(got, want.astype(np.float32))


@pytest.mark.parametrize("k,n", [(4096, 4096), (4096, 8 * 600 + 5), (8192, 2048 + 77), (12288, 4096), (12288, 1368 + 3)])
def test_q6k_one_row_over_4096_wide_row_groups(k, n):
    """Q6_K rows of 4096, 8192 and 12288 with one activation row take the v_dot4 kernel (8-row steps,
    one to three column groups a row tile); row counts with a ragged last tile and below one tile."""
    blocks = make_blocks(capi.Q6_K, n, k, 31)
    lhs = synth.normal(32 + n % 7, (1, k))
    got = capi.Weight.upload(capi.Q6_K, blocks, n, k).matmul_t(1, lhs)
    assert close(got, oracle.matmul_t(capi.Q6_K, (1, k, n), lhs, blocks, avx2=oracle.have_avx2()))


def q6k_integer_case(n, k, seed, nonzero=24, random_scales=False, small=3000):
    """Q6_K blocks with d = 1 and `nonzero` weights q - 32 in -32..31 a row (times the 16-element group's
    scale: 1, or any int8 value), and integer activations whose 32-element blocks peak at 32639 (activation
    scale exactly 1 per 32 and per 256 elements) where the weights are zero.  Returns (blocks, integer
    weights, activations)."""
    rng = np.random.default_rng(seed)
    q = np.zeros((n, k), np.int64)
    for r in range(n):
        idx = rng.choice(k, size=nonzero, replace=False)
        q[r, idx] = rng.integers(-32, 32, size=nonzero)
    x = rng.integers(-small, small + 1, size=k).astype(np.int64)
    peak = np.arange(0, k, 32) + int(rng.integers(0, 32))
    x[peak] = 32639 * rng.choice([-1, 1], size=k // 32)
    q[:, peak] = 0
    sc = rng.integers(-128, 128, size=(n, k // 16)) if random_scales else np.ones((n, k // 16), np.int64)
    qq = (q + 32).reshape(n, k // 256, 2, 4, 32)                   # [half][quarter][l]
    ql = np.zeros((n, k // 256, 2, 64), np.uint8)
    ql[..., :32] = (qq[:, :, :, 0, :] & 15) | ((qq[:, :, :, 2, :] & 15) << 4)
    ql[..., 32:] = (qq[:, :, :, 1, :] & 15) | ((qq[:, :, :, 3, :] & 15) << 4)
    qh = ((qq[:, :, :, 0, :] >> 4) | ((qq[:, :, :, 1, :] >> 4) << 2) | ((qq[:, :, :, 2, :] >> 4) << 4) |
          ((qq[:, :, :, 3, :] >> 4) << 6)).astype(np.uint8)
    blocks = np.zeros((n, k // 256, 210), np.uint8)
    blocks[:, :, 0:128] = ql.reshape(n, k // 256, 128)
    blocks[:, :, 128:192] = qh.reshape(n, k // 256, 64)
    blocks[:, :, 192:208] = sc.reshape(n, k // 256, 16).astype(np.int8).view(np.uint8)
    blocks[:, :, 208:210] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blocks = blocks.reshape(-1)
    w = q * sc.repeat(16, axis=1)
    assert np.array_equal(oracle.dequantize(capi.Q6_K, blocks).reshape(n, k), w.astype(np.float32))
    return blocks, w, x


def q2k_integer_case(n, k, seed, nonzero=16, min_blocks=3, small=400):
    """Q2_K blocks with d = dmin = 1: `nonzero` 2-bit weights a row under random 4-bit scales of their
    16-element sub-blocks, and `min_blocks` sub-blocks a row with a min of 1..15, so w = sc q - m in integers;
    integer activations that peak at 32639 once per 256 elements (activation scale exactly 1 per super-block).
    Returns (blocks, integer weights, activations)."""
    rng = np.random.default_rng(seed)
    q = np.zeros((n, k), np.int64)
    for r in range(n):
        q[r, rng.choice(k, size=nonzero, replace=False)] = rng.integers(1, 4, size=nonzero)
    sc = rng.integers(0, 16, size=(n, k // 16))
    mn = np.zeros((n, k // 16), np.int64)
    for r in range(n):
        mn[r, rng.choice(k // 16, size=min_blocks, replace=False)] = rng.integers(1, 16, size=min_blocks)
    x = rng.integers(-small, small + 1, size=k).astype(np.int64)
    peak = np.arange(0, k, 256) + int(rng.integers(0, 256))      # same slot in every super-block
    x[peak] = 32639 * rng.choice([-1, 1], size=k // 256)
    # element 128 sg + 32 f + 16 hf + i: field f of qs[32 sg + 16 hf + i], scale byte 8 sg + 2 f + hf
    qq = q.reshape(n, k // 256, 2, 4, 2, 16)                    # [sg][f][hf][i]
    qs = np.zeros((n, k // 256, 2, 2, 16), np.int64)             # [sg][hf][i]
    for f in range(4):
        qs |= qq[:, :, :, f, :, :] << (2 * f)
    blocks = np.zeros((n, k // 256, 84), np.uint8)
    blocks[:, :, 0:16] = (sc | (mn << 4)).reshape(n, k // 256, 16).astype(np.uint8)
    blocks[:, :, 16:80] = qs.reshape(n, k // 256, 64).astype(np.uint8)
    blocks[:, :, 80:82] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blocks[:, :, 82:84] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blocks = blocks.reshape(-1)
    w = q * sc.repeat(16, axis=1) - mn.repeat(16, axis=1)
    assert np.array_equal(oracle.dequantize(capi.Q2_K, blocks).reshape(n, k), w.astype(np.float32))
    return blocks, w, x


def q8_0_integer_case(n, k, seed, nonzero=16, small=400):
    """Q8_0 blocks whose scales are powers of two between 1/4 and 2 and `nonzero` weights q in -127..127 a
    row; integer activations that peak at 32639 once per 256 elements, where the weights are zero.  Returns
    (blocks, the weights d q as float64, activations)."""
    rng = np.random.default_rng(seed)
    q = np.zeros((n, k), np.int64)
    for r in range(n):
        q[r, rng.choice(k, size=nonzero, replace=False)] = rng.integers(-127, 128, size=nonzero)
    x = rng.integers(-small, small + 1, size=k).astype(np.int64)
    peak = np.arange(0, k, 256) + int(rng.integers(0, 256))      # same slot in every super-block
    x[peak] = 32639 * rng.choice([-1, 1], size=k // 256)
    q[:, peak] = 0
    d = rng.choice(np.array([0.25, 0.5, 1.0, 2.0]), size=(n, k // 32))
    blocks = np.zeros((n, k // 32, 34), np.uint8)
    blocks[:, :, 0:2] = d.astype(np.float16)[..., None].view(np.uint8)
    blocks[:, :, 2:] = q.reshape(n, k // 32, 32).astype(np.int8).view(np.uint8)
    blocks = blocks.reshape(-1)
    w = q * d.repeat(32, axis=1)
    assert np.array_equal(oracle.dequantize(capi.Q8_0, blocks).reshape(n, k), w.astype(np.float32))
    return blocks, w, x


def iq2xxs_integer_case(n, k, seed):
    """IQ2_XXS blocks of random codes, signs and scales with d = 8, so w = +-(2 s + 1) grid in integers (scale 0
    in the group that holds the activations' peak); activations in multiples of 2^-8: -1, 0 or 1 of them, and
    32639 of them at one slot of every 256 (activation scale exactly 2^-8 per super-block).  Returns (blocks,
    weights, activations as float64)."""
    rng = np.random.default_rng(seed)
    slot = int(rng.integers(0, 256))
    blocks = rng.integers(0, 256, size=(n, k // 256, 66), dtype=np.uint8)
    blocks[:, :, 0:2] = np.frombuffer(np.float16(8.0).tobytes(), np.uint8)
    blocks[:, :, 2 + 8 * (slot // 32) + 7] &= 0x0F           # the top nibble of the group's second word is its scale
    blocks = blocks.reshape(-1)
    w = oracle.dequantize(capi.IQ2_XXS, blocks).reshape(n, k).astype(np.float64)
    assert np.array_equal(w, np.round(w)) and np.abs(w).max() <= 1333 and np.abs(w[:, slot::256]).max() <= 43
    x = rng.integers(-1, 2, size=k).astype(np.float64)
    x[slot::256] = 32639 * rng.choice([-1, 1], size=k // 256)
    return blocks, w, x / 256.0


def mxfp4_integer_case(n, k, seed):
    """MXFP4 blocks of random codes with scales 1/4 to 1; activations in multiples of 2^-8: -2..2 of them, and
    32639 of them at one slot of every 256.  Returns (blocks, weights, activations as float64)."""
    rng = np.random.default_rng(seed)
    slot = int(rng.integers(0, 256))
    blocks = rng.integers(0, 256, size=(n, k // 32, 17), dtype=np.uint8)
    blocks[:, :, 0] = rng.integers(125, 128, size=(n, k // 32))
    blocks = blocks.reshape(-1)
    w = oracle.dequantize(capi.MXFP4, blocks).reshape(n, k).astype(np.float64)
    assert np.array_equal(8 * w, np.round(8 * w)) and np.abs(w).max() <= 6
    x = rng.integers(-2, 3, size=k).astype(np.float64)
    x[slot::256] = 32639 * rng.choice([-1, 1], size=k // 256)
    return blocks, w, x / 256.0


def q5k_integer_case(n, k, seed, nonzero=16, small=4000):
    """Q5_K blocks with d = 1, dmin = 0, every sub-block scale 1 and `nonzero` weights in 1..31 a row (the
    fifth bit of element l of sub-block j is bit j of qh[l]); integer activations that peak at 32639 at one
    slot of every 32, where the weights are zero.  Returns (blocks, integer weights, activations)."""
    rng = np.random.default_rng(seed)
    q = np.zeros((n, k), np.int64)
    x = rng.integers(-small, small + 1, size=k).astype(np.int64)
    peak = np.arange(0, k, 32) + int(rng.integers(0, 32))
    x[peak] = 32639 * rng.choice([-1, 1], size=k // 32)
    free = np.setdiff1d(np.arange(k), peak)
    for r in range(n):
        q[r, rng.choice(free, size=nonzero, replace=False)] = rng.integers(1, 32, size=nonzero)
    qb = q.reshape(n, k // 256, 4, 2, 32)                      # chunk c: sub-block 2c (low nibbles), 2c + 1 (high)
    packed = ((qb[:, :, :, 0, :] & 15) | ((qb[:, :, :, 1, :] & 15) << 4)).astype(np.uint8).reshape(n, k // 256, 128)
    qh = np.zeros((n, k // 256, 32), np.int64)
    for j in range(8):
        qh |= (q.reshape(n, k // 256, 8, 32)[:, :, j, :] >> 4) << j
    blocks = np.zeros((n, k // 256, 176), np.uint8)
    blocks[:, :, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blocks[:, :, 4:8] = 1                                       # sc_0..3 = 1, m = 0
    blocks[:, :, 12:16] = 1                                     # sc_4..7 = 1 (low 4 bits), m = 0
    blocks[:, :, 16:48] = qh.astype(np.uint8)
    blocks[:, :, 48:] = packed
    blocks = blocks.reshape(-1)
    assert np.array_equal(oracle.dequantize(capi.Q5_K, blocks).reshape(n, k), q.astype(np.float32))
    return blocks, q, x


def q4_0_integer_case(n, k, seed, nonzero=16, small=400):
    """Q4_0 blocks whose scales are powers of two between 1/2 and 4 and `nonzero` weights code - 8 in -8..7 a
    row; integer activations that peak at 32639 at one slot of every 256, where the weights are zero.
    Returns (blocks, the weights d (code - 8) as float64, activations)."""
    rng = np.random.default_rng(seed)
    q = np.zeros((n, k), np.int64)
    for r in range(n):
        q[r, rng.choice(k, size=nonzero, replace=False)] = rng.integers(-8, 8, size=nonzero)
    x = rng.integers(-small, small + 1, size=k).astype(np.int64)
    peak = np.arange(0, k, 256) + int(rng.integers(0, 256))
    x[peak] = 32639 * rng.choice([-1, 1], size=k // 256)
    q[:, peak] = 0
    d = rng.choice(np.array([0.5, 1.0, 2.0, 4.0]), size=(n, k // 32))
    codes = (q + 8).reshape(n, k // 32, 2, 16)                   # low nibbles: elements 0..15, high: 16..31
    blocks = np.zeros((n, k // 32, 18), np.uint8)
    blocks[:, :, 0:2] = d.astype(np.float16)[..., None].view(np.uint8)
    blocks[:, :, 2:] = (codes[:, :, 0, :] | (codes[:, :, 1, :] << 4)).astype(np.uint8)
    blocks = blocks.reshape(-1)
    w = q * d.repeat(32, axis=1)
    assert np.array_equal(oracle.dequantize(capi.Q4_0, blocks).reshape(n, k), w.astype(np.float32))
    return blocks, w, x


def q3k_integer_case(n, k, seed):
    """Q3_K blocks with d = 1: random 2-bit fields, third bits and 6-bit scales, so w = (sc - 32) (q - (hbit ? 0 :
    4)) in integers up to 128 in magnitude (scale 33 in the sub-block that holds the activations' peak);
    activations in multiples of 2^-8: -1, 0 or 1 of them, and 32639 of them at one slot of every 256.  Returns
    (blocks, weights, activations as float64)."""
    rng = np.random.default_rng(seed)
    slot = int(rng.integers(0, 256))
    nb = k // 256
    q2 = rng.integers(0, 4, size=(n, nb, 2, 4, 2, 16))            # [h][t][hf][i]: element 128 h + 32 t + 16 hf + i
    hb = rng.integers(0, 2, size=(n, nb, 2, 4, 2, 16))
    sc = rng.integers(0, 64, size=(n, nb, 16))                    # scale number 8 h + 2 t + hf
    h, t, hf = slot // 128, (slot % 128) // 32, (slot % 32) // 16
    sc[:, :, 8 * h + 2 * t + hf] = 33
    blocks = np.zeros((n, nb, 110), np.uint8)
    qs = np.zeros((n, nb, 2, 2, 16), np.int64)                    # [h][hf][i]
    hm = np.zeros((n, nb, 2, 16), np.int64)                       # [hf][i]
    for hh in range(2):
        for tt in range(4):
            qs[:, :, hh] |= q2[:, :, hh, tt] << (2 * tt)
            hm |= hb[:, :, hh, tt] << (4 * hh + tt)
    blocks[:, :, 0:32] = hm.reshape(n, nb, 32)
    blocks[:, :, 32:96] = qs.reshape(n, nb, 64)
    low, high = sc & 15, sc >> 4
    blocks[:, :, 96:104] = low[:, :, :8] | (low[:, :, 8:] << 4)
    for b in range(4):
        blocks[:, :, 104 + b] = high[:, :, b] | (high[:, :, 4 + b] << 2) | (high[:, :, 8 + b] << 4) | (high[:, :, 12 + b] << 6)
    blocks[:, :, 108:110] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blocks = blocks.reshape(-1)
    scale = sc.reshape(n, nb, 2, 4, 2)[..., None] - 32            # [h][t][hf] broadcast over i
    w = (scale * (q2 - 4 * (1 - hb))).reshape(n, k).astype(np.float64)
    assert np.array_equal(oracle.dequantize(capi.Q3_K, blocks).reshape(n, k), w.astype(np.float32))
    x = rng.integers(-1, 2, size=k).astype(np.float64)
    x[slot::256] = 32639 * rng.choice([-1, 1], size=k // 256)
    return blocks, w, x / 256.0


def q5_0_integer_case(n, k, seed, nonzero=16, small=400):
    """Q5_0 blocks whose scales are powers of two between 1/2 and 4 (some negative) and `nonzero` weights
    q - 16 in -16..15 a row, the fifth bit of element j in bit j of qh; integer activations that peak at 32639
    at one slot of every 256, where the weights are zero.  Returns (blocks, the weights d (q - 16) as float64,
    activations)."""
    rng = np.random.default_rng(seed)
    q = np.zeros((n, k), np.int64)
    for r in range(n):
        q[r, rng.choice(k, size=nonzero, replace=False)] = rng.integers(-16, 16, size=nonzero)
    x = rng.integers(-small, small + 1, size=k).astype(np.int64)
    peak = np.arange(0, k, 256) + int(rng.integers(0, 256))
    x[peak] = 32639 * rng.choice([-1, 1], size=k // 256)
    q[:, peak] = 0
    d = rng.choice(np.array([0.5, 1.0, 2.0, 4.0, -1.0]), size=(n, k // 32))
    codes = (q + 16).reshape(n, k // 32, 2, 16)                  # low nibbles: elements 0..15, high: 16..31
    qh = np.zeros((n, k // 32), np.int64)
    for j in range(16):
        qh |= ((codes[:, :, 0, j] >> 4) << j) | ((codes[:, :, 1, j] >> 4) << (16 + j))
    blocks = np.zeros((n, k // 32, 22), np.uint8)
    blocks[:, :, 0:2] = d.astype(np.float16)[..., None].view(np.uint8)
    blocks[:, :, 2:6] = qh.astype(np.uint32)[..., None].view(np.uint8)
    blocks[:, :, 6:] = ((codes[:, :, 0, :] & 15) | ((codes[:, :, 1, :] & 15) << 4)).astype(np.uint8)
    blocks = blocks.reshape(-1)
    w = q * d.repeat(32, axis=1)
    assert np.array_equal(oracle.dequantize(capi.Q5_0, blocks).reshape(n, k), w.astype(np.float32))
    return blocks, w, x


def q4_1_q5_1_integer_case(qtype, n, k, seed, nonzero=16, offset_blocks=3, small=400):
    """Q4_1 or Q5_1 blocks, w = d q + m: scales of 1/2 to 4, `nonzero` codes q in 1..15 (1..31) a row, and
    `offset_blocks` blocks a row with an offset m in multiples of 1/4 up to 4 in magnitude; integer activations
    that peak at 32639 at one slot of every 256, where the codes are zero.  Returns (blocks, weights as float64,
    activations)."""
    rng = np.random.default_rng(seed)
    five = qtype == capi.Q5_1
    q = np.zeros((n, k), np.int64)
    for r in range(n):
        q[r, rng.choice(k, size=nonzero, replace=False)] = rng.integers(1, 32 if five else 16, size=nonzero)
    x = rng.integers(-small, small + 1, size=k).astype(np.int64)
    peak = np.arange(0, k, 256) + int(rng.integers(0, 256))
    x[peak] = 32639 * rng.choice([-1, 1], size=k // 256)
    q[:, peak] = 0
    d = rng.choice(np.array([0.5, 1.0, 2.0, 4.0]), size=(n, k // 32))
    m = np.zeros((n, k // 32))
    for r in range(n):
        m[r, rng.choice(k // 32, size=offset_blocks, replace=False)] = rng.integers(-16, 17, size=offset_blocks) / 4.0
    codes = q.reshape(n, k // 32, 2, 16)                         # low nibbles: elements 0..15, high: 16..31
    nbytes = 24 if five else 20
    blocks = np.zeros((n, k // 32, nbytes), np.uint8)
    blocks[:, :, 0:2] = d.astype(np.float16)[..., None].view(np.uint8)
    blocks[:, :, 2:4] = m.astype(np.float16)[..., None].view(np.uint8)
    if five:
        qh = np.zeros((n, k // 32), np.int64)
        for j in range(16):
            qh |= ((codes[:, :, 0, j] >> 4) << j) | ((codes[:, :, 1, j] >> 4) << (16 + j))
        blocks[:, :, 4:8] = qh.astype(np.uint32)[..., None].view(np.uint8)
    blocks[:, :, nbytes - 16:] = ((codes[:, :, 0, :] & 15) | ((codes[:, :, 1, :] & 15) << 4)).astype(np.uint8)
    blocks = blocks.reshape(-1)
    w = q * d.repeat(32, axis=1) + m.repeat(32, axis=1)
    assert np.array_equal(oracle.dequantize(qtype, blocks).reshape(n, k), w.astype(np.float32))
    return blocks, w, x


def test_q6k_dot4_integer_dot_products_are_bit_exact():
    """d = 1, every scale 1, integer activations whose 32-element blocks peak at 32639 (activation
    scale exactly 1): the kernel's integer sums, f32 FMA and int64 arithmetic agree exactly."""
    n, k = 4096 + 3, 4096
    blocks, q, x = q6k_integer_case(n, k, 5)
    want = x @ q.T
    assert np.abs(want).max() < 2 ** 24
    got = capi.Weight.upload(capi.Q6_K, blocks, n, k).matmul_t(1, x[None, :].astype(np.float32))
    assert np.array_equal(got[0], want.astype(np.float32))


Q6K_MFMA_CHILD = """
import sys
import numpy as np
sys.path.insert(0, %r)
import oracle
from joshua_amd import capi, synth
from tests.test_gpu_matmul import q6k_integer_case, close, make_blocks
# exact integers: d = 1, random int8 scales per 16 elements, activation scale 1 per 32 elements
for (n, k, name) in [(300, 4096, "q6k_gemv_mfma_lds"), (1030, 12288, "q6k_gemv_mfma_cols")]:
    blocks, q, x = q6k_integer_case(n, k, 5, random_scales=True, small=40)
    want = x @ q.T
    assert np.abs(want).max() < 2 ** 24
    got = capi.Weight.upload(capi.Q6_K, blocks, n, k).matmul_t(1, x[None, :].astype(np.float32))
    assert capi.last_kernel() == name, capi.last_kernel()
    assert np.array_equal(got[0], want.astype(np.float32)), (n, k)
# ragged tiles, several tiles a workgroup (the ring of two slots wraps), one to three passes a row
for (n, k) in [(4096, 4096), (16 * 256 * 3 + 16 * 5 + 7, 4096), (2048 + 77, 8192), (4096, 12288), (1368 + 3, 12288), (257, 12288)]:
    blocks = make_blocks(capi.Q6_K, n, k, 31)
    lhs = synth.normal(32 + n %% 7, (1, k))
    got = capi.Weight.upload(capi.Q6_K, blocks, n, k).matmul_t(1, lhs)
    assert capi.last_kernel().startswith("q6k_gemv_mfma"), capi.last_kernel()
    assert close(got, oracle.matmul_t(capi.Q6_K, (1, k, n), lhs, blocks, avx2=oracle.have_avx2())), (n, k)
# a non-finite activation poisons the row, zeros stay zeros
lhs = synth.normal(9, (1, 4096)); lhs[0, 777] = np.inf
blocks = make_blocks(capi.Q6_K, 512, 4096, 33)
assert np.isnan(capi.Weight.upload(capi.Q6_K, blocks, 512, 4096).matmul_t(1, lhs)).all()
assert np.all(capi.Weight.upload(capi.Q6_K, blocks, 512, 4096).matmul_t(1, np.zeros((1, 4096), np.float32)) == 0.0)
print("q6k mfma ok")
"""


def test_q6k_matrix_core_gemv_at_every_shape_it_takes():
    """The Q6_K policy of the int8 matrix-core GEMV serves rows of 8192 and 12288 columns by default;
    JQ_Q6K_GEMV_MFMA=all sends it every shape it can take (rows of 4096 too, many tiles a workgroup), in a
    child process because the choice is read once: exact integer sums with random int8 group scales, ragged
    row counts, non-finite and zero activation rows."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, "-c", Q6K_MFMA_CHILD % root], env=dict(os.environ, JQ_Q6K_GEMV_MFMA="all"),
                         capture_output=True, text=True, timeout=110)
    assert res.returncode == 0 and "q6k mfma ok" in res.stdout, res.stdout + res.stderr


@pytest.mark.parametrize("k,n", [(4096, 4096), (4096, 8 * 600 + 5), (8192, 2048 + 77), (12288, 1368 + 3)])
def test_q8_0_one_row_over_4096_wide_row_groups(k, n):
    """Q8_0 rows of 4096, 8192 and 12288 with one activation row take the v_dot4 kernel (8-row steps,
    one to three column groups a row tile), with ragged last tiles."""
    blocks = make_blocks(capi.Q8_0, n, k, 41)
    lhs = synth.normal(42 + n % 7, (1, k))
    got = capi.Weight.upload(capi.Q8_0, blocks, n, k).matmul_t(1, lhs)
    assert close(got, oracle.matmul_t(capi.Q8_0, (1, k, n), lhs, blocks, avx2=oracle.have_avx2()))


def test_q8_0_dot4_integer_dot_products_are_bit_exact():
    """d = 1, integer activations whose 32-element blocks peak at 32639 (activation scale exactly 1)."""
    n, k = 4096 + 3, 4096
    rng = np.random.default_rng(6)
    q = np.zeros((n, k), np.int64)
    cols = rng.integers(0, k, size=(n, 12))
    q[np.arange(n)[:, None], cols] = rng.integers(-127, 128, size=(n, 12))
    x = rng.integers(-3000, 3001, size=k).astype(np.int64)
    peak = np.arange(0, k, 32) + int(rng.integers(0, 32))
    x[peak] = 32639 * rng.choice([-1, 1], size=k // 32)
    q[:, peak] = 0
    blocks = np.zeros((n, k // 32, 34), np.uint8)
    blocks[:, :, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blocks[:, :, 2:] = q.reshape(n, k // 32, 32).astype(np.int8).view(np.uint8)
    blocks = blocks.reshape(-1)
    assert np.array_equal(oracle.dequantize(capi.Q8_0, blocks).reshape(n, k), q.astype(np.float32))
    want = x @ q.T
    assert np.abs(want).max() < 2 ** 24
    got = capi.Weight.upload(capi.Q8_0, blocks, n, k).matmul_t(1, x[None, :].astype(np.float32))
    assert np.array_equal(got[0], want.astype(np.float32))


@pytest.mark.parametrize("qtype,m,k,n", [
    (capi.Q4_K, 1, 4096, 4096), (capi.Q4_K, 1, 2048, 512), (capi.Q4_K, 5, 4096, 512), (capi.Q4_K, 40, 1024, 256),
    (capi.Q6_K, 1, 4096, 4096), (capi.Q8_0, 1, 4096, 4096), (capi.Q4_K, 6, 512, 32768),
])
def test_non_finite_activations_show_in_the_result(qtype, m, k, n):
    """The fixed-point kernels scale every block of activations by its maximum; an inf or a NaN in a
    block must not be read as zeros: every output of that activation row comes out non-finite (as f32
    arithmetic would have it wherever the weights are not zero), the other rows are untouched."""
    blocks = make_blocks(qtype, n, k, 51)
    lhs = synth.normal(52, (m, k))
    want = oracle.matmul_t(qtype, (m, k, n), lhs, blocks, avx2=oracle.have_avx2())
    w = capi.Weight.upload(qtype, blocks, n, k)
    for bad in (np.inf, np.nan):
        x = lhs.copy()
        x[m - 1, k // 2 + 3] = bad
        got = w.matmul_t(m, x)
        assert not np.isfinite(got[m - 1]).any()
        if m > 1:
            assert close(got[:m - 1], want[:m - 1])


@pytest.mark.parametrize("qtype", [capi.Q6_K, capi.Q8_0, capi.Q2_K, capi.IQ2_XXS, capi.MXFP4])
@pytest.mark.parametrize("m,k,n", [(8, 12288, 1024), (16, 4096, 2100), (33, 4096, 2048 + 5), (48, 8192, 1100)])
def test_few_rows_against_a_large_matrix_take_the_int8_gemm(qtype, m, k, n):
    """8 to 63 activation rows against 8M weights or more: the int8 GEMM split over k, most of its
    activation-row tile empty; the partial sums are added in a fixed order (the same result on every call)."""
    blocks = make_blocks(qtype, n, k, 310 + m)
    lhs = synth.normal(311 + m, (m, k))
    w = capi.Weight.upload(qtype, blocks, n, k)
    got = w.matmul_t(m, lhs)
    name = {capi.Q6_K: "q6k", capi.Q8_0: "q8_0", capi.Q2_K: "q2k", capi.IQ2_XXS: "iq2xxs", capi.MXFP4: "mxfp4"}[qtype]
    assert capi.last_kernel() == name + "_gemm_i8+splitk"
    assert close(got, oracle.matmul_t(qtype, (m, k, n), lhs, blocks, avx2=True))
    assert np.array_equal(got, w.matmul_t(m, lhs))


@pytest.mark.parametrize("qtype,m,k,n", [(capi.Q5_1, 40, 2048, 1024), (capi.Q4_1, 33, 4096, 500), (capi.MXFP4, 20, 7168, 600),
                                         (capi.Q6_K, 512, 2048, 100), (capi.IQ2_XXS, 40, 5120, 300)])
def test_decoded_weights_gemm_split_over_k(qtype, m, k, n):
    """Products the int8 GEMM leaves to the GEMM over decoded weights: fewer than 64 rows against fewer than 8M
    weights, and many rows against few weight rows.  Its tiles alone leave compute units idle, so runs of
    chunks go to workgroups of their own and the partial sums are added in a fixed order (the same result on
    every call)."""
    blocks = synth.random_blocks(qtype, 300 + m, n * k) if qtype in capi.GENERIC_TYPES else make_blocks(qtype, n, k, 300 + m)
    lhs = synth.normal(301 + m, (m, k))
    w = capi.Weight.upload(qtype, blocks, n, k)
    got = w.matmul_t(m, lhs)
    assert close(got, oracle.matmul_t(qtype, (m, k, n), lhs, blocks))
    assert capi.last_kernel().startswith("gemm_decoded_mfma")
    assert np.array_equal(got, w.matmul_t(m, lhs))


@pytest.mark.parametrize("qtype", [capi.Q8_0, capi.Q2_K, capi.Q6_K, capi.IQ2_XXS, capi.MXFP4])
@pytest.mark.parametrize("m,k,n", [(17, 256, 64), (40, 768, 100), (130, 1024, 77), (64, 2048, 256)])
def test_many_rows_on_the_decoded_weights_gemm(qtype, m, k, n):
    """More than 16 activation rows of a format other than Q4_K: weights decoded to f16 in LDS, f16
    MFMA over two activation planes; ragged tiles in both directions."""
    blocks = make_blocks(qtype, n, k, 61)
    lhs = synth.normal(62 + m, (m, k))
    got = capi.Weight.upload(qtype, blocks, n, k).matmul_t(m, lhs)
    assert close(got, oracle.matmul_t(qtype, (m, k, n), lhs, blocks, avx2=oracle.have_avx2()))


@pytest.mark.parametrize("qtype", [capi.Q6_K, capi.MXFP4, capi.Q8_0])
def test_decoded_weights_gemm_on_views_at_odd_byte_offsets(qtype):
    """Experts of a stacked tensor start at any multiple of the block size (210, 17, 34 bytes): the
    kernel reads whole words from the word at or below each row chunk's first byte."""
    n, k, experts, m = 24, 512, 3, 33
    stacked_blocks = make_blocks(qtype, experts * n, k, 63)
    stacked = capi.Weight.upload(qtype, stacked_blocks, experts * n, k)
    lhs = synth.normal(64, (m, k))
    per = stacked_blocks.size // experts
    for e in range(experts):
        want = oracle.matmul_t(qtype, (m, k, n), lhs, stacked_blocks[e * per:(e + 1) * per], avx2=oracle.have_avx2())
        assert close(stacked.view(e * per, n, k).matmul_t(m, lhs), want)


def test_decoded_weights_gemm_activation_scales_span_many_orders():
    """256-element chunks of a row of very different magnitude, rows that are zero but for one value or
    for a stretch, and a row with a non-finite value."""
    n, k, m = 96, 2048, 48
    blocks = make_blocks(capi.Q6_K, n, k, 65)
    rng = np.random.default_rng(7)
    lhs = synth.normal(66, (m, k))
    lhs[0] *= (10.0 ** rng.integers(-6, 7, size=k // 256)).repeat(256).astype(np.float32)
    lhs[1, :] = 0.0
    lhs[1, 777] = -2.5
    lhs[2, 512:1024] = 0.0
    w = capi.Weight.upload(capi.Q6_K, blocks, n, k)
    assert close(w.matmul_t(m, lhs), oracle.matmul_t(capi.Q6_K, (m, k, n), lhs, blocks, avx2=oracle.have_avx2()))
    lhs[7, 300] = np.inf
    got = w.matmul_t(m, lhs)
    assert not np.isfinite(got[7]).any() and np.isfinite(got[8]).all()


def test_q4k_dot4_gemv_integer_dot_products_are_bit_exact():
    """4096-wide rows, one activation row: the v_dot4 kernel, activation range 32639 per 32-element
    sub-block."""
    n, k = 150, 4096
    blocks, q, x = q4k_integer_case(n, k, 7, group=32, big_value=32639, small=4000)
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(1, x[None, :].astype(np.float32))
    assert np.array_equal(got[0], (x @ q.T).astype(np.float32))


@pytest.mark.parametrize("k,n", [(8192, 1024), (12288, 1029), (12288, 4096), (8192, 2043), (8192, 4090), (12288, 3600)])
def test_q4k_dot4_gemv_long_rows(k, n):
    """Rows of 8192 and 12288, one activation row, 1024 weight rows or more: the v_dot4 kernel in steps
    of 8 rows x 4096 columns, or of 16 rows when that gives one tile per compute unit (3585 to 4096
    rows); row counts that leave a partial last step; wide-ranging activations."""
    blocks = make_blocks(capi.Q4_K, n, k, 51 + n)
    rng = np.random.default_rng(n)
    lhs = synth.normal(52 + n, (1, k))
    lhs[0] *= (10.0 ** rng.integers(-5, 1, size=k // 32)).repeat(32).astype(np.float32)
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    assert close(w.matmul_t(1, lhs), oracle.matmul_t(capi.Q4_K, (1, k, n), lhs, blocks, avx2=True))
    lhs[0, 5000] = np.nan
    assert np.isnan(w.matmul_t(1, lhs)).all()


@pytest.mark.parametrize("k,n", [(8192, 1040), (12288, 1040), (8192, 4000), (12288, 4096)])
def test_q4k_dot4_gemv_long_rows_integer_dot_products_are_bit_exact(k, n):
    blocks, q, x = q4k_integer_case(n, k, 9, group=32, big_value=32639, small=1000)
    want = x @ q.T
    assert np.abs(want).max() < 2 ** 24
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(1, x[None, :].astype(np.float32))
    assert np.array_equal(got[0], want.astype(np.float32))


@pytest.mark.parametrize("m,n", [(2, 1024), (5, 1030), (16, 14336), (16, 4097), (3, 5000), (8, 8190), (16, 4112),
                                 (17, 1024), (33, 4100), (64, 14336), (48, 1031), (130, 4096)])
def test_q4k_few_rows_over_4096_wide_rows(m, n):
    """2..64 activation rows over rows of 4096, 1024 weight rows or more: the int8 matrix-core kernel on
    the one-row kernel's weight stream, a pass per 16 activation rows; row counts with a partial last
    tile, one and several tiles a workgroup; wide-ranging activations, a zero row, a non-finite
    activation."""
    k = 4096
    blocks = make_blocks(capi.Q4_K, n, k, 61 + n)
    rng = np.random.default_rng(n + m)
    lhs = synth.normal(62 + n, (m, k))
    lhs[0] *= (10.0 ** rng.integers(-5, 2, size=k // 32)).repeat(32).astype(np.float32)
    lhs[m - 1, 1000:3000] = 0.0
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    got = w.matmul_t(m, lhs, np.full(m * n, 55.5, np.float32))
    assert close(got, oracle.matmul_t(capi.Q4_K, (m, k, n), lhs, blocks, avx2=True))
    one = w.matmul_t(1, lhs[1:2])
    assert close(one, got[1:2])
    lhs[1, 4000] = np.inf
    bad = w.matmul_t(m, lhs)
    assert np.isnan(bad[1]).all() and np.array_equal(bad[0], got[0])


@pytest.mark.parametrize("m,n", [(2, 1024), (16, 1040), (7, 4500), (37, 14336)])
def test_q4k_few_rows_over_4096_wide_rows_integer_dot_products_are_bit_exact(m, n):
    k = 4096
    blocks, q, x = q4k_integer_case(n, k, 13 + m, group=32, big_value=32639, small=1000)
    xs = np.stack([np.roll(x, 32 * i) * (1 if i % 2 == 0 else -1) for i in range(m)])
    want = xs @ q.T
    assert np.abs(want).max() < 2 ** 24
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(m, xs.astype(np.float32))
    assert np.array_equal(got, want.astype(np.float32))


@pytest.mark.parametrize("m", [17, 64, 200])
def test_q4k_gemm_integer_dot_products_are_bit_exact(m):
    """The same construction for the MFMA GEMM (m > 16): its activation range is 4193279
    per 256-element super-block; f16 products and f32 sums of integers below 2^24 are exact."""
    n, k = 150, 1024
    blocks, q, x = q4k_integer_case(n, k, 190 + m, group=256, big_value=4193279, small=4000)
    xs = np.stack([np.roll(x, 256 * (i % 4)) * (1 if i % 3 else -1) for i in range(m)])
    want = xs @ q.T
    assert np.abs(want).max() < 2 ** 24
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(m, xs.astype(np.float32))
    assert np.array_equal(got, want.astype(np.float32))


@pytest.mark.parametrize("m,k,n", [(17, 256, 64), (33, 512, 100), (128, 4096, 256), (130, 1024, 70),
                                   (512, 4096, 1024), (96, 12288, 128)])
def test_q4k_gemm_shapes(m, k, n):
    """Prefill GEMM: ragged activation rows (not multiples of 32/128), ragged weight rows
    (not multiples of 64), long rows."""
    blocks = make_blocks(capi.Q4_K, n, k, 41 + n)
    lhs = synth.normal(42 + m, (m, k))
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(m, lhs)
    assert close(got, oracle.matmul_t(capi.Q4_K, (m, k, n), lhs, blocks, avx2=True))


def test_q4k_gemm_activation_scales_span_many_orders():
    n, k, m = 96, 2048, 24
    blocks = make_blocks(capi.Q4_K, n, k, 79)
    rng = np.random.default_rng(6)
    lhs = synth.normal(80, (m, k))
    lhs[0] *= (10.0 ** rng.integers(-6, 7, size=k // 256)).repeat(256).astype(np.float32)
    lhs[1, :] = 0.0
    lhs[1, 777] = -2.5
    lhs[2, 512:1024] = 0.0
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(m, lhs)
    assert close(got, oracle.matmul_t(capi.Q4_K, (m, k, n), lhs, blocks, avx2=True))


def test_iq2xxs_fixture_matmul(golden_dir):
    # reference: src/iq2xxs.rs:758-804
    m, k, n = 3, 512, 7
    rhs = fixture_iq2xxs_rhs(golden_dir, k, n)
    lhs = ref_lhs(m, k, 7919)
    got = capi.Weight.upload(capi.IQ2_XXS, rhs, n, k).matmul_t(m, lhs)
    assert close(got, oracle.matmul_t(capi.IQ2_XXS, (m, k, n), lhs, rhs))


def test_mxfp4_pattern_matmul_exact():
    # reference: src/mxfp4.rs:351-388; small integers times powers of two sum exactly in f32
    m, k, n = 2, 64, 3
    rhs = mxfp4_pattern(n, k)
    lhs = (np.arange(m * k, dtype=np.float32) % np.float32(7.0) - np.float32(3.0)).reshape(m, k)
    got = capi.Weight.upload(capi.MXFP4, rhs, n, k).matmul_t(m, lhs)
    assert np.array_equal(got, oracle.matmul_t(capi.MXFP4, (m, k, n), lhs, rhs))


def test_matmul_assigns_into_dirty_destination():
    # reference: src/mxfp4.rs:390-416
    for qtype in capi.ALL_TYPES:
        n, k = 16, 512
        blocks = make_blocks(qtype, n, k, 3)
        w = capi.Weight.upload(qtype, blocks, n, k)
        lhs = synth.normal(4, (2, k))
        fresh = w.matmul_t(2, lhs, np.zeros(2 * n, np.float32))
        dirty = w.matmul_t(2, lhs, np.full(2 * n, 123.75, np.float32))
        assert np.array_equal(fresh, dirty)


def test_results_do_not_depend_on_how_rows_are_batched():
    """The reference requires bit-identical results whatever the thread count
    (src/kquant_dot.rs:916-929); here: a row's result must not depend on the
    launch it is part of."""
    for qtype in capi.ALL_TYPES:
        n, k = 64, 1024
        blocks = make_blocks(qtype, n, k, 5)
        _, bb = capi.block_geometry(qtype)
        row_bytes = bb * k // capi.block_geometry(qtype)[0]
        lhs = synth.normal(6, (3, k))
        w = capi.Weight.upload(qtype, blocks, n, k)
        full = w.matmul_t(3, lhs)
        for lo, hi in [(0, 1), (5, 16), (17, 64)]:
            part = w.view(lo * row_bytes, hi - lo, k).matmul_t(3, lhs)
            assert np.array_equal(part, full[:, lo:hi]), (qtype, lo, hi)
        again = w.matmul_t(3, lhs)
        assert np.array_equal(full, again)


def test_threads_sharing_the_default_stream_get_their_own_results():
    """Calls that prepare operands keep one scratch allocation per stream; host threads that share the
    stream enqueue their calls in turn, so every thread's result is the one it gets alone, bit for bit.
    The shapes take the 16-row int8 kernel, the Q4_K GEMM split over k and the decoded-weights GEMM, in
    sizes that make the scratch grow between calls."""
    import threading
    cases = []
    for i, (qtype, m, k, n) in enumerate([(capi.Q4_K, 16, 4096, 1024), (capi.Q4_K, 100, 2048, 300), (capi.Q6_K, 40, 1024, 200),
                                          (capi.Q4_K, 5, 4096, 2048)]):
        w = capi.Weight.upload(qtype, make_blocks(qtype, n, k, 500 + i), n, k)
        lhs = synth.normal(510 + i, (m, k))
        cases.append((w, m, lhs, w.matmul_t(m, lhs).copy()))
    failures = []

    def worker(tid):
        for it in range(6):
            w, m, lhs, want = cases[(tid + it) % len(cases)]
            got = w.matmul_t(m, lhs)
            if not np.array_equal(got, want):
                failures.append((tid, it))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, failures


@pytest.mark.parametrize("m,k,n", [(16, 12288, 4096), (3, 8192, 1030), (9, 16384, 1024), (40, 12288, 2050)])
def test_q4k_few_rows_over_rows_of_several_4096_column_groups(m, k, n):
    """Rows of 8192, 12288 and 16384: the 16-row kernel once per group of 4096 columns, the later launches
    adding to the result; a dirty destination, wide-ranging activations, a non-finite one."""
    blocks = make_blocks(capi.Q4_K, n, k, 71 + n)
    rng = np.random.default_rng(n + m)
    lhs = synth.normal(72 + n, (m, k))
    lhs[0] *= (10.0 ** rng.integers(-5, 2, size=k // 32)).repeat(32).astype(np.float32)
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    got = w.matmul_t(m, lhs, np.full(m * n, -7.25, np.float32))
    assert close(got, oracle.matmul_t(capi.Q4_K, (m, k, n), lhs, blocks, avx2=True))
    lhs[1, k - 5] = np.nan
    bad = w.matmul_t(m, lhs)
    assert np.isnan(bad[1]).all() and np.array_equal(bad[0], got[0])


def test_q4k_few_rows_over_long_rows_integer_dot_products_are_bit_exact():
    n, k, m = 1040, 12288, 7
    blocks, q, x = q4k_integer_case(n, k, 17, group=32, big_value=32639, small=300)
    xs = np.stack([np.roll(x, 32 * i) * (1 if i % 2 == 0 else -1) for i in range(m)])
    want = xs @ q.T
    assert np.abs(want).max() < 2 ** 24
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(m, xs.astype(np.float32))
    assert np.array_equal(got, want.astype(np.float32))


def test_q4k_few_rows_over_a_view_of_the_stacked_tensor():
    """The 16-row kernel over a view that starts some rows into the allocation (an expert slice)."""
    n, k, m = 3000, 4096, 9
    blocks = make_blocks(capi.Q4_K, n, k, 520)
    lhs = synth.normal(521, (m, k))
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    full = w.matmul_t(m, lhs)
    row_bytes = 144 * k // 256
    part = w.view(700 * row_bytes, 1500, k).matmul_t(m, lhs)
    assert np.array_equal(part, full[:, 700:2200])
    assert close(full, oracle.matmul_t(capi.Q4_K, (m, k, n), lhs, blocks, avx2=True))


def test_rejects_bad_shapes_and_leaves_dst_alone():
    # reference: src/quant_matmul.rs:597-608
    blocks = synth.quantize(capi.Q8_0, ref_weights(2, 256))
    w = capi.Weight.upload(capi.Q8_0, blocks, 2, 256)
    for m, x, dlen in [(1, np.zeros(100, np.float32), 2), (1, np.zeros(1, np.float32), 2),
                       (1, np.zeros(256, np.float32), 4), (2, np.zeros(256, np.float32), 4)]:
        dst = np.full(dlen, 5.0, np.float32)
        with pytest.raises(capi.JoshuaHipError):
            w.matmul_t(m, x, dst)
        assert np.all(dst == 5.0)
    with pytest.raises(capi.JoshuaHipError):  # k not a multiple of the block size
        capi.Weight.upload(capi.Q8_0, blocks, 2, 100)
    with pytest.raises(capi.JoshuaHipError):  # wrong block count for (n, k)
        capi.Weight.upload(capi.Q8_0, blocks, 4, 256)
    with pytest.raises(capi.JoshuaHipError):
        capi.Weight.upload(11, blocks, 2, 256)
    with pytest.raises(capi.JoshuaHipError):  # reference: src/mmap_tensor.rs:1002-1022 (out-of-bounds borrow declines)
        w.view(34 * 8, 2, 256)


def test_empty_problem_is_a_no_op():
    blocks = synth.quantize(capi.Q4_K, ref_weights(2, 256))
    w = capi.Weight.upload(capi.Q4_K, blocks, 2, 256)
    assert w.matmul_t(0, np.zeros(0, np.float32), np.zeros(0, np.float32)).size == 0


def test_embedding_gathers_decoded_rows():
    # reference: src/mmap_tensor.rs:140-167
    for qtype in (capi.Q4_K, capi.Q6_K, capi.Q8_0):
        n, k = 50, 512
        blocks = make_blocks(qtype, n, k, 9)
        w = capi.Weight.upload(qtype, blocks, n, k)
        ids = np.array([49, 0, 7, 7, 13], np.uint32)
        want = oracle.dequantize(qtype, blocks).reshape(n, k)[ids]
        assert np.array_equal(w.embedding(ids), want)
        with pytest.raises(capi.JoshuaHipError):
            w.embedding(np.array([50], np.uint32))


def test_expert_slices_alias_the_stacked_tensor():
    # reference: src/quantized_qwen3_moe.rs:596-631 (expert e at base + e*per_bytes)
    n_expert, n, k = 6, 24, 512
    blocks = make_blocks(capi.Q4_K, n_expert * n, k, 21)
    per = blocks.size // n_expert
    stacked = capi.Weight.upload(capi.Q4_K, blocks, n_expert * n, k)
    lhs = synth.normal(22, (1, k))
    for e in (0, 3, 5):
        ex = stacked.view(e * per, n, k)
        assert ex.device_ptr == stacked.device_ptr + e * per
        got = ex.matmul_t(1, lhs)
        assert close(got, oracle.matmul_t(capi.Q4_K, (1, k, n), lhs, blocks[e * per:(e + 1) * per]))


def test_try_matmul_fused_declines_like_the_reference():
    # reference: src/kquant_dot.rs:931-959
    import torch
    x = torch.zeros(256, device="cuda")
    y = torch.full((8,), 3.0, device="cuda")
    raw = torch.zeros(34 * 8 * 8, dtype=torch.uint8, device="cuda")
    assert not capi.try_matmul_fused(11, (1, 256, 2), x.data_ptr(), raw.data_ptr(), 34 * 16, y.data_ptr())
    assert not capi.try_matmul_fused(capi.Q8_0, (1, 256, 8), x.data_ptr(), raw.data_ptr(), 7, y.data_ptr())
    torch.cuda.synchronize()
    assert torch.all(y == 3.0)
    assert capi.try_matmul_fused(capi.Q8_0, (1, 256, 8), x.data_ptr(), raw.data_ptr(), 34 * 8 * 8, y.data_ptr())
    torch.cuda.synchronize()
    assert torch.all(y == 0.0)


def test_headline_shape_q4k_gemv():
    """Q4_K 14336 x 4096, M = 1 and 16, device pointers, against the AVX2 oracle."""
    import torch
    n, k = 14336, 4096
    blocks = make_blocks(capi.Q4_K, n, k, 102)
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    for m in (1, 16):
        lhs = synth.normal(202, (m, k))
        x = torch.from_numpy(lhs).cuda()
        y = torch.full((m, n), float("nan"), device="cuda")
        w.matmul_t_dev(m, x.data_ptr(), x.numel(), y.data_ptr(), y.numel(), torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        want = oracle.matmul_t(capi.Q4_K, (m, k, n), lhs, blocks, avx2=True)
        assert close(y.cpu().numpy(), want)


DOT4_CHILD = r"""
import sys, numpy as np
sys.path.insert(0, %r)
import oracle
from joshua_amd import capi, synth
from tests.test_gpu_matmul import q4k_integer_case, close
# exact integers: activation range 32639 per 32-element sub-block
n, k = 150, 4096
blocks, q, x = q4k_integer_case(n, k, 7, group=32, big_value=32639, small=4000)
import os
if os.environ["JQ_Q4K_DOT4"] != "0":
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(1, x[None, :].astype(np.float32))
    assert np.array_equal(got[0], (x @ q.T).astype(np.float32)), "integer case"
for (n, k) in [(14336, 4096), (100, 256), (4099, 1024), (33, 3840), (4099, 4096), (7, 4096)]:
    blocks = synth.normal_quantized(capi.Q4_K, 5 + n, n * k, 0.02)
    lhs = synth.normal(6 + k, (1, k))
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(1, lhs)
    assert close(got, oracle.matmul_t(capi.Q4_K, (1, k, n), lhs, blocks, avx2=oracle.have_avx2())), (n, k)
print("dot4 ok")
"""


@pytest.mark.parametrize("mode", ["regs", "0"])
def test_q4k_gemv_kernels_selected_by_environment(mode):
    """JQ_Q4K_DOT4 picks the one-row Q4_K kernel when the library first dispatches, so the non-default
    choices run in a child process: `regs` (v_dot4 with register prefetch, any row up to 4096) must be
    exact on the integer construction, `0` (the MFMA GEMV also for 4096-wide rows) skips that case;
    both within tolerance on random shapes (row counts that do not divide over the workgroups, short
    and 15-block rows)."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, JQ_Q4K_DOT4=mode)
    res = subprocess.run([sys.executable, "-c", DOT4_CHILD % root], env=env, capture_output=True, text=True, timeout=110)
    assert res.returncode == 0 and "dot4 ok" in res.stdout, res.stdout + res.stderr


# ---- the int8 matrix-core GEMV for one activation row (4096-wide rows, 8192 weight rows and more) ----

@pytest.mark.parametrize("n", [8192, 8192 + 5, 14336, 16 * 256 * 5 + 16 * 3 + 7, 65536 + 31])
def test_q4k_mfma_gemv_row_counts(n):
    """Row counts that give the workgroups equal and unequal numbers of tiles, more than four tiles a
    workgroup (the ring and the partial sums wrap) and a ragged last tile."""
    k = 4096
    blocks = make_blocks(capi.Q4_K, n, k, 300 + n % 97)
    lhs = synth.normal(301, (1, k))
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(1, lhs)
    assert capi.last_kernel() == "q4k_gemv_mfma_lds"
    assert close(got, oracle.matmul_t(capi.Q4_K, (1, k, n), lhs, blocks, avx2=oracle.have_avx2()))


def test_two_rows_against_a_mid_sized_matrix_run_the_one_row_kernel_twice():
    n, k = 4096 + 21, 4096
    blocks = make_blocks(capi.Q4_K, n, k, 305)
    lhs = synth.normal(306, (2, k))
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    got = w.matmul_t(2, lhs)
    assert capi.last_kernel() == "q4k_gemv_mfma_lds"
    assert close(got, oracle.matmul_t(capi.Q4_K, (2, k, n), lhs, blocks, avx2=oracle.have_avx2()))
    assert np.array_equal(got[1], w.matmul_t(1, lhs[1:])[0])


def test_q4k_mfma_gemv_integer_dot_products_are_bit_exact():
    """Activation range 32639 per 32-element sub-block, as in the v_dot4 kernel: the sums of the low-nibble
    sub-blocks come straight from the matrix cores, those of the high-nibble sub-blocks as
    (16 sum h X - 128 XS + 128 XS) / 16, all in integers."""
    n, k = 8192 + 48, 4096
    blocks, q, x = q4k_integer_case(n, k, 17, group=32, big_value=32639, small=4000)
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(1, x[None, :].astype(np.float32))
    assert capi.last_kernel() == "q4k_gemv_mfma_lds"
    assert np.array_equal(got[0], (x @ q.T).astype(np.float32))
    # every nibble value at every position of a chunk, negative and positive activations: random bytes
    rng = np.random.default_rng(3)
    raw = rng.integers(0, 256, size=n * 16 * 144, dtype=np.uint8).reshape(-1, 144)
    raw[:, 0:4] = np.frombuffer(np.float16([1.0, 1.0]).tobytes(), np.uint8)          # d = dmin = 1
    xi = rng.integers(-32639, 32640, size=k).astype(np.int64)
    xi[::32] = 32639                                                                 # scale exactly 1 per sub-block
    w = oracle.dequantize(capi.Q4_K, raw.reshape(-1)).reshape(n, k).astype(np.int64)  # integers: sc q - m
    want = w @ xi
    got = capi.Weight.upload(capi.Q4_K, raw.reshape(-1), n, k).matmul_t(1, xi[None, :].astype(np.float32))
    # sums reach 2^31: compare in f64 at f32 resolution of the per-block terms instead of bit for bit
    assert np.all(np.abs(got[0].astype(np.float64) - want) <= 2.0 ** -20 * np.abs(w).astype(np.float64) @ np.abs(xi))


def test_q4k_mfma_gemv_non_finite_and_wide_range_activations():
    n, k = 8192, 4096
    blocks = make_blocks(capi.Q4_K, n, k, 311)
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    rng = np.random.default_rng(9)
    lhs = synth.normal(312, (1, k))
    lhs[0] *= (10.0 ** rng.integers(-6, 7, size=k // 16)).repeat(16).astype(np.float32)
    # Magnitudes from 1e-6 to 1e6 inside one row: among 8192 rows some results cancel to a thousandth of
    # their terms, where no f32 summation order agrees with another to 1e-3 of the result.  The bound is
    # taken against the sum of the terms' magnitudes instead: 16-bit fixed point per 32 elements stays
    # below 2^-16 of it, and so must the kernel.
    wd = oracle.dequantize(capi.Q4_K, blocks).reshape(n, k).astype(np.float64)
    want, mag = wd @ lhs[0].astype(np.float64), np.abs(wd) @ np.abs(lhs[0].astype(np.float64))
    got = w.matmul_t(1, lhs)[0].astype(np.float64)
    assert np.all(np.abs(got - want) <= 2.0 ** -16 * mag)
    big = np.abs(want) >= 0.05 * mag          # rows without much cancellation: the usual bound
    assert big.sum() > n // 4 and np.all(np.abs(got - want)[big] <= TOL * np.abs(want)[big])
    for bad in (np.inf, -np.inf, np.nan):
        lhs = synth.normal(313, (1, k))
        lhs[0, 777] = bad
        got = w.matmul_t(1, lhs)
        assert capi.last_kernel() == "q4k_gemv_mfma_lds"
        assert np.all(np.isnan(got))            # every row has weights in that sub-block


def test_q4k_mfma_gemv_switched_off_by_environment():
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    child = ("import sys; sys.path.insert(0, %r)\n"
             "import numpy as np, oracle\nfrom joshua_amd import capi, synth\n"
             "n, k = 8192, 4096\nb = synth.normal_quantized(capi.Q4_K, 5, n * k, 0.02)\nx = synth.normal(6, (1, k))\n"
             "got = capi.Weight.upload(capi.Q4_K, b, n, k).matmul_t(1, x)\n"
             "assert capi.last_kernel() == 'q4k_gemv_dot4_lds', capi.last_kernel()\n"
             "want = oracle.matmul_t(capi.Q4_K, (1, k, n), x, b, avx2=oracle.have_avx2())\n"
             "assert np.all(np.abs(got - want) <= 1e-3 * np.maximum(np.abs(want), 1.0))\nprint('ok')\n") % root
    res = subprocess.run([sys.executable, "-c", child], env=dict(os.environ, JQ_Q4K_GEMV_MFMA="0"), capture_output=True,
                         text=True, timeout=110)
    assert res.returncode == 0 and "ok" in res.stdout, res.stdout + res.stderr


KERNEL_OF_SHAPE = [  # which kernel serves the shapes the benchmarks quote: (format, m, k, n) -> jq_last_kernel()
    (capi.Q4_K, 1, 4096, 14336, "q4k_gemv_mfma_lds"),        # headline
    (capi.Q4_K, 1, 4096, 4096, "q4k_gemv_mfma_lds"),
    (capi.Q4_K, 1, 4096, 1024, "q4k_gemv_dot4_lds"),         # fewer than 2048 weight rows
    (capi.Q4_K, 1, 12288, 4096, "q4k_gemv_mfma_cols"),       # a feed-forward down projection
    (capi.Q4_K, 1, 8192, 2048, "q4k_gemv_mfma_cols"),
    (capi.Q4_K, 1, 8192, 8192, "q4k_gemv_mfma_cols"),        # more than one row tile a workgroup
    (capi.Q4_K, 1, 2048, 768, "q4k_gemv_mfma_tile"),         # an expert's gate projection; a 2048-wide model's projections
    (capi.Q4_K, 1, 1024, 768, "q4k_gemv_mfma"),
    (capi.Q4_K, 1, 7168, 1536, "q4k_gemv_mfma_cols"),        # DeepSeek-V3's query down-projection
    (capi.Q4_K, 1, 16384, 7168, "q4k_gemv_mfma_cols"),       # its attention output projection
    (capi.Q4_K, 2, 2048, 768, "q4k_gemv_mfma"),
    (capi.Q4_K, 2, 4096, 4096, "q4k_gemv_mfma_lds"),         # two rows against a mid-sized matrix: the one-row kernel twice
    (capi.Q4_K, 2, 4096, 14336, "q4k_rows16_lds"),
    (capi.Q4_K, 16, 4096, 14336, "q4k_rows16_lds"),
    (capi.Q4_K, 16, 2048, 768, "q4k_stream_mfma"),
    (capi.Q4_K, 512, 4096, 14336, "q4k_gemm_i8"),           # 256 tiles of 256 x 112
    (capi.Q4_K, 128, 4096, 14336, "q4k_gemm_i8+splitk"),    # 224 tiles of 128 x 64, two splits
    (capi.Q4_K, 128, 4096, 4096, "q4k_gemm_i8+splitk"),     # 64 tiles of 128 x 64: split over k
    (capi.Q4_K, 512, 4096, 1024, "q4k_gemm_i8+splitk"),
    (capi.Q4_K, 128, 4096, 256, "q4k_gemm_mfma+splitk"),    # a small product: the f16 kernel
    (capi.Q8_0, 1, 4096, 4096, "q8_0_gemv_mfma_tile"),       # one tile of 16 rows a compute unit
    (capi.Q8_0, 1, 4096, 8192, "q8_0_gemv_dot4_lds"),
    (capi.Q6_K, 1, 12288, 4096, "q6k_gemv_mfma_cols"),      # a feed-forward down projection
    (capi.Q6_K, 1, 4096, 4096, "q6k_gemv_mfma_tile"),
    (capi.Q6_K, 1, 4096, 8192, "q6k_gemv_dot4_lds"),
    (capi.Q6_K, 1, 1024, 4096, "matmul_rows_staged"),
    (capi.Q6_K, 64, 4096, 1024, "q6k_gemm_i8+splitk"),
    (capi.Q6_K, 64, 2048, 256, "gemm_decoded_mfma+splitk"), # a small product: weights decoded in the workgroup
    (capi.Q6_K, 512, 12288, 4096, "q6k_gemm_i8+splitk"),    # a feed-forward down projection in prefill: 74 tiles of 256 x 112, three splits
    (capi.Q6_K, 32, 4096, 14336, "q6k_gemm_i8+splitk"),     # few rows against a large matrix
    (capi.Q8_0, 512, 4096, 14336, "q8_0_gemm_i8"),
    (capi.Q8_0, 16, 4096, 4096, "q8_0_gemm_i8+splitk"),
    (capi.Q8_0, 32, 2048, 2048, "gemm_decoded_mfma+splitk"),# few rows against a small matrix
    (capi.Q2_K, 512, 4096, 14336, "q2k_gemm_i8"),
    (capi.Q2_K, 64, 12288, 4096, "q2k_gemm_i8+splitk"),
    (capi.Q2_K, 1, 7680, 2048, "matmul_rows_staged"),
    (capi.Q2_K, 1, 4096, 14336, "q2k_gemv_mfma_lds"),
    (capi.MXFP4, 1, 7168, 2048, "matmul_rows_staged"),
    (capi.IQ2_XXS, 1, 7168, 2048, "matmul_rows_staged"),
]


@pytest.mark.parametrize("qtype,m,k,n,kernel", KERNEL_OF_SHAPE)
def test_kernel_chosen_for_a_shape(qtype, m, k, n, kernel):
    """The dispatcher's crossover points are measured constants; this pins what they select, so that a
    parity test named after a kernel keeps covering that kernel."""
    import torch
    blocks = make_blocks(qtype, n, k, 400)
    w = capi.Weight.upload(qtype, blocks, n, k)
    x = torch.zeros(m * k, device="cuda")
    y = torch.zeros(m * n, device="cuda")
    w.matmul_t_dev(m, x.data_ptr(), x.numel(), y.data_ptr(), y.numel(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert capi.last_kernel() == kernel


# ---- Q4_K, one activation row over rows of 2048 columns: one workgroup of 8 waves a tile of 16 rows ----

@pytest.mark.parametrize("n", [64, 100, 768 + 5, 4608, 16 * 300 + 9])
def test_q4k_mfma_gemv_over_rows_of_2048(n):
    """Whole and ragged last tiles, fewer and more tiles than compute units."""
    k = 2048
    blocks = make_blocks(capi.Q4_K, n, k, 500 + n % 89)
    lhs = synth.normal(501, (1, k))
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(1, lhs)
    assert capi.last_kernel() == "q4k_gemv_mfma_tile"
    assert close(got, oracle.matmul_t(capi.Q4_K, (1, k, n), lhs, blocks, avx2=oracle.have_avx2()))


@pytest.mark.parametrize("qtype,kernel", [(capi.Q6_K, "q6k_gemv_mfma_tile"), (capi.Q8_0, "q8_0_gemv_mfma_tile"),
                                          (capi.Q5_K, "q5k_gemv_mfma_tile")])
@pytest.mark.parametrize("n", [64, 512 + 7, 16 * 700 + 3])
def test_other_formats_one_row_over_rows_of_2048(qtype, kernel, n):
    """The same kernel over the Q6_K, Q8_0 and Q5_K policies (the attn_v and the output head of a 2048-wide model)."""
    k = 2048
    blocks = synth.random_blocks(qtype, 510 + n % 89, n * k) if qtype == capi.Q5_K else make_blocks(qtype, n, k, 510 + n % 89)
    lhs = synth.normal(511, (1, k))
    w = capi.Weight.upload(qtype, blocks, n, k)
    got = w.matmul_t(1, lhs)
    assert capi.last_kernel() == kernel
    assert close(got, oracle.matmul_t(qtype, (1, k, n), lhs, blocks, avx2=oracle.have_avx2()))
    lhs[0, 1234] = np.nan
    assert np.all(np.isnan(w.matmul_t(1, lhs)))


@pytest.mark.parametrize("qtype,kernel,n", [(capi.Q8_0, "q8_0_gemv_mfma_tile", 256), (capi.Q8_0, "q8_0_gemv_mfma_tile", 2048 + 7),
                                            (capi.Q8_0, "q8_0_gemv_mfma_tile", 4096), (capi.Q6_K, "q6k_gemv_mfma_tile", 2048),
                                            (capi.Q6_K, "q6k_gemv_mfma_tile", 4096 - 9)])
def test_q8_0_and_q6k_one_row_against_up_to_4096_rows_of_4096(qtype, kernel, n):
    """At most one tile of 16 rows a compute unit: 16 waves a tile, the whole matrix asked for at once."""
    k = 4096
    blocks = make_blocks(qtype, n, k, 520 + n % 89)
    lhs = synth.normal(521, (1, k))
    w = capi.Weight.upload(qtype, blocks, n, k)
    got = w.matmul_t(1, lhs)
    assert capi.last_kernel() == kernel
    assert close(got, oracle.matmul_t(qtype, (1, k, n), lhs, blocks, avx2=oracle.have_avx2()))
    lhs[0, 3000] = np.inf
    assert np.all(np.isnan(w.matmul_t(1, lhs)))


def test_q4k_mfma_gemv_over_rows_of_2048_integer_sums_and_odd_activations():
    n, k = 1024 + 48, 2048
    blocks, q, x = q4k_integer_case(n, k, 19, group=32, big_value=32639, small=4000)
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    got = w.matmul_t(1, x[None, :].astype(np.float32))
    assert capi.last_kernel() == "q4k_gemv_mfma_tile"
    assert np.array_equal(got[0], (x @ q.T).astype(np.float32))
    rng = np.random.default_rng(11)
    blocks = make_blocks(capi.Q4_K, n, k, 504)
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    lhs = synth.normal(502, (1, k))
    lhs[0] *= (10.0 ** rng.integers(-6, 7, size=k // 16)).repeat(16).astype(np.float32)
    wd = oracle.dequantize(capi.Q4_K, blocks).reshape(n, k).astype(np.float64)
    want, mag = wd @ lhs[0].astype(np.float64), np.abs(wd) @ np.abs(lhs[0].astype(np.float64))
    got = w.matmul_t(1, lhs)[0].astype(np.float64)
    assert np.all(np.abs(got - want) <= 2.0 ** -16 * mag)   # 16-bit fixed point per 32 elements
    for bad in (np.inf, -np.inf, np.nan):
        lhs = synth.normal(503, (1, k))
        lhs[0, 777] = bad
        assert np.all(np.isnan(w.matmul_t(1, lhs)))
    w.matmul_t(1, np.zeros((1, k), np.float32))
    assert np.array_equal(w.matmul_t(1, np.zeros((1, k), np.float32)), np.zeros((1, n), np.float32))


# ---- Q4_K, one activation row over rows of 17 to 64 super-blocks: the matrix-core GEMV in passes of 16 columns ----

@pytest.mark.parametrize("k,n", [(4352, 600), (5120, 512), (7168, 1536), (7168, 576 + 7), (8192 + 256, 1000), (12288 + 512, 4200),
                                 (13056, 4096 + 3), (16384, 7168), (16384, 4100), (16128, 4229)])
def test_q4k_mfma_gemv_in_passes_of_16_columns(k, n):
    """Two, three and four passes, a last pass of 1 to 16 columns, row counts that leave workgroups one tile
    more than others and a last tile part empty."""
    blocks = make_blocks(capi.Q4_K, n, k, 600 + n % 97)
    lhs = synth.normal(601 + k % 13, (1, k))
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(1, lhs)
    assert capi.last_kernel() == "q4k_gemv_mfma_cols"
    assert close(got, oracle.matmul_t(capi.Q4_K, (1, k, n), lhs, blocks, avx2=oracle.have_avx2()))


@pytest.mark.parametrize("k,n", [(5120, 530), (12032, 530), (16384, 4130)])
def test_q4k_mfma_gemv_in_passes_integer_sums_and_odd_activations(k, n):
    """Exact integer products (activation scale 1 in every 32-element group), then a row that spans many
    orders of magnitude and a non-finite value."""
    blocks, q, x = q4k_integer_case(n, k, 33 + k % 7, group=32, big_value=32639, small=300)
    want = x @ q.T
    assert np.abs(want).max() < 2 ** 24
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    got = w.matmul_t(1, x[None, :].astype(np.float32))
    assert capi.last_kernel() == "q4k_gemv_mfma_cols"
    assert np.array_equal(got[0], want.astype(np.float32))
    blocks = make_blocks(capi.Q4_K, n, k, 610)
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    rng = np.random.default_rng(k)
    lhs = synth.normal(611, (1, k))
    lhs[0] *= (10.0 ** rng.integers(-6, 7, size=k // 32)).repeat(32).astype(np.float32)
    # 16-bit fixed point per 32 elements: 2^-15 of a group's largest magnitude an element; held to 2^-14 of the
    # sum of the terms' magnitudes everywhere and to the usual bound where the terms do not cancel below a
    # twentieth of it
    wd = oracle.dequantize(capi.Q4_K, blocks).reshape(n, k).astype(np.float64)
    ref, mag = wd @ lhs[0].astype(np.float64), np.abs(wd) @ np.abs(lhs[0].astype(np.float64))
    err = np.abs(w.matmul_t(1, lhs)[0] - ref)
    assert np.all(err <= 2.0 ** -14 * mag)
    big = np.abs(ref) >= 0.05 * mag
    assert big.sum() > n // 8 and np.all(err[big] <= 1e-3 * np.abs(ref[big]))
    lhs[0, k - 5] = np.inf
    assert np.all(np.isnan(w.matmul_t(1, lhs)))


# ---- Q2_K, one activation row over 4096-wide rows: the int8 matrix-core GEMV ----

@pytest.mark.parametrize("n", [256, 1000, 4096, 14336, 16 * 256 * 5 + 16 * 3 + 7])
def test_q2k_mfma_gemv_row_counts(n):
    k = 4096
    blocks = make_blocks(capi.Q2_K, n, k, 500 + n % 89)
    lhs = synth.normal(501, (1, k))
    got = capi.Weight.upload(capi.Q2_K, blocks, n, k).matmul_t(1, lhs)
    assert capi.last_kernel() == "q2k_gemv_mfma_lds"
    assert close(got, oracle.matmul_t(capi.Q2_K, (1, k, n), lhs, blocks, avx2=oracle.have_avx2()))


def test_q2k_mfma_gemv_integer_dot_products_are_exact():
    """Random block bytes with d = dmin = 1 (integer weights sc q - m, every two-bit value at every position,
    every scale nibble) against integer activations whose 32-element groups have maximum magnitude 32639,
    so that their fixed-point scale is exactly 1: every per-group sum is an integer the kernel must get
    exactly; the f32 sum over a row's 256 groups is checked at 2^-20 of the terms' magnitudes."""
    n, k = 1024 + 48, 4096
    rng = np.random.default_rng(11)
    raw = rng.integers(0, 256, size=n * 16 * 84, dtype=np.uint8).reshape(-1, 84)
    raw[:, 80:84] = np.frombuffer(np.float16([1.0, 1.0]).tobytes(), np.uint8)
    xi = rng.integers(-32639, 32640, size=k).astype(np.int64)
    xi[::32] = 32639
    w = oracle.dequantize(capi.Q2_K, raw.reshape(-1)).reshape(n, k).astype(np.int64)
    want = w @ xi
    got = capi.Weight.upload(capi.Q2_K, raw.reshape(-1), n, k).matmul_t(1, xi[None, :].astype(np.float32))
    assert capi.last_kernel() == "q2k_gemv_mfma_lds"
    assert np.all(np.abs(got[0].astype(np.float64) - want) <= 2.0 ** -20 * (np.abs(w).astype(np.float64) @ np.abs(xi)))
    # one group at a time: a single non-zero activation group isolates its scale byte, field and plane sums
    for g in (0, 1, 7, 8, 9, 15, 100, 255):
        x1 = np.zeros(k, np.int64)
        x1[16 * g:16 * g + 16] = rng.integers(-32639, 32640, size=16)
        x1[16 * g] = 32639
        got = capi.Weight.upload(capi.Q2_K, raw.reshape(-1), n, k).matmul_t(1, x1[None, :].astype(np.float32))
        assert np.array_equal(got[0], (w @ x1).astype(np.float32)), g


def test_q2k_mfma_gemv_non_finite_activations():
    n, k = 512, 4096
    blocks = make_blocks(capi.Q2_K, n, k, 511)
    w = capi.Weight.upload(capi.Q2_K, blocks, n, k)
    for bad in (np.inf, np.nan):
        lhs = synth.normal(513, (1, k))
        lhs[0, 2000] = bad
        assert np.all(np.isnan(w.matmul_t(1, lhs)))


# ---- Q4_K and Q6_K with many activation rows on the int8 matrix cores ----

GEMM_I8_CHILD = r"""
import sys, numpy as np
sys.path.insert(0, %r)
import oracle
from joshua_amd import capi, synth
from tests.test_gpu_matmul import (q4k_integer_case, q6k_integer_case, q2k_integer_case, q8_0_integer_case,
                                   iq2xxs_integer_case, mxfp4_integer_case, q5k_integer_case, q4_0_integer_case,
                                   q3k_integer_case, q5_0_integer_case, q4_1_q5_1_integer_case, close)
FMT, KERNEL = {"q4k": (capi.Q4_K, "q4k_gemm_i8"), "q6k": (capi.Q6_K, "q6k_gemm_i8"), "q2k": (capi.Q2_K, "q2k_gemm_i8"),
               "q8_0": (capi.Q8_0, "q8_0_gemm_i8"), "iq2xxs": (capi.IQ2_XXS, "iq2xxs_gemm_i8"),
               "mxfp4": (capi.MXFP4, "mxfp4_gemm_i8"), "q5k": (capi.Q5_K, "q5k_gemm_i8"),
               "q4_0": (capi.Q4_0, "q4_0_gemm_i8"), "q3k": (capi.Q3_K, "q3k_gemm_i8"),
               "q5_0": (capi.Q5_0, "q5_0_gemm_i8"), "q4_1": (capi.Q4_1, "q4_1_gemm_i8"),
               "q5_1": (capi.Q5_1, "q5_1_gemm_i8")}[sys.argv[1]]
_synth = synth
class _Synth:  # the formats without a quantiser of normal weights get random blocks
    normal = staticmethod(_synth.normal)
    @staticmethod
    def normal_quantized(fmt, seed, count, sigma):
        return _synth.random_blocks(fmt, seed, count) if fmt in capi.GENERIC_TYPES else _synth.normal_quantized(fmt, seed, count, sigma)
synth = _Synth
AVX2 = oracle.have_avx2() and FMT not in capi.GENERIC_TYPES
# the same products split over k: the parts are summed in a fixed order
if __import__("os").environ.get("JQ_Q4K_GEMM_I8_SPLITS", "1") != "1":
    for (m, k, n) in [(40, 4096, 100), (300, 4096, 130), (64, 12288, 70)]:
        blocks = synth.normal_quantized(FMT, 15 + n, n * k, 0.02)
        lhs = synth.normal(16 + k, (m, k))
        w = capi.Weight.upload(FMT, blocks, n, k)
        got = w.matmul_t(m, lhs)
        assert capi.last_kernel() == KERNEL + "+splitk", (capi.last_kernel(), m, k, n)
        assert close(got, oracle.matmul_t(FMT, (m, k, n), lhs, blocks, avx2=AVX2)), (m, k, n)
        assert np.array_equal(got, w.matmul_t(m, lhs))
    print("gemm i8 ok")
    sys.exit(0)
# one to three tiles in either direction, ragged row and column counts
for (m, k, n) in [(17, 256, 64), (33, 512, 100), (64, 1024, 300), (100, 1024, 257), (130, 1024, 70), (200, 768, 1000),
                  (257, 512, 113), (300, 4096, 450), (512, 2048, 2048)]:
    blocks = synth.normal_quantized(FMT, 5 + n, n * k, 0.02)
    lhs = synth.normal(6 + k, (m, k))
    got = capi.Weight.upload(FMT, blocks, n, k).matmul_t(m, lhs)
    assert capi.last_kernel() == KERNEL, (capi.last_kernel(), m, k, n)
    assert close(got, oracle.matmul_t(FMT, (m, k, n), lhs, blocks, avx2=AVX2)), (m, k, n)
# exact integers: activation range 32639 per 32-element sub-block
n, k, m = 160, 2048, 40
if FMT == capi.Q4_K:
    blocks, q, x = q4k_integer_case(n, k, 23, group=32, big_value=32639, small=4000)
elif FMT == capi.Q6_K:  # every int8 scale value times q - 32, eight weights a row: sums below 2^24
    blocks, q, x = q6k_integer_case(n, k, 23, nonzero=8, random_scales=True, small=400)
elif FMT == capi.Q2_K:  # 4-bit scales and mins over sub-blocks of 16
    blocks, q, x = q2k_integer_case(n, k, 23)
elif FMT == capi.Q8_0:  # scales of 1/4 to 2 inside a run of 256: the common scale holds every weight exactly, the
    # sum 256 q d / D against the activations stays below 2^24
    blocks, q, x = q8_0_integer_case(n, k, 23)
elif FMT == capi.IQ2_XXS:  # dense integer weights up to 1333 against activations in multiples of 2^-8
    blocks, q, x = iq2xxs_integer_case(n, k, 23)
elif FMT == capi.MXFP4:  # dense weights in multiples of 1/8 under scales of 1/4 to 1 against activations in multiples of 2^-8
    blocks, q, x = mxfp4_integer_case(n, k, 23)
elif FMT == capi.Q5_K:  # the fifth bits
    blocks, q, x = q5k_integer_case(n, k, 23)
elif FMT == capi.Q4_0:  # scales of 1/2 to 4 inside a run of 256
    blocks, q, x = q4_0_integer_case(n, k, 23)
elif FMT == capi.Q3_K:  # every scale, field and third bit: dense integer weights up to 128
    blocks, q, x = q3k_integer_case(n, k, 23)
elif FMT == capi.Q5_0:  # fifth bits; scales of 1/2 to 4, some negative, inside a run of 256
    blocks, q, x = q5_0_integer_case(n, k, 23)
else:  # an f16 offset per block of 32
    blocks, q, x = q4_1_q5_1_integer_case(FMT, n, k, 23)
lhs = np.stack([np.roll(x, (32 if FMT in (capi.Q4_K, capi.Q6_K, capi.Q5_K) else 256) * i) for i in range(m)])
assert np.abs(lhs @ q.T).max() < {capi.IQ2_XXS: 2 ** 16, capi.Q3_K: 2 ** 16, capi.MXFP4: 2 ** 13}.get(FMT, 2 ** 24)
if FMT in (capi.Q8_0, capi.Q4_0, capi.Q5_0, capi.Q4_1, capi.Q5_1):  # per run of 256, 1024 times the sum is still an integer that f32 holds
    runs = np.einsum("mbe,nbe->mnb", lhs.reshape(m, -1, 256).astype(np.float64), q.reshape(n, -1, 256))
    assert np.abs(runs).max() < 2 ** 19
got = capi.Weight.upload(FMT, blocks, n, k).matmul_t(m, lhs.astype(np.float32))
assert capi.last_kernel() == KERNEL
assert np.array_equal(got, (lhs @ q.T).astype(np.float32)), "integer case"
# a row whose 16-element groups span twelve orders of magnitude, a row with a single non-zero element, a
# row with an empty stretch.  One 16-bit scale per 256 activations resolves each super-block relative to its
# largest magnitude: the wide row is held to 2^-12 of the sum of its terms' magnitudes on every output, and to
# the usual bound where the terms do not cancel below a twentieth of that sum.
n, k = 64, 4096
blocks = synth.normal_quantized(FMT, 77, n * k, 0.02)
rng = np.random.default_rng(5)
lhs = synth.normal(78, (40, k))
lhs[0] *= (10.0 ** rng.integers(-6, 7, size=k // 16)).repeat(16).astype(np.float32)
lhs[1, :] = 0.0
lhs[1, 1234] = 3.5
lhs[2, 512:1024] = 0.0
got = capi.Weight.upload(FMT, blocks, n, k).matmul_t(40, lhs)
assert capi.last_kernel() == KERNEL
want = oracle.matmul_t(FMT, (40, k, n), lhs, blocks, avx2=AVX2)
assert close(got[1:], want[1:]), "rows of ordinary range"
wd = oracle.dequantize(FMT, blocks).reshape(n, k).astype(np.float64)
x0 = lhs[0].astype(np.float64)
w0, mag = wd @ x0, np.abs(wd) @ np.abs(x0)
err = np.abs(got[0] - w0)
print("wide row: max err / mag = 2^%.1f" % np.log2((err / mag).max()))
assert np.all(err <= 2.0 ** -12 * mag), "wide range"
big = np.abs(w0) >= 0.05 * mag
assert big.sum() > n // 4 and np.all(err[big] <= 1e-3 * np.abs(w0[big])), "wide range, rows without cancellation"
# non-finite activations poison their own row only
lhs = synth.normal(79, (20, k))
lhs[3, 100] = np.inf
lhs[7, 4000] = np.nan
got = capi.Weight.upload(FMT, blocks, n, k).matmul_t(20, lhs)
want = oracle.matmul_t(FMT, (20, k, n), lhs, blocks, avx2=AVX2)
assert np.all(np.isnan(got[3])) and np.all(np.isnan(got[7]))
ok = np.ones(20, bool); ok[[3, 7]] = False
assert close(got[ok], want[ok])
print("gemm i8 ok")
"""


GEMM_I8_FORMATS = ["q4k", "q6k", "q2k", "q8_0", "iq2xxs", "mxfp4", "q5k", "q4_0", "q3k", "q5_0", "q4_1", "q5_1"]


# every format under the largest and the smallest workgroup shape; the two in between for the formats that differ
# in what the kernel holds in LDS (row meta of 48 or 80 bytes, a lookup table) or in how many planes it multiplies
@pytest.mark.parametrize("shape,fmt", [(s, f) for s in ("8,7", "2,4") for f in GEMM_I8_FORMATS] +
                         [("4,4", f) for f in ("q4k", "q6k", "q2k", "iq2xxs", "q4_1")] +
                         [("8,6", f) for f in ("q4k", "q6k", "q2k")])
def test_int8_gemm_small_shapes_in_a_child_process(shape, fmt):
    """The int8 GEMM serves products of 64 activation rows or more; with the thresholds lowered and the workgroup
    shape forced through the environment (read when the library first dispatches, hence the child process) every
    shape runs on small products: parity, ragged edges, exact integer sums, wide-range and non-finite
    activation rows."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, JQ_Q4K_GEMM_I8_MIN_TILES="1", JQ_Q4K_GEMM_I8_MIN_M="17", JQ_Q4K_GEMM_I8_SHAPE=shape, JQ_Q4K_GEMM_I8_SPLITS="1")
    res = subprocess.run([sys.executable, "-c", GEMM_I8_CHILD.replace("%r", repr(root), 1), fmt], env=env, capture_output=True, text=True, timeout=170)
    assert res.returncode == 0 and "gemm i8 ok" in res.stdout, res.stdout + res.stderr
    # forced splits of 2 and 4 (k of 4096 and 12288: 16 and 48 super-blocks)
    for splits in ("2", "4") if shape in ("8,7", "4,4") else ():
        env["JQ_Q4K_GEMM_I8_SPLITS"] = splits
        res = subprocess.run([sys.executable, "-c", GEMM_I8_CHILD.replace("%r", repr(root), 1), fmt], env=env, capture_output=True, text=True, timeout=170)
        assert res.returncode == 0 and "gemm i8 ok" in res.stdout, splits + res.stdout + res.stderr


def test_graph_captured_before_the_stream_scratch_grows_still_replays():
    """A 16-row Q4_K product (prepared activations in the stream's scratch buffer) is captured in a HIP graph;
    then a 512-row product on the same stream makes that buffer grow.  The old buffer is retired, not freed,
    so the graph, which names it, replays to the eager result every time, with eager work in between."""
    import torch
    n, k = 2048, 4096
    blocks = make_blocks(capi.Q4_K, n, k, 411)
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    big = capi.Weight.upload(capi.Q4_K, make_blocks(capi.Q4_K, 14336, k, 412), 14336, k)
    stream = torch.cuda.Stream()
    x16 = torch.from_numpy(synth.normal(413, (16, k))).cuda()
    y16 = torch.zeros(16 * n, device="cuda")
    xb = torch.from_numpy(synth.normal(414, (512, k))).cuda()
    yb = torch.zeros(512 * 14336, device="cuda")
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        w.matmul_t_dev(16, x16.data_ptr(), x16.numel(), y16.data_ptr(), y16.numel(), stream.cuda_stream)  # first use allocates
        stream.synchronize()
        want = y16.clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            w.matmul_t_dev(16, x16.data_ptr(), x16.numel(), y16.data_ptr(), y16.numel(), torch.cuda.current_stream().cuda_stream)
        cap_stream = stream.cuda_stream
        for rep in range(3):
            # a larger product on the stream the first call warmed up: its scratch buffer grows on the first pass
            big.matmul_t_dev(512, xb.data_ptr(), xb.numel(), yb.data_ptr(), yb.numel(), cap_stream)
            y16.fill_(float("nan"))
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y16, want), rep
    assert np.all(np.isfinite(yb[:14336].cpu().numpy()))
    del graph
    torch.cuda.synchronize()
    capi.stream_release(stream.cuda_stream)
    capi.stream_release(stream.cuda_stream)      # nothing left to free: not an error
    with torch.cuda.stream(stream):              # the stream serves calls again after a release
        w.matmul_t_dev(16, x16.data_ptr(), x16.numel(), y16.data_ptr(), y16.numel(), stream.cuda_stream)
        stream.synchronize()
    assert torch.equal(y16, want)


def _random_shapes(seed, count):
    rng = np.random.default_rng(seed)
    ms = [1, 2, 3, 4, 7, 8, 15, 16, 17, 24, 33, 64, 65, 100, 128, 200, 300]
    ks = [256, 512, 768, 1024, 2048, 4096, 8192, 12288]
    out = []
    while len(out) < count:
        m, k = int(rng.choice(ms)), int(rng.choice(ks))
        n = int(rng.integers(1, 20000)) if rng.random() < 0.3 else int(rng.integers(1, 3000))
        if m * k * n <= 1.2e9:
            out.append((m, k, n))
    return out


@pytest.mark.parametrize("m,k,n", _random_shapes(2024, 48))
def test_q4k_random_shapes_across_the_dispatcher(m, k, n):
    """Seeded random (rows, row length, weight rows) triples: whatever kernel the dispatcher picks for a shape
    (one-row kernels, 16-row passes, streaming, ring, int8 and f16 GEMMs, their ragged edges), the result
    holds the reference's bound against the oracle."""
    blocks = make_blocks(capi.Q4_K, n, k, 500 + (m * 31 + k * 7 + n) % 1000)
    lhs = synth.normal(600 + n % 97, (m, k))
    got = capi.Weight.upload(capi.Q4_K, blocks, n, k).matmul_t(m, lhs)
    want = oracle.matmul_t(capi.Q4_K, (m, k, n), lhs, blocks, avx2=oracle.have_avx2())
    assert close(got, want), (m, k, n, capi.last_kernel())


@pytest.mark.parametrize("qtype", [capi.Q8_0, capi.Q2_K, capi.Q6_K, capi.IQ2_XXS, capi.MXFP4])
@pytest.mark.parametrize("m,k,n", _random_shapes(77, 6))
def test_other_formats_random_shapes(qtype, m, k, n):
    n = min(n, 2500)
    blocks = make_blocks(qtype, n, k, 700 + qtype)
    lhs = synth.normal(800 + n % 89, (m, k))
    got = capi.Weight.upload(qtype, blocks, n, k).matmul_t(m, lhs)
    want = oracle.matmul_t(qtype, (m, k, n), lhs, blocks, avx2=oracle.have_avx2())
    assert close(got, want), (capi.TYPE_NAMES[qtype], m, k, n, capi.last_kernel())


def _large_random_shapes(seed, count):
    """Shapes of 8M weights or more, where every format's products of 8 rows and more take the int8 GEMM."""
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        m = int(rng.choice([8, 11, 16, 17, 31, 32, 33, 63, 64, 100, 130, 257, 300]))
        k = int(rng.choice([2048, 4096, 5120, 7168, 8192]))
        n = int(rng.integers((8 << 20) // k + 1, 3 * (8 << 20) // k))
        out.append((m, k, n))
    return out


@pytest.mark.parametrize("qtype", [t for t in capi.ALL_TYPES + capi.GENERIC_TYPES if t != capi.Q4_K])
@pytest.mark.parametrize("m,k,n", _large_random_shapes(78, 4))
def test_every_format_on_the_int8_gemm_at_random_large_shapes(qtype, m, k, n):
    """Seeded random shapes against large matrices: whatever tile shape and split over k the estimate picks
    (32 x 64 tiles up to 32 rows, 128 x 64, 256 x 96 or 256 x 112 beyond), ragged in both directions, the result
    holds the reference's bound against the oracle on a sample of the weight rows."""
    blocks = synth.random_blocks(qtype, 710 + qtype, n * k) if qtype in capi.GENERIC_TYPES else make_blocks(qtype, n, k, 710 + qtype)
    lhs = synth.normal(810 + n % 89, (m, k))
    got = capi.Weight.upload(qtype, blocks, n, k).matmul_t(m, lhs)
    assert "gemm_i8" in capi.last_kernel(), capi.last_kernel()
    rows = np.unique(np.concatenate([np.arange(130), np.arange(n - 130, n), np.arange(130, n - 130, 7)[:240]]))
    sub = blocks.reshape(n, -1)[rows].reshape(-1)
    want = oracle.matmul_t(qtype, (m, k, rows.size), lhs, sub, avx2=oracle.have_avx2() and qtype not in capi.GENERIC_TYPES)
    assert close(got[:, rows], want), (capi.TYPE_NAMES[qtype], m, k, n, capi.last_kernel())
