"""Q4_0, Q4_1, Q5_0, Q5_1, Q3_K, Q5_K: the formats the reference serves through the canonical decode
plus its 8-lane dot (src/quant_matmul.rs:228-248).  The oracle's decode against an independent numpy
decode written from the block definitions, exhaustive sweeps of every field, the matmul against a
float64 product of the decoded weights.  Host only."""
import numpy as np
import pytest

import oracle
from joshua_amd import synth
from tests import np_decode

NP = {2: np_decode.q4_0, 3: np_decode.q4_1, 6: np_decode.q5_0, 7: np_decode.q5_1, 11: np_decode.q3_k, 13: np_decode.q5_k}
GEOM = {2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 11: (256, 110), 13: (256, 176)}
F16_ONE = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)


@pytest.mark.parametrize("qtype", oracle.GENERIC_TYPES)
def test_geometry(qtype):
    assert oracle.block_geometry(qtype) == GEOM[qtype]     # reference: src/gguf_ext.rs:487-500


@pytest.mark.parametrize("qtype", oracle.GENERIC_TYPES)
def test_decode_equals_independent_decode_on_random_bytes(qtype):
    elems, nbytes = GEOM[qtype]
    rng = np.random.default_rng(qtype)
    raw = rng.integers(0, 256, size=300 * nbytes, dtype=np.uint8)
    blk = raw.reshape(-1, nbytes)
    for off in {2: (0,), 3: (0, 2), 6: (0,), 7: (0, 2), 11: (108,), 13: (0, 2)}[qtype]:
        blk[:, off + 1] &= 0x7B        # finite f16 scales
    a, b = oracle.dequantize(qtype, raw), NP[qtype](raw)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    r = synth.random_blocks(qtype, 3, elems * 64)
    assert np.array_equal(oracle.dequantize(qtype, r).view(np.uint32), NP[qtype](r).view(np.uint32))


def test_q4_and_q5_nibble_and_fifth_bit_maps():
    """Every nibble value at every position, every fifth bit: element j rides on the low nibble of byte
    j, element j + 16 on the high nibble, bit e of qh is the fifth bit of element e
    (vendor/candle-metal-kernels/src/metal_src/quantized.metal:6482-6567)."""
    for qtype, hdr, has_m, has_h in ((2, 2, False, False), (3, 4, True, False), (6, 6, False, True), (7, 8, True, True)):
        nbytes = GEOM[qtype][1]
        for pos in range(32):
            for val in range(32 if has_h else 16):
                b = np.zeros(nbytes, np.uint8)
                b[0:2] = F16_ONE
                if has_m:
                    b[2:4] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
                b[hdr + pos % 16] = (val & 15) << (4 * (pos // 16))
                if has_h and val >= 16:
                    word = np.uint32(1) << np.uint32(pos)
                    b[hdr - 4:hdr] = np.frombuffer(word.tobytes(), np.uint8)
                y = oracle.dequantize(qtype, b)
                zero = {2: -8.0, 3: 0.5, 6: -16.0, 7: 0.5}[qtype]
                want = np.full(32, zero, np.float32)
                want[pos] = zero + val
                assert np.array_equal(y, want), (qtype, pos, val)


def test_q3_k_fields():
    """All 64 scale codes at all 16 scale slots, all 8 three-bit values at sampled positions
    (vendor/candle-metal-kernels/src/metal_src/quantized.metal:6597-6623)."""
    for slot in range(16):
        for code in range(64):
            b = np.zeros(110, np.uint8)
            b[108:110] = F16_ONE
            b[0:32] = 0xFF                       # third bits set: q = low two bits
            b[32:96] = 0x55                      # every 2-bit field = 1
            b[96 + slot % 8] = (code & 15) << (4 * (slot // 8))
            b[104 + slot % 4] = (code >> 4) << (2 * (slot // 4))
            y = oracle.dequantize(11, b)
            want = np.full(256, -32.0, np.float32)
            want[16 * slot:16 * slot + 16] = code - 32
            assert np.array_equal(y, want), (slot, code)
    for e in list(range(0, 256, 7)) + [255]:
        h, t, l = e // 128, (e % 128) // 32, e % 32
        for v in range(8):                       # v = low two bits + 4 * third bit -> value v - 4
            b = np.zeros(110, np.uint8)
            b[108:110] = F16_ONE
            b[96:104] = 0x11                     # low nibbles 1 ...
            b[104:108] = 0xAA                    # ... high bits 2: every scale 33 -> factor 1
            b[32 + 32 * h + l] = (v & 3) << (2 * t)
            b[l] = (v >> 2) << (4 * h + t)
            y = oracle.dequantize(11, b)
            want = np.full(256, -4.0, np.float32)
            want[e] = v - 4
            assert np.array_equal(y, want), (e, v)


def test_q5_k_fields():
    """All (scale, min) codes of the 6-bit packing through Q5_K, all 32 five-bit values at sampled
    positions (vendor/candle-metal-kernels/src/metal_src/quantized.metal:6649-6670)."""
    for j in range(8):
        for code in (0, 1, 31, 32, 45, 63):
            for mcode in (0, 7, 63):
                b = np.zeros(176, np.uint8)
                b[0:2] = F16_ONE
                b[2:4] = F16_ONE
                s = b[4:16]
                if j < 4:
                    s[j], s[j + 4] = code, mcode
                else:
                    s[j + 4] = (code & 15) | ((mcode & 15) << 4)
                    s[j - 4] |= (code >> 4) << 6
                    s[j] |= (mcode >> 4) << 6
                b[48:] = 0x11                    # every nibble 1
                y = oracle.dequantize(13, b).reshape(8, 32)
                assert np.all(y[j] == code - mcode), (j, code, mcode)
    for e in list(range(0, 256, 5)) + [255]:
        j, l = e // 32, e % 32
        for v in (0, 1, 15, 16, 21, 31):
            b = np.zeros(176, np.uint8)
            b[0:2] = F16_ONE
            b[4:8] = 1                           # scales 0..3 = 1
            b[12:16] = 1                         # scales 4..7 = 1 (low nibble), mins 0
            b[48 + 32 * (j // 2) + l] = (v & 15) << (4 * (j & 1))
            b[16 + l] = (v >> 4) << j
            y = oracle.dequantize(13, b)
            want = np.zeros(256, np.float32)
            want[e] = v
            assert np.array_equal(y, want), (e, v)


@pytest.mark.parametrize("qtype", oracle.GENERIC_TYPES)
@pytest.mark.parametrize("m,k,n", [(1, 256, 40), (3, 512, 13), (5, 768, 9)])
def test_matmul_equals_f64_product_of_decoded_weights(qtype, m, k, n):
    blocks = synth.random_blocks(qtype, 5, n * k)
    lhs = synth.normal(6, (m, k))
    w = oracle.dequantize(qtype, blocks).reshape(n, k).astype(np.float64)
    want = lhs.astype(np.float64) @ w.T
    got = oracle.matmul_t(qtype, (m, k, n), lhs, blocks)
    assert np.all(np.abs(got - want) <= 1e-3 * np.maximum(np.abs(want), 1.0))   # src/kquant_dot.rs:853
    if oracle.have_avx2():
        for threads in (1, 3):
            fast = oracle.matmul_t(qtype, (m, k, n), lhs, blocks, avx2=True, threads=threads)
            assert np.array_equal(fast.view(np.uint32), got.view(np.uint32))


@pytest.mark.parametrize("qtype", oracle.GENERIC_TYPES)
def test_shape_errors(qtype):
    elems, nbytes = GEOM[qtype]
    blocks = synth.random_blocks(qtype, 7, 2 * 256)
    with pytest.raises(oracle.OracleError):
        oracle.matmul_t(qtype, (1, 256 + elems // 2, 2), np.zeros((1, 256 + elems // 2), np.float32), blocks)
    with pytest.raises(oracle.OracleError):
        oracle.matmul_t(qtype, (1, 256, 3), np.zeros((1, 256), np.float32), blocks)
