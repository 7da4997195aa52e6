"""Pins the CPU oracle's block decoders: the reference's own golden vectors and
closed-form cases (reference tests: src/iq2xxs.rs:712-903, src/mxfp4.rs:281-458),
an independent numpy decode on random byte patterns, and exhaustive sweeps of
the packed fields."""
import hashlib
import os
import re

import numpy as np
import pytest

import oracle
from tests import np_decode

RNG = np.random.default_rng(20240611)


def test_block_geometry_matches_gguf_table():
    # reference: src/gguf_ext.rs:483-512
    assert oracle.block_geometry(oracle.Q8_0) == (32, 34)
    assert oracle.block_geometry(oracle.Q2_K) == (256, 84)
    assert oracle.block_geometry(oracle.Q4_K) == (256, 144)
    assert oracle.block_geometry(oracle.Q6_K) == (256, 210)
    assert oracle.block_geometry(oracle.IQ2_XXS) == (256, 66)
    assert oracle.block_geometry(oracle.MXFP4) == (32, 17)
    with pytest.raises(oracle.OracleError):
        oracle.block_geometry(15)


def test_f16_conversion_every_code():
    codes = np.arange(65536, dtype=np.uint16)
    want = codes.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_to_f32(int(c)) for c in codes], dtype=np.float32)
    assert np.array_equal(want.view(np.uint32)[~np.isnan(want)], got.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(got[np.isnan(want)]).all()


# ---- IQ2_XXS: llama.cpp golden vectors held by the reference -------------------

def test_iq2xxs_dequant_matches_llamacpp_golden(golden_dir):
    blocks = np.fromfile(os.path.join(golden_dir, "iq2xxs_blocks.bin"), dtype=np.uint8)
    want = np.loadtxt(os.path.join(golden_dir, "iq2xxs_ref.txt"), dtype=np.float64)
    assert blocks.size == 264 and want.size == 1024
    got = oracle.dequantize(oracle.IQ2_XXS, blocks)
    assert np.all(np.abs(got - want) <= 1e-6 * np.maximum(np.abs(want), 1.0))


def test_iq2xxs_grid_checksum_and_sign_rule():
    grid = oracle.iq2xxs_grid_table()
    assert set(np.unique(grid)) == {8, 25, 43}
    assert hashlib.sha256(grid.tobytes()).hexdigest() == \
        "05826b5d3e472a3a78f196be62ac78acf81df0f909626e12ab9fa2a5d490dd54"
    for i in range(128):
        s = oracle.lib().orc_iq2xxs_signs(i)
        assert s & 127 == i and bin(s).count("1") % 2 == 0


def test_iq2xxs_grid_equals_reference_table_when_present():
    path = "/root/reference/src/iq2xxs.rs"
    if not os.path.exists(path):
        pytest.skip("reference checkout not present on this machine")
    src = open(path).read()
    i = src.index("pub const IQ2XXS_GRID")
    vals = [int(v, 16) for v in re.findall(r"0x([0-9a-f]{16})", src[i:src.index("];", i)])]
    ref = np.array(vals, dtype="<u8").view(np.uint8).reshape(256, 8)
    assert np.array_equal(ref, oracle.iq2xxs_grid_table())


def test_iq2xxs_bound_and_finite():
    # reference: src/iq2xxs.rs:742-756, 890-902
    blk = np.zeros(66, np.uint8)
    blk[1] = 0x3C  # d = 1.0
    assert np.isfinite(oracle.dequantize(oracle.IQ2_XXS, blk)).all()
    blk[2:] = 0xFF
    out = oracle.dequantize(oracle.IQ2_XXS, blk)
    assert np.all(np.abs(out) <= 43.0 * 0.25 * 15.5 + 1e-6)
    assert np.abs(out).max() == pytest.approx(43.0 * 0.25 * 15.5)


def test_iq2xxs_random_bytes_match_independent_decode():
    raw = RNG.integers(0, 256, size=66 * 64, dtype=np.uint8)
    raw.reshape(-1, 66)[:, 1] &= 0x3F  # keep the f16 scale finite
    want = np_decode.iq2_xxs(raw, oracle.iq2xxs_grid_table())
    assert np.array_equal(oracle.dequantize(oracle.IQ2_XXS, raw), want)


# ---- MXFP4: the reference's closed-form cases ----------------------------------

def test_mxfp4_e8m0_powers_of_two():
    assert oracle.e8m0(127) == 1.0 and oracle.e8m0(128) == 2.0
    assert oracle.e8m0(126) == 0.5 and oracle.e8m0(130) == 8.0
    tiny = oracle.e8m0(0)
    assert tiny > 0 and np.float32(tiny).view(np.uint32) == 0x00400000
    assert oracle.e8m0(0xFF) is None
    for e in range(1, 255):
        assert oracle.e8m0(e) == 2.0 ** (e - 127)


def _mx(e, qs):
    return np.array([e] + list(qs), dtype=np.uint8)


def test_mxfp4_split_half_nibble_order():
    qs = [0] * 16
    qs[0] = 0x7 | (0x1 << 4)
    out = oracle.dequantize(oracle.MXFP4, _mx(127, qs))
    assert out[0] == 6.0 and out[16] == 0.5 and out[1] == 0.0


def test_mxfp4_scale_and_table_and_nan_scale():
    qs = [0] * 16
    qs[3] = 0xF
    assert oracle.dequantize(oracle.MXFP4, _mx(129, qs))[3] == -24.0
    out = oracle.dequantize(oracle.MXFP4, _mx(127, range(16)))
    table = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]
    assert list(out[:16]) == table
    assert np.signbit(out[8])
    assert np.all(oracle.dequantize(oracle.MXFP4, _mx(0xFF, [0xFF] * 16)) == 0.0)


def test_mxfp4_random_bytes_match_independent_decode():
    raw = RNG.integers(0, 256, size=17 * 512, dtype=np.uint8)
    raw.reshape(-1, 17)[::7, 0] = 0xFF
    raw.reshape(-1, 17)[1::7, 0] = 0
    assert np.array_equal(oracle.dequantize(oracle.MXFP4, raw), np_decode.mxfp4(raw))


# ---- k-quants: independent decode + exhaustive field sweeps --------------------

def _finite_f16(raw, block, offsets):
    v = raw.reshape(-1, block)
    for off in offsets:
        v[:, off + 1] &= 0x7B  # clear the top exponent bits: no inf/nan scales
    return raw


@pytest.mark.parametrize("qtype,block,f16_at,fn", [
    (oracle.Q8_0, 34, (0,), np_decode.q8_0),
    (oracle.Q2_K, 84, (80, 82), np_decode.q2_k),
    (oracle.Q4_K, 144, (0, 2), np_decode.q4_k),
    (oracle.Q6_K, 210, (208,), np_decode.q6_k),
])
def test_kquant_random_bytes_match_independent_decode(qtype, block, f16_at, fn):
    raw = _finite_f16(RNG.integers(0, 256, size=block * 97, dtype=np.uint8), block, f16_at)
    got, want = oracle.dequantize(qtype, raw), fn(raw)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_q4k_every_scale_code_and_nibble():
    """d = dmin = 1: element value is sc*q - m; sweep every 6-bit code in every
    pair slot with every nibble value, against the packing rule stated
    directly (reference: src/kquant_dot.rs:108-118)."""
    for j in range(8):
        for code in range(64):
            sc, mn = code, 63 - code
            s = np.zeros(12, np.uint8)
            if j < 4:
                s[j], s[j + 4] = sc, mn
            else:
                s[j + 4] = (sc & 0xF) | ((mn & 0xF) << 4)
                s[j - 4] |= (sc >> 4) << 6
                s[j] |= (mn >> 4) << 6
            blk = np.zeros(144, np.uint8)
            blk[1] = blk[3] = 0x3C
            blk[4:16] = s
            q = (np.arange(32) + code) % 16
            c, r = j // 2, j % 2
            blk[16 + 32 * c:16 + 32 * c + 32] = (q << 4) if r else q
            out = oracle.dequantize(oracle.Q4_K, blk).reshape(8, 32)
            assert np.array_equal(out[j], sc * q.astype(np.float32) - mn)
            others = np.delete(out, j, axis=0)
            assert np.all(others == 0.0)


def test_q2k_every_scale_and_field():
    for g in range(16):
        for s in range(256):
            blk = np.zeros(84, np.uint8)
            blk[81] = blk[83] = 0x3C
            blk[g] = s
            sgrp, j = g // 8, g % 8
            q = (np.arange(16) + s) % 4
            lo = 16 + 32 * sgrp + (16 if j % 2 else 0)
            blk[lo:lo + 16] = q << (2 * (j // 2))
            out = oracle.dequantize(oracle.Q2_K, blk).reshape(16, 16)
            assert np.array_equal(out[g], (s & 0xF) * q.astype(np.float32) - (s >> 4))


def test_q6k_every_value_and_position():
    for e in range(256):
        for q in (0, 1, 31, 32, 33, 63):
            blk = np.zeros(210, np.uint8)
            blk[209] = 0x3C                      # d = 1
            blk[192:208] = 1                     # all scales 1
            blk[192 + e // 16] = np.uint8(np.int8(-3))
            h, r = e // 128, e % 128
            l, t = r % 32, r // 32
            blk[64 * h + l + 32 * (t & 1)] |= (q & 0xF) << (4 if t >= 2 else 0)
            blk[128 + 32 * h + l] |= (q >> 4) << (2 * t)
            out = oracle.dequantize(oracle.Q6_K, blk)
            assert out[e] == -3.0 * (q - 32)
            rest = np.delete(out, e).reshape(-1)
            grp = np.delete(np.arange(256), e) // 16 == e // 16
            assert np.all(rest[grp] == -3.0 * -32) and np.all(rest[~grp] == -32.0)


def test_q8_0_closed_form():
    blk = np.zeros(34, np.uint8)
    blk[0:2] = np.array([0.25], np.float16).view(np.uint8)
    blk[2:] = np.arange(-16, 16, dtype=np.int8).view(np.uint8)
    assert np.array_equal(oracle.dequantize(oracle.Q8_0, blk), np.arange(-16, 16, dtype=np.float32) * 0.25)


def test_dequantize_rejects_partial_blocks():
    # reference: src/mxfp4.rs:452-457, src/iq2xxs.rs:422-429
    with pytest.raises(oracle.OracleError):
        oracle.dequantize(oracle.MXFP4, np.zeros(20, np.uint8))
    with pytest.raises(oracle.OracleError):
        oracle.dequantize(oracle.IQ2_XXS, np.zeros(65, np.uint8))
    assert oracle.dequantize(oracle.MXFP4, np.zeros(34, np.uint8)).size == 64
