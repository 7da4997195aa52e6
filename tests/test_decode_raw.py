"""decode_raw_to_f32 (reference: src/quant_matmul.rs:36-103): the oracle against numpy written from the
formats' definitions, then the device entry point against the oracle.  F16 is pinned by numpy's own
float16 conversion, Q8_K by d * q in numpy; Q8_1 follows ggml's published layout (parity unpinned: the
reference hands it to candle-core 0.11, which is not in the tree)."""
import os

import numpy as np
import pytest

import oracle


def q8_k_blocks(rng, n):
    raw = np.zeros((n, 292), np.uint8)
    d = rng.normal(size=n).astype(np.float32) * 0.01
    q = rng.integers(-128, 128, size=(n, 256), dtype=np.int8)
    raw[:, :4] = d.view(np.uint8).reshape(n, 4)
    raw[:, 4:260] = q.view(np.uint8)
    raw[:, 260:] = rng.integers(0, 256, size=(n, 32), dtype=np.uint8)  # bsums: not part of the decode
    return raw.reshape(-1), (d[:, None] * q.astype(np.float32)).reshape(-1)


def q8_1_blocks(rng, n):
    raw = np.zeros((n, 36), np.uint8)
    d = (rng.normal(size=n) * 0.01).astype(np.float16)
    q = rng.integers(-128, 128, size=(n, 32), dtype=np.int8)
    raw[:, :2] = d.view(np.uint8).reshape(n, 2)
    raw[:, 2:4] = rng.integers(0, 256, size=(n, 2), dtype=np.uint8)  # s: not part of the decode
    raw[:, 4:] = q.view(np.uint8)
    return raw.reshape(-1), (d.astype(np.float32)[:, None] * q.astype(np.float32)).reshape(-1)


def cases():
    rng = np.random.default_rng(3)
    h = np.concatenate([rng.normal(size=1000).astype(np.float16),
                        np.array([0.0, -0.0, 65504.0, -65504.0, 6e-8, 6.1e-5, np.inf, -np.inf], np.float16)])
    yield 1, h.view(np.uint8), h.size, h.astype(np.float32)
    raw, want = q8_k_blocks(rng, 7)
    yield 15, raw, 7 * 256, want
    raw, want = q8_1_blocks(rng, 9)
    yield 9, raw, 9 * 32, want


def test_oracle_plain_types_against_numpy():
    for dtype, raw, elems, want in cases():
        got = oracle.decode_raw_to_f32(dtype, raw, elems)
        assert np.array_equal(got, want), dtype
    nan = np.array([np.nan], np.float16)
    assert np.isnan(oracle.decode_raw_to_f32(1, nan.view(np.uint8), 1)[0])


def test_oracle_none_and_errors():
    assert oracle.decode_raw_to_f32(0, np.zeros(16, np.uint8), 4) is None          # F32: the caller's reader
    assert oracle.decode_raw_to_f32(26, np.zeros(16, np.uint8), 4) is None         # an I32 table: no decoder
    assert oracle.decode_raw_to_f32(30, np.zeros(8, np.uint8), 4) is None          # BF16: no arm in the reference's match
    with pytest.raises(oracle.OracleError, match="dtype F16: 7 bytes for 4 elements"):
        oracle.decode_raw_to_f32(1, np.zeros(7, np.uint8), 4)
    with pytest.raises(oracle.OracleError, match="144-byte|per 256-block"):
        oracle.decode_raw_to_f32(12, np.zeros(143, np.uint8), 256)


def test_oracle_block_formats_go_through_the_block_decoders():
    from joshua_amd import synth
    for qt in (8, 10, 12, 14, 16, 39):
        blocks = synth.normal_quantized(qt, 40 + qt, 1024, 0.02)
        assert np.array_equal(oracle.decode_raw_to_f32(qt, blocks, 1024), oracle.dequantize(qt, blocks))


@pytest.mark.gpu
def test_device_decode_raw_against_the_oracle():
    from joshua_amd import capi, synth
    for dtype, raw, elems, want in cases():
        got = capi.decode_raw_to_f32(dtype, raw, elems)
        if dtype == 1:
            assert np.array_equal(got, want)                       # infinities included
        else:
            assert np.array_equal(got, want), dtype
    for qt in (8, 10, 12, 14, 16, 39):
        blocks = synth.normal_quantized(qt, 60 + qt, 2048, 0.02)
        assert np.array_equal(capi.decode_raw_to_f32(qt, blocks, 2048), oracle.decode_raw_to_f32(qt, blocks, 2048)), qt
    # a tensor beyond the decoders' int column index goes through as rows of 2^20 blocks and a shorter last one:
    # the same walk with rows of 3 blocks (7 blocks: two whole rows and a rest, for every block format)
    os.environ["JQ_DECODE_CHUNK_BLOCKS"] = "3"
    try:
        for qt in (8, 10, 12, 14, 16, 39):
            elems = 7 * (32 if qt in (8, 39) else 256)
            blocks = synth.normal_quantized(qt, 70 + qt, elems, 0.02)
            assert np.array_equal(capi.decode_raw_to_f32(qt, blocks, elems), oracle.decode_raw_to_f32(qt, blocks, elems)), qt
    finally:
        del os.environ["JQ_DECODE_CHUNK_BLOCKS"]
    assert capi.decode_raw_to_f32(0, np.zeros(16, np.uint8), 4) is None
    assert capi.decode_raw_to_f32(26, np.zeros(16, np.uint8), 4) is None
    assert capi.decode_raw_to_f32(30, np.zeros(8, np.uint8), 4) is None
    with pytest.raises(capi.JoshuaHipError, match="dtype F16: 7 bytes for 4 elements"):
        capi.decode_raw_to_f32(1, np.zeros(7, np.uint8), 4)
    with pytest.raises(capi.JoshuaHipError, match="per 256-block"):
        capi.decode_raw_to_f32(12, np.zeros(143, np.uint8), 256)
    # the in-mapping formats answer in their block readers' words (src/iq2xxs.rs:75-82,422-429, src/mxfp4.rs:99-106,265-272)
    with pytest.raises(capi.JoshuaHipError, match="iq2_xxs: 65 bytes is not a whole number of 66 byte blocks"):
        capi.decode_raw_to_f32(16, np.zeros(65, np.uint8), 256)
    with pytest.raises(capi.JoshuaHipError, match="iq2_xxs: output holds 512 values, expected 256"):
        capi.decode_raw_to_f32(16, np.zeros(66, np.uint8), 512)
    with pytest.raises(capi.JoshuaHipError, match="mxfp4: 18 bytes is not a whole number of 17-byte blocks"):
        capi.decode_raw_to_f32(39, np.zeros(18, np.uint8), 32)
    with pytest.raises(capi.JoshuaHipError, match="mxfp4: output holds 64 values, expected 32"):
        capi.decode_raw_to_f32(39, np.zeros(17, np.uint8), 64)
