"""Pins the CPU oracle's matmul: float64 GEMM over decoded weights at the
reference's own tolerances and shapes, scalar build == AVX2 build bit for bit,
thread-count independence, assign semantics and shape rejection
(reference tests: src/kquant_dot.rs:781-959, src/quant_matmul.rs:373-608,
src/iq2xxs.rs:758-886, src/mxfp4.rs:351-450)."""
import os

import numpy as np
import pytest

import oracle
from joshua_amd import synth

needs_avx2 = pytest.mark.skipif(not oracle.have_avx2(), reason="host CPU lacks AVX2/FMA/F16C")


def ref_weights(n, k):
    i = np.arange(n * k, dtype=np.uint64)
    return (((i * np.uint64(2654435761)) % np.uint64(100000)).astype(np.float32) / np.float32(1000.0)
            - np.float32(50.0)).reshape(n, k)


def ref_lhs(m, k, mul=40503):
    i = np.arange(m * k, dtype=np.uint64)
    return (((i * np.uint64(mul)) % np.uint64(1000)).astype(np.float32) / np.float32(100.0)
            - np.float32(5.0)).reshape(m, k)


def same_order_dot(lhs, w):
    """The reference tests' "Reference A": 8 lane accumulators fed in column
    order with single-rounding multiply-adds, then summed
    (reference: src/kquant_dot.rs:832-852).  float64 holds x*w exactly, so
    rounding x*w + acc once to f32 differs from a true fma only by rare double
    rounding."""
    m, k = lhs.shape
    n = w.shape[0]
    acc = np.zeros((m, n, 8), np.float32)
    x64, w64 = lhs.astype(np.float64), w.astype(np.float64)
    for c in range(0, k, 8):
        acc = (x64[:, None, c:c + 8] * w64[None, :, c:c + 8] + acc.astype(np.float64)).astype(np.float32)
    s0, s1, s2, s3 = (acc[..., i] + acc[..., i + 4] for i in range(4))
    return (s0 + s2) + (s1 + s3)


def fixture_iq2xxs_rhs(golden_dir, k, n):
    blocks = np.fromfile(os.path.join(golden_dir, "iq2xxs_blocks.bin"), dtype=np.uint8).reshape(4, 66)
    idx = np.arange(n * (k // 256)) % 4
    return np.ascontiguousarray(blocks[idx]).reshape(-1)


def mxfp4_pattern(n, k):
    """Deterministic blocks of the reference's MXFP4 tests (src/mxfp4.rs:356-368)."""
    bpr = k // 32
    out = np.empty((n, bpr, 17), np.uint8)
    j = np.arange(16)
    for r in range(n):
        for b in range(bpr):
            out[r, b, 0] = 127 + r % 3
            out[r, b, 1:] = ((j + r * 3 + b * 5) % 16) | (((j + r) % 16) << 4)
    return out.reshape(-1)


KQ_CASES = [  # reference: src/kquant_dot.rs:894-901, src/quant_matmul.rs:499-515
    (oracle.Q8_0, 1, 256, 40), (oracle.Q8_0, 3, 512, 17), (oracle.Q8_0, 5, 128, 9), (oracle.Q8_0, 1, 256, 64),
    (oracle.Q2_K, 1, 256, 40), (oracle.Q2_K, 3, 512, 11), (oracle.Q2_K, 5, 768, 9),
    (oracle.Q4_K, 1, 256, 40), (oracle.Q4_K, 3, 512, 13), (oracle.Q4_K, 4, 768, 25),
    (oracle.Q6_K, 1, 256, 40), (oracle.Q6_K, 3, 512, 13), (oracle.Q6_K, 6, 768, 10),
]


@pytest.mark.parametrize("qtype,m,k,n", KQ_CASES)
def test_kquant_matmul_equals_gemm_over_decoded_weights(qtype, m, k, n):
    blocks = synth.quantize(qtype, ref_weights(n, k))
    lhs = ref_lhs(m, k)
    got = oracle.matmul_t(qtype, (m, k, n), lhs, blocks)
    w = oracle.dequantize(qtype, blocks).reshape(n, k).astype(np.float64)
    want = lhs.astype(np.float64) @ w.T
    # reference A tolerance (same-order): 1e-3*max(|s|,1); the float64 GEMM is
    # an any-order reference, for which the reference allows 2e-2.
    assert np.all(np.abs(got - want) <= 1e-3 * np.maximum(np.abs(want), 1.0))


@pytest.mark.parametrize("qtype,m,k,n", [
    (oracle.Q2_K, 1, 7680, 64), (oracle.Q4_K, 1, 2048, 96), (oracle.Q8_0, 32, 4096, 48),
])
def test_kquant_matmul_at_model_row_lengths(qtype, m, k, n):
    # reference: src/kquant_dot.rs:906-914 (row lengths kept, row counts cut to stay fast)
    blocks = synth.quantize(qtype, ref_weights(n, k))
    lhs = ref_lhs(m, k)
    got = oracle.matmul_t(qtype, (m, k, n), lhs, blocks)
    w = oracle.dequantize(qtype, blocks).reshape(n, k)
    # Reference A (same lane order): 1e-3*max(|s|,1); the decode inside the dot
    # differs from to_float by one rounding per weight.
    same = same_order_dot(lhs, w)
    assert np.all(np.abs(got - same) <= 1e-3 * np.maximum(np.abs(same), 1.0))
    # Reference B (any order): 2e-2*max(|acc|,1).
    want = lhs.astype(np.float64) @ w.astype(np.float64).T
    assert np.all(np.abs(got - want) <= 2e-2 * np.maximum(np.abs(want), 1.0))


def test_fused_decode_differs_from_to_float_by_one_rounding_only():
    """The fused kernels use one fmsub where to_float uses two rounded ops
    (reference: src/kquant_dot.rs:258-260): per-element weights agree to 1 ulp
    of the larger operand, checked through an identity activation."""
    for qtype in (oracle.Q2_K, oracle.Q4_K):
        blocks = synth.quantize(qtype, ref_weights(3, 256))
        eye = np.eye(256, dtype=np.float32)
        fused = oracle.matmul_t(qtype, (256, 256, 3), eye, blocks).T  # [n, k] decoded inside the dot
        plain = oracle.dequantize(qtype, blocks).reshape(3, 256)
        assert np.all(np.abs(fused - plain) <= 2.0 ** -22 * np.maximum(np.abs(plain), 1.0))


@needs_avx2
@pytest.mark.parametrize("qtype,m,k,n", KQ_CASES + [
    (oracle.IQ2_XXS, 3, 1024, 11), (oracle.IQ2_XXS, 5, 512, 9), (oracle.MXFP4, 4, 1024, 23), (oracle.MXFP4, 2, 64, 3),
])
def test_scalar_build_equals_avx2_build_bit_for_bit(qtype, m, k, n, golden_dir):
    if qtype == oracle.IQ2_XXS:
        blocks = fixture_iq2xxs_rhs(golden_dir, k, n)
    elif qtype == oracle.MXFP4:
        blocks = mxfp4_pattern(n, k)
    else:
        blocks = synth.quantize(qtype, ref_weights(n, k))
    lhs = ref_lhs(m, k, 104729)
    a = oracle.matmul_t(qtype, (m, k, n), lhs, blocks)
    for threads in (1, 3, 8):
        b = oracle.matmul_t(qtype, (m, k, n), lhs, blocks, avx2=True, threads=threads)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (qtype, threads)


@needs_avx2
def test_threaded_matches_serial_bit_exact():
    # reference: src/kquant_dot.rs:916-929, src/quant_matmul.rs:583-595
    lhs = (np.arange(3 * 256, dtype=np.float32) * np.float32(0.01) - np.float32(1.0)).reshape(3, 256)
    for qtype in (oracle.Q8_0, oracle.Q2_K, oracle.Q4_K, oracle.Q6_K):
        blocks = synth.quantize(qtype, ref_weights(24, 256))
        ser = oracle.matmul_t(qtype, (3, 256, 24), lhs, blocks, avx2=True, threads=1)
        par = oracle.matmul_t(qtype, (3, 256, 24), lhs, blocks, avx2=True, threads=8)
        assert np.array_equal(ser, par)


def test_iq2xxs_matmul_matches_naive_f32(golden_dir):
    # reference: src/iq2xxs.rs:758-804
    m, k, n = 3, 512, 7
    rhs = fixture_iq2xxs_rhs(golden_dir, k, n)
    lhs = ref_lhs(m, k, 7919)
    got = oracle.matmul_t(oracle.IQ2_XXS, (m, k, n), lhs, rhs)
    w = oracle.dequantize(oracle.IQ2_XXS, rhs).reshape(n, k)
    want = np.zeros((m, n), np.float32)
    for i in range(m):
        for j in range(n):
            acc = np.float32(0)
            for kk in range(k):
                acc = np.float32(acc + np.float32(lhs[i, kk] * w[j, kk]))
            want[i, j] = acc
    assert np.all(np.abs(got - want) <= 1e-4 * np.maximum(np.abs(want), 1.0))


def test_iq2xxs_fused_and_portable_paths_agree(golden_dir):
    # reference: src/iq2xxs.rs:834-866
    m, k, n = 3, 1024, 11
    rhs = fixture_iq2xxs_rhs(golden_dir, k, n)
    lhs = ref_lhs(m, k, 7919)
    fast = oracle.matmul_t(oracle.IQ2_XXS, (m, k, n), lhs, rhs)
    scalar = oracle.iq2xxs_matmul_scalar((m, k, n), lhs, rhs)
    assert np.all(np.abs(fast - scalar) <= 1e-4 * np.maximum(np.abs(scalar), 1.0))


def test_mxfp4_matmul_matches_explicit_reference():
    # reference: src/mxfp4.rs:351-388
    m, k, n = 2, 64, 3
    rhs = mxfp4_pattern(n, k)
    lhs = (np.arange(m * k, dtype=np.float32) % np.float32(7.0) - np.float32(3.0)).reshape(m, k)
    got = oracle.matmul_t(oracle.MXFP4, (m, k, n), lhs, rhs)
    w = oracle.dequantize(oracle.MXFP4, rhs).reshape(n, k).astype(np.float64)
    assert np.all(np.abs(got - lhs.astype(np.float64) @ w.T) < 1e-3)
    # products of small integers and powers of two: the f32 sum is exact here
    assert np.array_equal(got.astype(np.float64), lhs.astype(np.float64) @ w.T)


@pytest.mark.parametrize("avx2", [False, pytest.param(True, marks=needs_avx2)])
def test_matmul_assigns_rather_than_accumulating(avx2):
    # reference: src/mxfp4.rs:390-416
    m, k, n = 1, 32, 2
    rhs = np.array([127] + [0x21] * 16 + [128] + [0x34] * 16, np.uint8)
    lhs = (np.arange(k) % 5 - 2).astype(np.float32)
    fresh = oracle.matmul_t(oracle.MXFP4, (m, k, n), lhs, rhs, avx2=avx2, dst=np.zeros(2, np.float32))
    dirty = oracle.matmul_t(oracle.MXFP4, (m, k, n), lhs, rhs, avx2=avx2, dst=np.full(2, 123.75, np.float32))
    assert np.array_equal(fresh, dirty)
    for qtype in (oracle.Q8_0, oracle.Q4_K, oracle.Q6_K):
        blocks = synth.quantize(qtype, ref_weights(4, 256))
        x = ref_lhs(2, 256)
        a = oracle.matmul_t(qtype, (2, 256, 4), x, blocks, avx2=avx2, dst=np.zeros(8, np.float32))
        b = oracle.matmul_t(qtype, (2, 256, 4), x, blocks, avx2=avx2, dst=np.full(8, -9.5, np.float32))
        assert np.array_equal(a, b)


@pytest.mark.parametrize("avx2", [False, pytest.param(True, marks=needs_avx2)])
def test_rejects_bad_shapes_and_leaves_dst_alone(avx2):
    # reference: src/quant_matmul.rs:597-608, src/iq2xxs.rs:806-816
    blocks = synth.quantize(oracle.Q8_0, ref_weights(2, 256))
    lhs = np.zeros(256, np.float32)
    for mkn, x in [((1, 100, 2), lhs), ((1, 256, 4), lhs), ((1, 256, 2), np.zeros(1, np.float32))]:
        dst = np.full(max(mkn[0] * mkn[2], 1), 5.0, np.float32)
        with pytest.raises(oracle.OracleError):
            oracle.matmul_t(oracle.Q8_0, mkn, x, blocks, avx2=avx2, dst=dst)
        assert np.all(dst == 5.0)
    rhs = np.zeros(264, np.uint8)
    with pytest.raises(oracle.OracleError):
        oracle.matmul_t(oracle.IQ2_XXS, (1, 100, 1), np.zeros(100, np.float32), rhs, avx2=avx2)
    with pytest.raises(oracle.OracleError):
        oracle.matmul_t(oracle.IQ2_XXS, (1, 256, 1), np.zeros(256, np.float32), rhs, avx2=avx2)
    with pytest.raises(oracle.OracleError):
        oracle.matmul_t(oracle.IQ2_XXS, (2, 256, 1), np.zeros(256, np.float32), rhs[:66], avx2=avx2,
                        dst=np.zeros(2, np.float32))
    with pytest.raises(oracle.OracleError):
        oracle.matmul_t(11, (1, 256, 1), np.zeros(256, np.float32), rhs[:66], avx2=avx2)


def test_empty_problem_is_a_no_op():
    # reference: src/quant_matmul.rs:176-178
    blocks = synth.quantize(oracle.Q4_K, ref_weights(2, 256))
    out = oracle.matmul_t(oracle.Q4_K, (0, 256, 2), np.zeros(0, np.float32), blocks, dst=np.zeros(0, np.float32))
    assert out.size == 0
    out = oracle.matmul_t(oracle.Q4_K, (3, 256, 0), np.zeros(768, np.float32), np.zeros(0, np.uint8),
                          dst=np.zeros(0, np.float32))
    assert out.size == 0
