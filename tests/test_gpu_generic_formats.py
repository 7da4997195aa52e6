"""Q4_0, Q4_1, Q5_0, Q5_1, Q3_K, Q5_K on the device (the formats the reference serves through the
canonical decode plus its 8-lane dot, src/quant_matmul.rs:228-248): decode bit for bit, matmul for few
and many activation rows, row gather, expert slices at odd byte offsets, a mixture-of-experts layer."""
import numpy as np
import pytest

import oracle
from oracle.moe import MoeOracle
from joshua_amd import capi, synth

pytestmark = pytest.mark.gpu
TYPES = capi.GENERIC_TYPES
SCALE_OFFSETS = {2: (0,), 3: (0, 2), 6: (0,), 7: (0, 2), 11: (108,), 13: (0, 2)}


def close(got, want, tol=1e-3):
    return np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1.0))


@pytest.mark.parametrize("qtype", TYPES)
def test_geometry_and_dequantize_bit_exact(qtype):
    elems, nbytes = capi.block_geometry(qtype)
    assert (elems, nbytes) == oracle.block_geometry(qtype) and capi.type_size_bytes(qtype, elems * 3) == 3 * nbytes
    n, k = 37, 1024
    for blocks in (synth.random_blocks(qtype, 11, n * k), None):
        if blocks is None:      # every byte pattern is a valid block (reference: src/kquant_dot.rs:37-40)
            blocks = np.random.default_rng(qtype).integers(0, 256, size=n * (k // elems) * nbytes, dtype=np.uint8)
            for off in SCALE_OFFSETS[qtype]:
                blocks.reshape(-1, nbytes)[:, off + 1] &= 0x7B
        got = capi.Weight.upload(qtype, blocks, n, k).dequantize()
        want = oracle.dequantize(qtype, blocks).reshape(n, k)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("qtype", TYPES)
@pytest.mark.parametrize("m", [1, 2, 3, 5, 8, 16, 17])
def test_matmul_few_rows(qtype, m):
    n, k = 203, 1536
    blocks = synth.random_blocks(qtype, 100 + qtype, n * k)
    lhs = synth.normal(200 + m, (m, k))
    got = capi.Weight.upload(qtype, blocks, n, k).matmul_t(m, lhs)
    assert close(got, oracle.matmul_t(qtype, (m, k, n), lhs, blocks, avx2=oracle.have_avx2()))


@pytest.mark.parametrize("qtype", TYPES)
@pytest.mark.parametrize("m,k,n", [(64, 1024, 130), (200, 4096, 96)])
def test_matmul_many_rows(qtype, m, k, n):
    blocks = synth.random_blocks(qtype, 300 + qtype, n * k)
    lhs = synth.normal(301 + m, (m, k))
    got = capi.Weight.upload(qtype, blocks, n, k).matmul_t(m, lhs)
    assert close(got, oracle.matmul_t(qtype, (m, k, n), lhs, blocks, avx2=oracle.have_avx2()))


@pytest.mark.parametrize("qtype", TYPES)
def test_row_lengths_that_are_not_multiples_of_256_and_non_finite_rows(qtype):
    elems, _ = capi.block_geometry(qtype)
    k = 256 * 3 + (elems if elems < 256 else 256)
    n, m = 33, 20
    blocks = synth.random_blocks(qtype, 41, n * k)
    lhs = synth.normal(42, (m, k))
    w = capi.Weight.upload(qtype, blocks, n, k)
    assert close(w.matmul_t(m, lhs), oracle.matmul_t(qtype, (m, k, n), lhs, blocks))
    k2 = 1024
    blocks = synth.random_blocks(qtype, 43, n * k2)
    lhs = synth.normal(44, (m, k2))
    lhs[3, 700] = np.inf
    got = capi.Weight.upload(qtype, blocks, n, k2).matmul_t(m, lhs)
    assert not np.isfinite(got[3]).any() and np.isfinite(np.delete(got, 3, axis=0)).all()


@pytest.mark.parametrize("qtype", TYPES)
def test_row_gather_and_expert_slices(qtype):
    # reference: src/mmap_tensor.rs:140-167 (embedding), src/quantized_qwen3_moe.rs:596-631 (expert slices)
    n_expert, n, k = 5, 24, 768
    blocks = synth.random_blocks(qtype, 51, n_expert * n * k)
    stacked = capi.Weight.upload(qtype, blocks, n_expert * n, k)
    ids = np.array([n_expert * n - 1, 0, 7, 7, 13], np.uint32)
    assert np.array_equal(stacked.embedding(ids), oracle.dequantize(qtype, blocks).reshape(-1, k)[ids])
    with pytest.raises(capi.JoshuaHipError):
        stacked.embedding(np.array([n_expert * n], np.uint32))
    per = blocks.size // n_expert
    for m in (1, 40):
        lhs = synth.normal(52 + m, (m, k))
        for e in (1, 4):            # slices that start at byte offsets which are not multiples of 16
            got = stacked.view(e * per, n, k).matmul_t(m, lhs)
            assert close(got, oracle.matmul_t(qtype, (m, k, n), lhs, blocks[e * per:(e + 1) * per]))


@pytest.mark.parametrize("qtype", [capi.Q5_K, capi.Q4_0, capi.Q3_K])
@pytest.mark.parametrize("tokens", [1, 9])
def test_mixture_of_experts_layer(qtype, tokens):
    h, inter, E, k = 512, 256, 16, 4
    rw = synth.normal(60, (E, h), sigma=0.02)
    gate, up = synth.random_blocks(qtype, 61, E * inter * h), synth.random_blocks(qtype, 62, E * inter * h)
    down = synth.random_blocks(qtype, 63, E * h * inter)
    ora = MoeOracle(qtype, h, inter, E, k, rw, gate, up, down, avx2=oracle.have_avx2())
    dev = capi.Moe(capi.MoeConfig(E, k, h, inter, 0, 1, 0.0, 1, 1), rw, capi.Weight.upload(qtype, gate, E * inter, h),
                   capi.Weight.upload(qtype, up, E * inter, h), capi.Weight.upload(qtype, down, E * h, inter))
    x = synth.normal(64, (tokens, h))
    assert close(dev.forward(x), ora.forward(x))


I8_GEMV_KERNEL = {2: "q4_0_gemv_mfma_lds", 3: "q4_1_gemv_mfma_lds", 6: "q5_0_gemv_mfma_lds", 7: "q5_1_gemv_mfma_lds",
                  13: "q5k_gemv_mfma_lds", 11: "q3k_gemv_mfma_lds"}


@pytest.mark.parametrize("qtype", sorted(I8_GEMV_KERNEL))
def test_one_row_against_rows_of_4096_runs_on_the_int8_matrix_cores(qtype):
    """One activation row against 256 weight rows or more of 4096 columns: the int8 matrix-core GEMV over the codes
    as they are in the file, with the format's offset (-8 d, m, -16 d, dmin m) on the activations' sums.  A row
    count that ends inside a tile of 16 and inside a workgroup's round; activations whose 32-element sub-blocks
    differ by orders of magnitude (each has its own 15-bit fixed-point scale: tiny sub-blocks keep their digits, and
    with a sub-block 10^4 times the others the error stays below 10^-4 of the sum of the terms' magnitudes; the
    element-wise bound cannot hold there for the rows whose large terms cancel); a row of zeros; an
    infinity (the whole result is NaN, as for every integer kernel)."""
    k = 4096
    for n in (256, 1000, 4099):
        blocks = synth.random_blocks(qtype, 60 + qtype + n, n * k)
        x = synth.normal(61 + n, (1, k))
        x[0, 1024:1056] *= 1e-5
        x[0, 2048:2080] *= 1e-2
        w = capi.Weight.upload(qtype, blocks, n, k)
        got = w.matmul_t(1, x)
        assert capi.last_kernel() == I8_GEMV_KERNEL[qtype]
        assert close(got, oracle.matmul_t(qtype, (1, k, n), x, blocks, avx2=oracle.have_avx2()))
    dense = oracle.dequantize(qtype, blocks).reshape(n, k).astype(np.float64)
    xb = x.copy()
    xb[0, 96:128] *= 1e4
    exact, terms = dense @ xb[0].astype(np.float64), np.abs(dense) @ np.abs(xb[0]).astype(np.float64)
    assert np.all(np.abs(w.matmul_t(1, xb)[0] - exact) <= 1e-4 * terms)
    only = np.zeros((1, k), np.float32)
    only[0, 1024:1056] = x[0, 1024:1056]                                      # the tiny sub-block alone: its own digits
    assert close(w.matmul_t(1, only) * 1e5, (dense @ only[0].astype(np.float64))[None, :] * 1e5, 1e-4)
    assert np.array_equal(w.matmul_t(1, np.zeros((1, k), np.float32)), np.zeros((1, n), np.float32))
    x[0, 7] = np.inf
    assert np.all(np.isnan(w.matmul_t(1, x)))
