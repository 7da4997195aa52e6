"""jq_matmul_t_f16: f16 activations in, f16 results out (reference: src/mmap_tensor.rs:136-138, :378-380,
:451-453; wrappers src/mxfp4.rs:242-258, src/iq2xxs.rs:396-412).  The f32 product inside is the one the
other tests check; here: the widening is exact, the result is the f32 result rounded once to f16, overflow
becomes infinity, host and device pointers agree, bad lengths are refused.
Tolerance: |gpu - ref| <= 1e-3 * max(|ref|, 1) for the f32 sums (src/kquant_dot.rs:853) plus one f16
rounding step, 2^-10 |ref|."""
import numpy as np
import pytest

import oracle
from joshua_amd import capi, synth

pytestmark = pytest.mark.gpu


def close16(got, want):
    g, w = got.astype(np.float32), want.astype(np.float32)
    return bool(np.all(np.abs(g - w) <= 1e-3 * np.maximum(np.abs(w), 1.0) + 2.0 ** -10 * np.abs(w)))


@pytest.mark.parametrize("qtype,m,k,n", [(capi.Q4_K, 1, 4096, 512), (capi.Q4_K, 5, 1024, 300), (capi.Q8_0, 3, 512, 100),
                                         (capi.Q6_K, 40, 1024, 200), (capi.Q2_K, 2, 768, 64), (capi.IQ2_XXS, 2, 512, 96),
                                         (capi.MXFP4, 7, 256, 130)])
def test_f16_product_is_the_f32_product_rounded_once(qtype, m, k, n):
    blocks = synth.normal_quantized(qtype, 300 + n, n * k, 0.05)
    lhs = synth.normal(301 + k, (m, k)).astype(np.float16)
    got = capi.Weight.upload(qtype, blocks, n, k).matmul_t_f16(m, lhs)
    assert got.dtype == np.float16 and got.shape == (m, n)
    want = oracle.matmul_t_f16(qtype, (m, k, n), lhs, blocks, avx2=oracle.have_avx2())
    assert close16(got, want)
    # against the library's own f32 entry point over the widened activations: one rounding, nothing else
    y32 = capi.Weight.upload(qtype, blocks, n, k).matmul_t(m, lhs.astype(np.float32))
    assert np.array_equal(got, y32.astype(np.float16))


def q8_0_integer_blocks(n, k, seed):
    rng = np.random.default_rng(seed)
    q = np.zeros((n, k), np.int64)
    for r in range(n):
        q[r, rng.choice(k, size=16, replace=False)] = rng.integers(-3, 4, size=16)
    blocks = np.zeros((n, k // 32, 34), np.uint8)
    blocks[:, :, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blocks[:, :, 2:] = q.reshape(n, k // 32, 32).astype(np.int8).view(np.uint8)
    return blocks.reshape(-1), q


def test_small_integers_come_back_exactly():
    """Q8_0 blocks with d = 1 and 16 weights in -3..3 a row against integer activations in -4..4: every sum
    is an integer below 2048, which f16 holds exactly."""
    n, k, m = 96, 512, 6
    blocks, q = q8_0_integer_blocks(n, k, 8)
    assert np.array_equal(oracle.dequantize(capi.Q8_0, blocks).reshape(n, k), q.astype(np.float32))
    x = np.random.default_rng(9).integers(-4, 5, size=(m, k))
    got = capi.Weight.upload(capi.Q8_0, blocks, n, k).matmul_t_f16(m, x.astype(np.float16))
    assert np.array_equal(got.astype(np.int64), x @ q.T)


def test_overflow_rounds_to_infinity_and_non_finite_inputs_propagate():
    n, k = 64, 256
    blocks, q = q8_0_integer_blocks(n, k, 10)
    w = capi.Weight.upload(capi.Q8_0, blocks, n, k)
    x = np.zeros((3, k), np.float16)
    x[0, :] = 60000.0                      # sums reach several 10^5: beyond the largest f16, 65504
    x[1, 5] = np.inf
    x[2, 7] = 1.0
    got = w.matmul_t_f16(3, x).astype(np.float32)
    s0 = 60000.0 * q.sum(axis=1)
    big = np.abs(s0) > 65520
    assert big.any() and np.all(np.isinf(got[0][big])) and np.array_equal(np.sign(got[0][big]), np.sign(s0[big]))
    # 0 * inf inside the row: NaN wherever the weight at the infinite activation is zero, signed infinity elsewhere
    assert np.all(~np.isfinite(got[1]))
    assert np.array_equal(got[2], q[:, 7].astype(np.float32))


def test_device_pointers_give_the_host_result():
    import torch
    n, k, m = 1000, 4096, 16
    blocks = synth.normal_quantized(capi.Q4_K, 21, n * k, 0.02)
    lhs = synth.normal(22, (m, k)).astype(np.float16)
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    host = w.matmul_t_f16(m, lhs)
    x = torch.from_numpy(lhs).cuda()
    y = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(3):
            w.matmul_t_f16_dev(m, x.data_ptr(), x.numel(), y.data_ptr(), y.numel(), stream.cuda_stream)
    stream.synchronize()
    assert np.array_equal(y.cpu().numpy(), host)


def test_f16_product_on_a_warmed_up_stream_is_captured_into_a_graph():
    """The f32 copies of the operands live in a buffer kept per stream: after one call of the size, the next
    allocates nothing and goes into a HIP graph, which replays to the eager result with eager calls in between."""
    import torch
    n, k, m = 1536, 4096, 16
    w = capi.Weight.upload(capi.Q6_K, synth.normal_quantized(capi.Q6_K, 41, n * k, 0.02), n, k)
    x = torch.from_numpy(synth.normal(42, (m, k)).astype(np.float16)).cuda()
    x2 = torch.from_numpy(synth.normal(43, (m, k)).astype(np.float16)).cuda()
    y = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    y2 = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    stream = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        w.matmul_t_f16_dev(m, x.data_ptr(), x.numel(), y.data_ptr(), y.numel(), stream.cuda_stream)   # first use allocates
        stream.synchronize()
        want = y.clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            w.matmul_t_f16_dev(m, x.data_ptr(), x.numel(), y.data_ptr(), y.numel(), torch.cuda.current_stream().cuda_stream)
        for rep in range(3):
            w.matmul_t_f16_dev(m, x2.data_ptr(), x2.numel(), y2.data_ptr(), y2.numel(), stream.cuda_stream)  # eager, same buffer
            y.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, want), rep
    assert not torch.equal(y2, want)
    del graph
    torch.cuda.synchronize()
    capi.stream_release(stream.cuda_stream)


def test_bad_lengths_are_refused_and_empty_products_succeed():
    n, k = 32, 256
    blocks = synth.normal_quantized(capi.Q4_K, 31, n * k, 0.02)
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    x = np.zeros(2 * k - 1, np.float16)
    dst = np.full(2 * n, 7.0, np.float16)
    rc = capi.lib().jq_matmul_t_f16(w._h, 2, x.ctypes.data, x.size, dst.ctypes.data, dst.size, 0, None)
    assert rc != 0 and "lhs" in capi.last_error() and np.all(dst == 7.0)
    x = np.zeros(2 * k, np.float16)
    rc = capi.lib().jq_matmul_t_f16(w._h, 2, x.ctypes.data, x.size, dst.ctypes.data, dst.size - 1, 0, None)
    assert rc != 0 and np.all(dst == 7.0)
    assert capi.lib().jq_matmul_t_f16(w._h, 0, None, 0, None, 0, 0, None) == 0
