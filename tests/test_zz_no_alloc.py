"""jq_matmul_t_noalloc, the entry point that allocates no device memory, against jq_matmul_t on the
same device-resident inputs.  Both run the same kernels, so the results are compared bit for bit
(which is inside the 1e-3 bound of the other parity tests) and the first one of every pair also
against the CPU oracle.  Each case makes two calls in a row, the second with fewer activation rows:
the fixed scratch array keeps the first call's contents, and the second must not see them."""
import numpy as np
import pytest

import oracle
from joshua_amd import capi, synth

pytestmark = pytest.mark.gpu

TOL = 1e-3


def run_both(w, m, lhs):
    import torch
    x = torch.from_numpy(np.ascontiguousarray(lhs, dtype=np.float32)).cuda()
    stream = torch.cuda.current_stream().cuda_stream
    y_ref = torch.full((m, w.n), float("nan"), device="cuda")
    y_new = torch.full((m, w.n), float("nan"), device="cuda")
    w.matmul_t_dev(m, x.data_ptr(), x.numel(), y_ref.data_ptr(), y_ref.numel(), stream)
    w.matmul_t_noalloc(m, x.data_ptr(), x.numel(), y_new.data_ptr(), y_new.numel(), stream)
    torch.cuda.synchronize()
    return y_ref.cpu().numpy(), y_new.cpu().numpy()


CASES = [  # (format, k, n, first m, second m): shapes whose kernels keep operands or partial sums in scratch
    (capi.Q4_K, 4096, 2048, 16, 5),      # 16-row int8 kernel: prepared activation operands
    (capi.Q4_K, 4096, 1024, 96, 40),     # int8 and f16 GEMMs split over k: activation planes and partial sums
    (capi.Q6_K, 4096, 1024, 128, 64),    # Q6_K int8 GEMM split over k
    (capi.Q4_K, 1024, 512, 12, 3),       # streaming kernel (no scratch) and one row
    (capi.MXFP4, 2048, 4096, 48, 9),     # GEMM over decoded weights, split over k
    (capi.Q8_0, 4096, 4096, 40, 9),      # Q8_0 int8 GEMM on few rows, split over k
    (capi.Q2_K, 4096, 2048, 128, 20),    # Q2_K int8 GEMM
    (capi.Q8_0, 4096, 4096, 1, 1),       # one row: no scratch at all
]


@pytest.mark.parametrize("qtype,k,n,m1,m2", CASES)
def test_noalloc_matches_matmul_t_twice(qtype, k, n, m1, m2):
    blocks = synth.normal_quantized(qtype, 31, n * k, 0.02)
    w = capi.Weight.upload(qtype, blocks, n, k)
    for i, m in enumerate((m1, m2)):
        lhs = synth.normal(40 + i, (m, k))
        ref, new = run_both(w, m, lhs)
        assert np.array_equal(ref.view(np.uint32), new.view(np.uint32)), (capi.TYPE_NAMES[qtype], m)
        want = oracle.matmul_t(qtype, (m, k, n), lhs, blocks)
        assert np.all(np.abs(new - want) <= TOL * np.maximum(np.abs(want), 1.0)), (capi.TYPE_NAMES[qtype], m)


def test_noalloc_rejects_a_product_beyond_its_scratch():
    import torch
    k, n, m = 4096, 256, 4096            # the Q4_K GEMM wants 4 m k = 64 MiB of activation planes
    w = capi.Weight.upload(capi.Q4_K, synth.normal_quantized(capi.Q4_K, 5, n * k, 0.02), n, k)
    x = torch.zeros(m * k, device="cuda")
    y = torch.full((m * n,), 7.0, device="cuda")
    with pytest.raises(capi.JoshuaHipError, match="scratch"):
        w.matmul_t_noalloc(m, x.data_ptr(), x.numel(), y.data_ptr(), y.numel(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.all(y == 7.0)           # nothing written
    # shape errors read like jq_matmul_t's
    with pytest.raises(capi.JoshuaHipError, match="lhs/dst sized"):
        w.matmul_t_noalloc(2, x.data_ptr(), k, y.data_ptr(), 2 * n, 0)


def test_noalloc_leaves_device_memory_alone_on_a_stream_never_used_before():
    """jq_matmul_t keeps a scratch allocation per stream, made at a stream's first call; the entry point that
    allocates nothing must not.  On a fresh stream (no allocation of its own yet) the free device memory reads
    the same before and after a product that needs prepared operands and partial sums, and the result still
    equals jq_matmul_t's (which runs afterwards, on the default stream)."""
    import torch
    k, n, m = 4096, 1024, 96
    blocks = synth.normal_quantized(capi.Q4_K, 77, n * k, 0.02)
    w = capi.Weight.upload(capi.Q4_K, blocks, n, k)
    lhs = synth.normal(78, (m, k))
    x = torch.from_numpy(lhs).cuda()
    y_new = torch.full((m, n), float("nan"), device="cuda")
    y_ref = torch.full((m, n), float("nan"), device="cuda")
    fresh = torch.cuda.Stream()
    with torch.cuda.stream(fresh):   # the runtime's own first-use allocations of a stream (2 MiB of queue memory),
        y_new.fill_(float("nan"))    # by a launch that is not this library's
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    w.matmul_t_noalloc(m, x.data_ptr(), x.numel(), y_new.data_ptr(), y_new.numel(), fresh.cuda_stream)
    fresh.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)
    w.matmul_t_dev(m, x.data_ptr(), x.numel(), y_ref.data_ptr(), y_ref.numel(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert np.array_equal(y_ref.cpu().numpy().view(np.uint32), y_new.cpu().numpy().view(np.uint32))
