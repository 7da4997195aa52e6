#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input: one
Q4_K GEMV, W 14336 x 4096 (Llama-3-8B FFN-up shape) times a 1 x 4096 f32
activation, inputs already resident in HBM.  Steps rotate over distinct copies
of the weight totalling several times the 256 MB Infinity Cache, so every step
streams its 33 MB of blocks from HBM.

Prints ONE JSON line: whole-job throughput in GB/s of algorithmic bytes
(packed weights + activations + result), the roofline fraction against the
8 TB/s HBM peak, and the CPU baseline (the AVX2 restatement of the reference's
kernels on this host's cores) on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

N, K = 14336, 4096
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the headline kernel, from rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE runs
# of this benchmark (profiles/), each scaled by what the same counter reads for joshua_amd/calib/copy_kernel
# (a plain copy of 33 030 144 bytes).  A counter run cannot happen inside this process, so the figure is
# quoted only while the dispatcher still chooses the kernel it was measured on (jq_last_kernel); any other
# kernel reports null until its own counter runs are in.
MEASURED_TRAFFIC = {"kernel": "q4k_gemv_mfma_lds", "m": 1, "bytes": 33_248_154}
SEED_W, SEED_X = 102, 202


def algorithmic_bytes(m: int) -> int:
    # packed Q4_K blocks + f32 activations + f32 result
    return N * (K // 256) * 144 + m * K * 4 + m * N * 4


def cpu_baseline(blocks: np.ndarray, lhs: np.ndarray, budget_s: float) -> dict:
    """Times the oracle's AVX2 build (the reference's row kernels and thread
    schedule) on the same GEMV; the only place the benchmark touches oracle/."""
    import oracle
    if not oracle.have_avx2():
        return {"value": None, "unit": "GB/s", "cores": 0, "kind": "port", "sample": "host CPU lacks AVX2/FMA/F16C"}
    threads = min(oracle.default_threads(), len(os.sched_getaffinity(0)))
    m = lhs.shape[0]
    dst = np.empty(m * N, np.float32)
    for _ in range(3):
        oracle.matmul_t(12, (m, K, N), lhs, blocks, avx2=True, threads=threads, dst=dst)
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 20 or (time.perf_counter() < t_end and len(times) < 2000):
        t0 = time.perf_counter()
        oracle.matmul_t(12, (m, K, N), lhs, blocks, avx2=True, threads=threads, dst=dst)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return {"value": round(algorithmic_bytes(m) / med / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"median of {len(times)} runs of the same Q4_K {N}x{K} M={m} GEMV, AVX2 row kernels, "
                      f"{threads} threads, 3 warm-up runs", "ms_per_step": round(med * 1e3, 4)}


BLOCK = {8: (32, 34), 10: (256, 84), 12: (256, 144), 14: (256, 210), 16: (256, 66), 39: (32, 17),
         2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 11: (256, 110), 13: (256, 176)}
# the formats the reference serves through its canonical decode plus the 8-lane dot (src/quant_matmul.rs:228-248)
F2_FORMATS = {2: "q4_0", 3: "q4_1", 6: "q5_0", 7: "q5_1", 11: "q3_k", 13: "q5_k"}
F16_MFMA_PEAK_TFLOPS = 2500.0
INT8_MFMA_PEAK_TOPS = 5000.0


def _time_calls(torch, stream, fn, count: int) -> float:
    """ms per call: `count` calls of fn(i) between two events on the launch stream."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record(stream)
    for i in range(count):
        fn(i)
    e1.record(stream)
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / count


def _timed_replays(torch, stream, enqueue, reps: int) -> list:
    """ms of each of `reps` repetitions of enqueue(), enqueued back to back with an event between them
    (the device never idles, so a repetition's time is that of its own launches)."""
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
    torch.cuda.synchronize()
    ev[0].record(stream)
    for i in range(reps):
        enqueue()
        ev[i + 1].record(stream)
    torch.cuda.synchronize()
    return [ev[i].elapsed_time(ev[i + 1]) for i in range(reps)]


def _cpu_timed(fn, budget_s: float, min_runs: int = 3, max_runs: int = 200) -> tuple:
    """(median seconds, runs) of fn() on the host within a time budget, one warm-up run first."""
    fn()
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < min_runs or (time.perf_counter() < t_end and len(times) < max_runs):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return float(np.median(times)), len(times)


def _close(got, want) -> bool:
    return bool(np.all(np.abs(got - want) <= 1e-3 * np.maximum(np.abs(want), 1.0)))


def matmul_workload(torch, capi, synth, qtype: int, n: int, k: int, m: int, seed: int, steps: int, copies: int,
                    cpu_seconds: float) -> dict:
    """One quantized matmul shape, weights rotated over `copies` distinct HBM copies; the result of the last
    timed call is checked against the oracle (all of it, or for many activation rows a sample of 1536
    weight rows), and the oracle's AVX2 build is timed on the same product."""
    import oracle
    be, bb = BLOCK[qtype]
    # (formats without a quantiser here: seeded random blocks with scales of a N(0, 0.02) tensor's size)
    blocks = synth.random_blocks(qtype, seed, n * k) if qtype in F2_FORMATS else synth.normal_quantized(qtype, seed, n * k, 0.02)
    lhs = synth.normal(seed + 100, (m, k))
    dev = torch.device("cuda:0")
    x = torch.from_numpy(lhs).to(dev)
    y = torch.zeros((m, n), device=dev)
    base = capi.Weight.upload(qtype, blocks, n, k)
    ws = [base] + [capi.Weight.upload_device(qtype, base.device_ptr, base.nbytes, n, k) for _ in range(copies - 1)]
    stream = torch.cuda.current_stream()
    sh = stream.cuda_stream

    def call(i):
        ws[i % len(ws)].matmul_t_dev(m, x.data_ptr(), x.numel(), y.data_ptr(), y.numel(), sh)

    _time_calls(torch, stream, call, max(steps // 10, 3))
    ms = _time_calls(torch, stream, call, steps)
    kernel = capi.last_kernel()
    abytes = n * (k // be) * bb + 4 * m * k + 4 * m * n
    res = {"us": round(ms * 1e3, 2), "kernel": kernel, "algorithmic_bytes": abytes, "gbs": round(abytes / ms / 1e6, 1),
           "hbm_frac": round(abytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
    if m > 16:
        tflops = 2.0 * m * n * k / ms / 1e9
        res["useful_tflops"] = round(tflops, 1)
        res["mfma_frac_of_f16_peak"] = round(tflops / F16_MFMA_PEAK_TFLOPS, 4)
        if "gemm_i8" in kernel:
            # the many-row GEMM multiplies on the int8 matrix cores (two int8 planes of activations: two integer MACs a
            # useful one); against that unit's dense peak, counting useful operations only
            res["mfma_frac_of_int8_peak"] = round(tflops / INT8_MFMA_PEAK_TOPS, 4)
    got = y.cpu().numpy()
    avx2 = oracle.have_avx2()
    if m * n * k <= (1 << 32):
        rows = np.arange(n)
    else:
        rows = np.unique(np.concatenate([np.arange(128), np.arange(n - 128, n), np.arange(128, n - 128, 11)[:1280]]))
    sub = blocks.reshape(n, -1)[rows].reshape(-1)
    res["parity_ok"] = _close(got[:, rows], oracle.matmul_t(qtype, (m, k, rows.size), lhs, sub, avx2=avx2))
    res["parity_rows_checked"] = int(rows.size)
    if cpu_seconds > 0 and avx2:
        threads = min(oracle.default_threads(), len(os.sched_getaffinity(0)))
        dst = np.empty(m * n, np.float32)
        med, runs = _cpu_timed(lambda: oracle.matmul_t(qtype, (m, k, n), lhs, blocks, avx2=True, threads=threads, dst=dst),
                               cpu_seconds)
        res["cpu_baseline"] = {"value": round(abytes / med / 1e9, 3), "unit": "GB/s", "us": round(med * 1e6, 1),
                               "cores": threads, "kind": "port",
                               "sample": f"median of {runs} runs of the same product, AVX2 oracle, {threads} threads"}
    return res


def moe_workload(torch, capi, synth, qtype: int, h: int, inter: int, n_expert: int, k_used: int, batch: int, seed: int,
                 steps: int, shared: bool, gating: int, cpu_seconds: float) -> dict:
    """One MoE layer call.  Every expert holds its own bytes (one quantised template per matrix, its packed
    quants rotated by the expert id: joshua_amd.synth.experts); tokens rotate so the routed experts change.
    The last token set is checked against the oracle, which is also timed on it."""
    import oracle
    from oracle.moe import MoeOracle
    from joshua_amd.synth.experts import RolledExperts
    be, bb = BLOCK[qtype]
    dev = torch.device("cuda:0")
    stacks, weights = [], []
    for i, (rows, cols) in enumerate(((inter, h), (inter, h), (h, inter))):
        st = RolledExperts(qtype, synth.normal_quantized(qtype, seed + i, rows * cols, 0.02), n_expert)
        d = st.device_stack(torch, dev)
        weights.append(capi.Weight.upload_device(qtype, d.data_ptr(), d.numel(), n_expert * rows, cols))
        del d
        stacks.append(st)
    sh_w = sh_o = None
    if shared:
        sb = [synth.normal_quantized(qtype, seed + 3 + i, inter * h, 0.02) for i in range(3)]
        sh_o = (qtype, inter, sb[0], sb[1], sb[2])
        sh_w = (capi.Weight.upload(qtype, sb[0], inter, h), capi.Weight.upload(qtype, sb[1], inter, h),
                capi.Weight.upload(qtype, sb[2], h, inter))
    router = synth.normal(seed + 6, (n_expert, h), 0.02)
    cfg = capi.MoeConfig(n_expert, k_used, h, inter, gating, 1, 0.0, 1, 1)
    moe = capi.Moe(cfg, router, weights[0], weights[1], weights[2], shared=sh_w)
    n_sets = 16 if batch == 1 else 4
    xs_host = [synth.normal(seed + 10 + i, (batch, h)) for i in range(n_sets)]
    xs = [torch.from_numpy(a).to(dev) for a in xs_host]
    y = torch.zeros((batch, h), device=dev)
    stream = torch.cuda.current_stream()
    sh = stream.cuda_stream
    per_expert = 3 * inter * (h // be) * bb
    distinct = [len(np.unique(moe.route(a)[0])) for a in xs_host]
    abytes = float(np.mean(distinct)) * per_expert + 4 * n_expert * h + (per_expert if shared else 0) + 8 * batch * h

    def call(i):
        moe.forward_dev(batch, xs[i % n_sets].data_ptr(), y.data_ptr(), sh)

    _time_calls(torch, stream, call, max(steps // 10, 3))
    ms = _time_calls(torch, stream, call, steps)
    res = {"us": round(ms * 1e3, 2), "distinct_experts_mean": round(float(np.mean(distinct)), 1),
           "algorithmic_bytes": int(abytes), "gbs": round(abytes / ms / 1e6, 1),
           "hbm_frac": round(abytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
    last = (steps - 1) % n_sets
    ora = MoeOracle(qtype, h, inter, n_expert, k_used, router, stacks[0], stacks[1], stacks[2],
                    gating="sigmoid" if gating else "softmax", norm_topk=True, shared=sh_o, avx2=oracle.have_avx2())
    res["parity_ok"] = _close(y.cpu().numpy(), ora.forward(xs_host[last]))
    if cpu_seconds > 0 and oracle.have_avx2():
        med, runs = _cpu_timed(lambda: ora.forward(xs_host[last]), cpu_seconds, min_runs=2)
        res["cpu_baseline"] = {"value": round(abytes / med / 1e9, 3), "unit": "GB/s", "us": round(med * 1e6, 1),
                               "cores": min(oracle.default_threads(), len(os.sched_getaffinity(0))), "kind": "port",
                               "sample": f"median of {runs} calls of the oracle's layer on one of the token sets (numpy "
                                         "routing and expert loop around the C kernels: AVX2 rows for Q4_K and IQ2_XXS, "
                                         "the reference's scalar loop for MXFP4; expert bytes built per call)"}
    moe.close()
    return res


DEEPSEEK_V3_MLA = dict(n_embd=7168, n_head=128, q_lora_rank=1536, kv_lora_rank=512, qk_nope_head_dim=128,
                       qk_rope_head_dim=64, v_head_dim=128, rms_eps=1e-6, rope_theta=10000.0, yarn_factor=40.0,
                       yarn_mscale_all_dim=1.0, yarn_orig_context_length=4096)


def mla_workload(torch, capi, synth, qtype: int, context: int, steps: int, seed: int, cpu_seconds: float = 0.0) -> dict:
    """One multi-head latent attention block of DeepSeek-V3 size: a prompt of `context` tokens in chunks of
    512, then `steps` single-token calls (the cache grows by one token a call)."""
    c = DEEPSEEK_V3_MLA
    be, bb = BLOCK[qtype]
    dev = torch.device("cuda:0")
    nh, qd = c["n_head"], c["qk_nope_head_dim"] + c["qk_rope_head_dim"]
    shapes = {"q_a": (c["q_lora_rank"], c["n_embd"]), "q_b": (nh * qd, c["q_lora_rank"]),
              "kv_a": (c["kv_lora_rank"] + c["qk_rope_head_dim"], c["n_embd"]),
              "kv_b": (nh * (c["qk_nope_head_dim"] + c["v_head_dim"]), c["kv_lora_rank"]),
              "o": (c["n_embd"], nh * c["v_head_dim"])}
    blocks = {name: synth.normal_quantized(qtype, seed + i, n * k, 0.02) for i, (name, (n, k)) in enumerate(shapes.items())}
    w = {name: capi.Weight.upload(qtype, blocks[name], n, k) for name, (n, k) in shapes.items()}
    cfg = capi.MlaConfig(n_ctx=context + 2 * steps + 64, **c)
    mla = capi.Mla(cfg, (w["q_a"], np.ones(c["q_lora_rank"], np.float32), w["q_b"]), w["kv_a"],
                   np.ones(c["kv_lora_rank"], np.float32), w["kv_b"], w["o"])
    stream = torch.cuda.current_stream()
    sh = stream.cuda_stream
    chunk = 512
    xs_host = synth.normal(seed + 10, (chunk, c["n_embd"]))
    # parity at this size on a short context (the oracle expands every cached token per head: minutes at 8192)
    from oracle import mla as om
    oc = dict(n_embd=c["n_embd"], n_head=nh, q_lora_rank=c["q_lora_rank"], kv_lora_rank=c["kv_lora_rank"],
              qk_nope=c["qk_nope_head_dim"], qk_rope=c["qk_rope_head_dim"], v_head_dim=c["v_head_dim"],
              rms_eps=c["rms_eps"], rope_theta=c["rope_theta"], context_length=context + 2 * steps + 64,
              yarn=dict(factor=c["yarn_factor"], orig_context_length=c["yarn_orig_context_length"],
                        mscale_all_dim=c["yarn_mscale_all_dim"]))
    ot = {"q_a": (qtype, blocks["q_a"]), "q_b": (qtype, blocks["q_b"]), "kv_a_mqa": (qtype, blocks["kv_a"]),
          "kv_b": (qtype, blocks["kv_b"]), "o": (qtype, blocks["o"]),
          "kv_a_norm": np.ones(c["kv_lora_rank"], np.float32), "q_a_norm": np.ones(c["q_lora_rank"], np.float32)}
    ref = om.MlaOracle(oc, ot)
    # parity at the order of the timed context: a prefill of min(context, 1024) tokens in chunks of 512 on both sides
    # (the oracle's unabsorbed form takes ~15 s of host time for 1024 tokens), then single-token steps at that
    # context, which also give the CPU figure; without a CPU budget a 64-token prefill and one step
    pc = min(context, 1024) if cpu_seconds > 0 else 64
    xp = synth.normal(seed + 11, (pc + 4, c["n_embd"]))
    parity_ok, pos = True, 0
    while pos < pc:
        t = min(chunk, pc - pos)
        parity_ok = _close(mla.forward(xp[pos:pos + t], pos), ref.forward(xp[pos:pos + t], pos)) and parity_ok
        pos += t
    cpu = None
    import time
    t_cpu = []
    for p in range(pc, pc + (3 if cpu_seconds > 0 else 1)):
        t0 = time.perf_counter()
        want = ref.forward(xp[p:p + 1], p)
        t_cpu.append(time.perf_counter() - t0)
        parity_ok = _close(mla.forward(xp[p:p + 1], p), want) and parity_ok
    if cpu_seconds > 0:
        cpu = {"us": round(sorted(t_cpu)[1] * 1e6, 1), "cores": os.cpu_count(), "kind": "port", "context": pc,
               "sample": f"median of 3 single-token steps of oracle/mla.py (numpy, the reference's unabsorbed form over "
                         f"decoded weights) at a context of {pc} tokens"}
    mla.reset()
    xs = torch.from_numpy(xs_host).to(dev)
    y = torch.zeros((chunk, c["n_embd"]), device=dev)
    pos, prefill_ms = 0, 0.0
    while pos < context:
        t = min(chunk, context - pos)
        p0 = pos
        prefill_ms += _time_calls(torch, stream, lambda i: mla.forward_dev(t, p0, xs.data_ptr(), y.data_ptr(), sh), 1)
        pos += t
    state = {"pos": pos}

    def call(i):
        mla.forward_dev(1, state["pos"], xs.data_ptr() + 4 * c["n_embd"] * (i % chunk), y.data_ptr(), sh)
        state["pos"] += 1

    _time_calls(torch, stream, call, max(steps // 10, 3))
    ms = _time_calls(torch, stream, call, steps)
    quantized = sum(n * (k // be) * bb for name, (n, k) in shapes.items() if name != "kv_b")
    kv_b_f32 = 4 * shapes["kv_b"][0] * shapes["kv_b"][1]  # the up-projection is held decoded
    cache = 4 * (c["kv_lora_rank"] + c["qk_rope_head_dim"]) * (context + steps // 2)
    abytes = quantized + kv_b_f32 + cache + 8 * c["n_embd"]
    res = {"us": round(ms * 1e3, 2), "context": context, "algorithmic_bytes": abytes, "gbs": round(abytes / ms / 1e6, 1),
           "hbm_frac": round(abytes / ms / 1e6 / HBM_PEAK_GBS, 4),
           "prefill_tokens_per_s": round(context / prefill_ms * 1e3, 1),
           "parity_ok": parity_ok,
           "parity_note": f"{pc}-token prefill in chunks of 512 and single-token steps at that context against the "
                          "reference's unabsorbed form",
           "cache_bytes_per_token": 4 * (c["kv_lora_rank"] + c["qk_rope_head_dim"]),
           "reference_cache_bytes_per_token": 4 * nh * (qd + c["v_head_dim"])}
    if cpu:
        res["cpu_baseline"] = cpu
    mla.close()
    return res


def extra_workloads(steps: int, only: str = "", cpu_seconds: float = 0.0) -> dict:
    """The other configurations of the path, one figure each (cold HBM unless noted), each with a parity
    check of what was timed and the CPU oracle's time beside it."""
    import torch
    from joshua_amd import capi, synth
    out = {}
    cs = min(cpu_seconds, 2.0)
    if only:  # a single workload, for profiling
        if "mla" in only:
            out["mla_deepseek_v3_q4_k_ctx%s_b1" % only.split(":")[-1]] = mla_workload(
                torch, capi, synth, 12, int(only.split(":")[-1]), steps, 107)
        elif only == "m16":
            out["q4_k_14336x4096_m16"] = matmul_workload(torch, capi, synth, 12, N, K, 16, 102, steps, 24, 0.0)
        elif only == "m512":
            out["q4_k_14336x4096_m512"] = matmul_workload(torch, capi, synth, 12, N, K, 512, 102, max(steps // 10, 10), 4, 0.0)
        elif only == "q6k_m512":
            out["q6_k_4096x12288_m512"] = matmul_workload(torch, capi, synth, 14, 4096, 12288, 512, 109, max(steps // 10, 10), 4, 0.0)
        elif only == "q8_0_m512":
            out["q8_0_4096x4096_m512"] = matmul_workload(torch, capi, synth, 8, 4096, 4096, 512, 110, max(steps // 10, 10), 8, 0.0)
        elif only == "q2k_m512":
            out["q2_k_14336x4096_m512"] = matmul_workload(torch, capi, synth, 10, N, K, 512, 111, max(steps // 10, 10), 4, 0.0)
        elif only == "q2k":
            out["q2_k_gemv_14336x4096_m1"] = matmul_workload(torch, capi, synth, 10, N, K, 1, 108, steps, 24, 0.0)
        elif only == "f2":
            for qt, name in F2_FORMATS.items():
                out[f"{name}_gemv_4096x4096_m1"] = matmul_workload(torch, capi, synth, qt, 4096, 4096, 1, 120 + qt, steps, 24, 0.0)
                out[f"{name}_4096x4096_m512"] = matmul_workload(torch, capi, synth, qt, 4096, 4096, 512, 140 + qt,
                                                                max(steps // 10, 10), 8, 0.0)
        elif only == "moe_b1":
            out["moe_qwen3_30b_a3b_q4_k_b1"] = moe_workload(torch, capi, synth, 12, 2048, 768, 128, 8, 1, 104, steps, False, 0, 0.0)
        elif only == "moe_b64":
            out["moe_qwen3_30b_a3b_q4_k_b64"] = moe_workload(torch, capi, synth, 12, 2048, 768, 128, 8, 64, 104, max(steps // 10, 10),
                                                             False, 0, 0.0)
        elif only == "moe_v3":
            out["moe_deepseek_v3_iq2_xxs_b1"] = moe_workload(torch, capi, synth, 16, 7168, 2048, 256, 8, 1, 105, steps, True, 1, 0.0)
        elif only == "moe_v3_b64":  # a 64-token call of the same layer: experts decoded once, their pairs streamed past
            out["moe_deepseek_v3_iq2_xxs_b64"] = moe_workload(torch, capi, synth, 16, 7168, 2048, 256, 8, 64, 105, max(steps // 10, 5),
                                                              True, 1, 0.0)
        elif only == "moe_v3_b512":  # a 512-token call of the same layer: the grouped int8 GEMM
            out["moe_deepseek_v3_iq2_xxs_b512"] = moe_workload(torch, capi, synth, 16, 7168, 2048, 256, 8, 512, 105, max(steps // 10, 5),
                                                               True, 1, 0.0)
        elif only == "moe_v3_mxfp4":
            out["moe_deepseek_v3_mxfp4_b1"] = moe_workload(torch, capi, synth, 39, 7168, 2048, 256, 8, 1, 105, steps, True, 1, 0.0)
        return out
    out["q8_0_gemv_4096x4096_m1"] = matmul_workload(torch, capi, synth, 8, 4096, 4096, 1, 101, steps, 24, cs)
    out["q4_k_14336x4096_m16"] = matmul_workload(torch, capi, synth, 12, N, K, 16, 102, steps, 24, cs)
    out["q4_k_14336x4096_m512"] = matmul_workload(torch, capi, synth, 12, N, K, 512, 102, max(steps // 10, 10), 4, cs)
    out["q6_k_gemv_4096x12288_m1"] = matmul_workload(torch, capi, synth, 14, 4096, 12288, 1, 106, steps, 12, cs)
    out["q6_k_4096x12288_m512"] = matmul_workload(torch, capi, synth, 14, 4096, 12288, 512, 109, max(steps // 10, 10), 4, cs)
    out["q2_k_gemv_14336x4096_m1"] = matmul_workload(torch, capi, synth, 10, N, K, 1, 108, steps, 24, cs)
    out["q2_k_14336x4096_m512"] = matmul_workload(torch, capi, synth, 10, N, K, 512, 111, max(steps // 10, 10), 4, cs)
    out["q8_0_4096x4096_m512"] = matmul_workload(torch, capi, synth, 8, 4096, 4096, 512, 110, max(steps // 10, 10), 8, cs)
    for qt, name in F2_FORMATS.items():   # (no CPU timing: the parity run is the oracle's sample here)
        out[f"{name}_gemv_4096x4096_m1"] = matmul_workload(torch, capi, synth, qt, 4096, 4096, 1, 120 + qt, steps, 24, 0.0)
        out[f"{name}_4096x4096_m512"] = matmul_workload(torch, capi, synth, qt, 4096, 4096, 512, 140 + qt, max(steps // 10, 10), 8, 0.0)
    torch.cuda.empty_cache()
    out["moe_qwen3_30b_a3b_q4_k_b1"] = moe_workload(torch, capi, synth, 12, 2048, 768, 128, 8, 1, 104, steps, False, 0, cs)
    out["moe_qwen3_30b_a3b_q4_k_b64"] = moe_workload(torch, capi, synth, 12, 2048, 768, 128, 8, 64, 104, max(steps // 10, 10),
                                                     False, 0, cs)
    torch.cuda.empty_cache()
    out["moe_deepseek_v3_iq2_xxs_b1"] = moe_workload(torch, capi, synth, 16, 7168, 2048, 256, 8, 1, 105, max(steps // 4, 10),
                                                     True, 1, cs)
    torch.cuda.empty_cache()
    # the same layer over 64 tokens (experts decoded once into registers, their pairs streamed past) and over 512
    # (a prompt: the grouped int8 GEMM); no CPU timing (the oracle's parity run is the bounded sample here)
    out["moe_deepseek_v3_iq2_xxs_b64"] = moe_workload(torch, capi, synth, 16, 7168, 2048, 256, 8, 64, 105, 10, True, 1, 0.0)
    torch.cuda.empty_cache()
    out["moe_deepseek_v3_iq2_xxs_b512"] = moe_workload(torch, capi, synth, 16, 7168, 2048, 256, 8, 512, 105, 8, True, 1, 0.0)
    torch.cuda.empty_cache()
    out["moe_deepseek_v3_mxfp4_b1"] = moe_workload(torch, capi, synth, 39, 7168, 2048, 256, 8, 1, 105, max(steps // 4, 10),
                                                   True, 1, cs)
    torch.cuda.empty_cache()
    for context in (1024, 8192):
        out[f"mla_deepseek_v3_q4_k_ctx{context}_b1"] = mla_workload(torch, capi, synth, 12, context, min(steps, 100), 107, cs)
        torch.cuda.empty_cache()
    return out


QWEN3_8B = dict(n_layer=36, hidden=4096, n_head=32, n_kv_head=8, head_dim=128, ffn=12288, vocab=151936, n_ctx=768,
                rms_eps=1e-6, rope_theta=1e6)


def decode_leg(prompt_len: int, n_decode: int, cpu_seconds: float, share_layers: bool, prefill_parity: int = 0) -> dict:
    """End-to-end greedy decode of a random-init Qwen3-8B-shaped Q4_K_M model: prefill of
    prompt_len uniform-random ids, then n_decode greedy tokens, one host round trip per
    token (the engine's loop, reference: src/engine.rs:1149-1294).  The CPU leg runs the
    same graph over the oracle's AVX2 kernels for a bounded number of tokens."""
    from joshua_amd import capi
    from joshua_amd.synth import uniform_u32
    from joshua_amd.synth.model import qwen3_tensors

    cfg = dict(QWEN3_8B, n_ctx=prompt_len + n_decode)
    t0 = time.perf_counter()
    tensors = {n: (qt, d) for n, qt, d in qwen3_tensors(cfg, 7, "q4_k_m", share_layers=share_layers)}
    t_gen = time.perf_counter() - t0
    c = capi.Qwen3Config(cfg["n_layer"], cfg["hidden"], cfg["n_head"], cfg["n_kv_head"], cfg["head_dim"], cfg["ffn"],
                         cfg["vocab"], cfg["n_ctx"], cfg["rms_eps"], cfg["rope_theta"])
    model = capi.Qwen3(c)
    wbytes = 0
    for name, (qt, d) in tensors.items():
        model.set_tensor(name, qt, d)
        if qt != 0 and name != "token_embd.weight":
            wbytes += d.nbytes
    prompt = uniform_u32(31, prompt_len, cfg["vocab"])
    # warm-up: a short prefill and a few steps, then start over
    model.forward_only(prompt[:16], 0)
    for i in range(4):
        model.forward_only([model.greedy()], 16 + i)
    model.reset()
    capi.stream_synchronize()
    t0 = time.perf_counter()
    model.forward_only(prompt, 0)
    tok = model.greedy()
    t_prefill = time.perf_counter() - t0
    out_tokens = [tok]
    t0 = time.perf_counter()
    for i in range(n_decode - 1):
        model.forward_only([tok], prompt_len + i)
        tok = model.greedy()
        out_tokens.append(tok)
    t_dec = time.perf_counter() - t0
    tps = (n_decode - 1) / t_dec
    res = {"tokens_per_s": round(tps, 2), "ms_per_token": round(1e3 / tps, 4),
           "prefill_tokens_per_s": round(prompt_len / t_prefill, 1),
           "workload": f"Qwen3-8B-shaped random-init model, Q4_K_M mix (Q4_K + Q6_K + Q8_0), weights N(0, 1/sqrt(k)) (unit gain per "
                       f"product; at the N(0, 0.02) of the kernel workloads the 36-layer logits leave the 1e-3 bound: 1.7e-3), {prompt_len} uniform-random "
                       f"prompt ids then {n_decode} greedy tokens, batch 1, f32 activations and KV cache",
           "weight_bytes_per_token": wbytes, "weights_gbs": round(wbytes * tps / 1e9, 1),
           "hbm_frac": round(wbytes * tps / 1e9 / HBM_PEAK_GBS, 4),
           "layers_share_bytes": share_layers, "model_gen_s": round(t_gen, 1)}
    if cpu_seconds > 0:
        import oracle
        from oracle import qwen3 as oq
        if oracle.have_avx2():
            threads = min(oracle.default_threads(), len(os.sched_getaffinity(0)))
            o = oq.Qwen3Oracle(cfg, tensors, avx2=True, threads=threads)
            n_pre = 8
            ref_logits = o.forward(list(prompt[:n_pre]), 0)
            # parity of the graph at full size: the same 8-token prefill on the device (the few-row kernels),
            # then greedy single-token steps (the fused launches and the 151936-row head), teacher-forced
            # with the oracle's pick; a step's pick is compared where the oracle's top two logits are further
            # apart than the tolerance
            model.reset()
            got = model.forward(prompt[:n_pre], 0)
            ok = _close(got, ref_logits)
            times, t, agree, decided, steps_ok = [], int(oq.greedy(ref_logits)), 0, 0, 0
            worst = float(np.max(np.abs(got - ref_logits) / np.maximum(np.abs(ref_logits), 1.0)))
            t_end = time.perf_counter() + cpu_seconds
            o.mm_seconds = 0.0
            while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 64):
                t0 = time.perf_counter()
                ref_step = o.forward([t], n_pre + len(times))
                times.append(time.perf_counter() - t0)
                got_step = model.forward([t], n_pre + len(times) - 1)
                steps_ok += int(_close(got_step, ref_step))
                worst = max(worst, float(np.max(np.abs(got_step - ref_step) / np.maximum(np.abs(ref_step), 1.0))))
                top2 = np.sort(ref_step)[-2:]
                if top2[1] - top2[0] > 2e-3 * max(abs(float(top2[1])), 1.0):
                    decided += 1
                    agree += int(model.greedy() == oq.greedy(ref_step))
                t = int(oq.greedy(ref_step))
            res["parity_ok"] = bool(ok and steps_ok == len(times) and agree == decided)
            res["parity"] = {"prefill_tokens": n_pre, "single_token_steps": len(times), "steps_within_tolerance": steps_ok,
                             "greedy_picks_compared": decided, "greedy_picks_equal": agree,
                             "largest_error_over_max_abs_ref_1": worst}
            cpu_tps = 1.0 / float(np.median(times))
            share = o.mm_seconds / float(np.sum(times))
            res["cpu_baseline"] = {"value": round(cpu_tps, 3), "unit": "tokens/s", "cores": threads, "kind": "port",
                                   "sample": f"median of {len(times)} greedy decode steps of the same model after an "
                                             f"{n_pre}-token prefill, AVX2 row kernels, {threads} threads",
                                   "share_of_time_in_c_kernels": round(share, 3),
                                   "tokens_per_s_counting_kernel_time_only": round(cpu_tps / max(share, 1e-6), 3)}
            if prefill_parity > 0:
                # the many-row path at full size: the first `prefill_parity` prompt tokens in one step through all
                # layers (int8 GEMMs, tiled attention) against the same graph over the oracle's kernels: the last
                # token's logits over the whole vocabulary.
                n_pp = min(prefill_parity, prompt_len)
                model.reset()
                o.reset()
                t0 = time.perf_counter()
                ref_pp = o.forward(list(prompt[:n_pp]), 0)
                t_ref = time.perf_counter() - t0
                got_pp = model.forward(prompt[:n_pp], 0)
                err = np.abs(got_pp - ref_pp) / np.maximum(np.abs(ref_pp), 1.0)
                res["prefill_parity"] = {"tokens": n_pp, "logits_compared": int(ref_pp.size), "within_1e-3": bool(err.max() <= 1e-3),
                                         "largest_error": float(err.max()), "greedy_equal": bool(oq.greedy(got_pp) == oq.greedy(ref_pp)),
                                         "oracle_seconds": round(t_ref, 1)}
                res["parity_ok"] = bool(res["parity_ok"] and err.max() <= 1e-3)
            res["speedup_vs_cpu"] = round(tps / cpu_tps, 2)
            res["speedup_vs_cpu_kernel_time_only"] = round(tps / (cpu_tps / max(share, 1e-6)), 2)
    model.close()
    return res


def plugin_leg(prompt_len: int, n_decode: int, share_layers: bool) -> dict:
    """The same model written to a GGUF file, loaded and driven through the four joshua_npu_* symbols as
    the reference engine drives a backend plugin (reference: src/npu/vendor.rs:95-185): the load (header,
    mapping, one upload per tensor), a prefill and greedy steps whose logits come back to the host."""
    import tempfile

    from joshua_amd import capi
    from joshua_amd.synth import gguf as gw
    from joshua_amd.synth import uniform_u32
    from joshua_amd.synth.model import qwen3_tensor_plan, qwen3_tensors

    cfg = dict(QWEN3_8B, n_ctx=prompt_len + n_decode)
    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "qwen3-8b-shaped-q4_k_m.gguf")
        t0 = time.perf_counter()
        gw.write_qwen3(path, cfg, qwen3_tensors(cfg, 7, "q4_k_m", share_layers=share_layers), qwen3_tensor_plan(cfg))
        t_write = time.perf_counter() - t0
        size = os.path.getsize(path)
        t0 = time.perf_counter()
        plug = capi.NpuPlugin(path, cfg["n_ctx"])
        t_load = time.perf_counter() - t0
        if plug.rc != 0:
            raise RuntimeError(f"joshua_npu_init failed ({plug.rc}): {capi.last_error()}")
        prompt = uniform_u32(31, prompt_len, cfg["vocab"])
        rc, logits = plug.forward(prompt[:16], 0)       # warm-up, then start over
        assert rc == 0 and plug.reset() == 0
        t0 = time.perf_counter()
        rc, logits = plug.forward(prompt, 0)
        t_prefill = time.perf_counter() - t0
        assert rc == 0
        t0 = time.perf_counter()
        for i in range(n_decode - 1):
            # greedy on the host, as the engine's sampler does: the last index holding the maximum
            tok = int(logits.size - 1 - np.argmax(logits[::-1]))
            rc, logits = plug.forward([tok], prompt_len + i)
            assert rc == 0
        t_dec = time.perf_counter() - t0
        plug.close()
    return {"gguf_bytes": size, "write_s": round(t_write, 1), "load_s": round(t_load, 2),
            "load_gbs": round(size / t_load / 1e9, 2), "prefill_tokens_per_s": round(prompt_len / t_prefill, 1),
            "tokens_per_s": round((n_decode - 1) / t_dec, 2),
            "note": "logits of every step copied to the host (608 KB) and the arg-max taken there"}


QWEN3_30B_A3B = dict(n_layer=48, hidden=2048, n_head=32, n_kv_head=4, head_dim=128, ffn=0, vocab=151936,
                     rms_eps=1e-6, rope_theta=1e6, n_expert=128, n_expert_used=8, expert_ffn=768)


def plugin_moe_leg(prompt_len: int, n_decode: int, share_layers: bool, n_layer: int, cpu_seconds: float) -> dict:
    """A Qwen3-30B-A3B-shaped random-init qwen3moe file (Q4_K_M mix) through the joshua_npu_* symbols, in the
    shape of the reference's own model benchmark (reference: examples/bench_qwen3moe.rs:147-174): load, one
    prefill of prompt_len copies of token 42, then n_decode single-token steps that each feed token 42 and
    take the arg-max of the returned logits on the host."""
    import tempfile

    from joshua_amd import capi
    from joshua_amd.synth import gguf as gw
    from joshua_amd.synth.model import qwen3_tensor_plan, qwen3_tensors

    cfg = dict(QWEN3_30B_A3B, n_layer=n_layer, n_ctx=prompt_len + n_decode)
    res = {}
    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "qwen3-30b-a3b-shaped-q4_k_m.gguf")
        t0 = time.perf_counter()
        gw.write_qwen3(path, cfg, qwen3_tensors(cfg, 9, "q4_k_m", share_layers=share_layers), qwen3_tensor_plan(cfg))
        t_write = time.perf_counter() - t0
        size = os.path.getsize(path)
        t0 = time.perf_counter()
        plug = capi.NpuPlugin(path, cfg["n_ctx"])
        t_load = time.perf_counter() - t0
        if plug.rc != 0:
            raise RuntimeError(f"joshua_npu_init failed ({plug.rc}): {capi.last_error()}")
        rc, logits = plug.forward([42] * 16, 0)       # warm-up (builds the layer objects), then start over
        assert rc == 0 and plug.forward([42], 16)[0] == 0 and plug.reset() == 0
        t0 = time.perf_counter()
        rc, logits = plug.forward([42] * prompt_len, 0)
        t_prefill = time.perf_counter() - t0
        assert rc == 0
        prefill_top = int(logits.size - 1 - np.argmax(logits[::-1]))
        t0 = time.perf_counter()
        last_top = prefill_top
        for i in range(n_decode):
            rc, logits = plug.forward([42], prompt_len + i)
            assert rc == 0
            last_top = int(logits.size - 1 - np.argmax(logits[::-1]))
        t_dec = time.perf_counter() - t0
        if cpu_seconds > 0:
            # parity at these sizes: a 6-token prompt and three single-token steps against the numpy graph over
            # the oracle matmul on the same tensors
            import oracle
            from oracle import qwen3 as oq
            tensors = {n: (qt, d) for n, qt, d in qwen3_tensors(cfg, 9, "q4_k_m", share_layers=share_layers)}
            o = oq.Qwen3Oracle(cfg, tensors, avx2=oracle.have_avx2(), threads=min(oracle.default_threads(), len(os.sched_getaffinity(0))))
            assert plug.reset() == 0
            toks, ok, steps = [42, 7, 1000, 42, 99999, 5], True, 0
            t0 = time.perf_counter()
            ref = o.forward(toks, 0)
            ok = ok and _close(plug.forward(toks, 0)[1], ref)
            cpu_times = []
            for i in range(3):
                t1 = time.perf_counter()
                ref = o.forward([42], len(toks) + i)
                cpu_times.append(time.perf_counter() - t1)
                ok = ok and _close(plug.forward([42], len(toks) + i)[1], ref)
                steps += 1
            res["parity_ok"] = bool(ok)
            res["parity"] = {"prefill_tokens": len(toks), "single_token_steps": steps}
            res["cpu_tokens_per_s"] = round(1.0 / float(np.median(cpu_times)), 3)
        plug.close()
    res.update({"gguf_bytes": size, "write_s": round(t_write, 1), "load_s": round(t_load, 2),
                "load_gbs": round(size / t_load / 1e9, 2), "prefill_tokens_per_s": round(prompt_len / t_prefill, 1),
                "tokens_per_s": round(n_decode / t_dec, 2), "ms_per_token": round(1e3 * t_dec / n_decode, 4),
                "top_token_after_prefill": prefill_top, "top_token_after_decode": last_top,
                "workload": f"Qwen3-30B-A3B-shaped random-init qwen3moe model, {n_layer} of 48 layers, Q4_K_M mix, 128 experts "
                            f"(8 used) of 768 rows, prefill of {prompt_len} x token 42 then {n_decode} steps feeding token 42",
                "layers_share_bytes": share_layers,
                "note": "logits of every step copied to the host (608 KB) and the arg-max taken there"})
    return res


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--m", type=int, default=1, help="activation rows (1 = decode GEMV)")
    ap.add_argument("--copies", type=int, default=24, help="distinct weight copies rotated through (cold HBM)")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="time budget of the CPU baseline (0 = skip)")
    ap.add_argument("--extras", type=int, default=1, help="1: also time the other configurations of the path")
    ap.add_argument("--only", default="", help="with --extras 1: a single extra workload, e.g. mla:1024")
    ap.add_argument("--decode", type=int, default=1, help="1: also run the Qwen3-8B-shaped end-to-end decode leg")
    ap.add_argument("--prompt", type=int, default=512)
    ap.add_argument("--new-tokens", type=int, default=256)
    ap.add_argument("--share-layers", type=int, default=0, help="1: draw each layer role's bytes once (faster set-up)")
    ap.add_argument("--no-graph", action="store_true", help="enqueue launches one by one instead of a HIP graph")
    ap.add_argument("--replays", type=int, default=0,
                    help="repetitions of the K timed steps whose median is reported (0: enough for ~30 ms, 5..400)")
    ap.add_argument("--plugin", type=int, default=0,
                    help="1: also write the model to a GGUF file and run it through the joshua_npu_* symbols")
    ap.add_argument("--prefill-parity", type=int, default=512,
                    help="N > 0: the decode leg also checks a one-step prefill of N prompt tokens of the 36-layer model against "
                         "the oracle (15 s of host time at 512 on 16 threads; skipped with --cpu-seconds 0)")
    ap.add_argument("--plugin-moe", type=int, default=-1,
                    help="N > 0: also write a Qwen3-30B-A3B-shaped qwen3moe GGUF of N layers (48 = the whole model) and run "
                         "it through the joshua_npu_* symbols; -1 (default): the whole model, every layer role's bytes drawn "
                         "once, as part of a full run (with the decode leg and all workloads) where 25 GB of temporary "
                         "space are free; 0: never")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2

    import torch
    from joshua_amd import capi, synth

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    capi.init(0)
    m = args.m

    blocks = synth.normal_quantized(capi.Q4_K, SEED_W, N * K, 0.02)
    lhs = synth.normal(SEED_X, (m, K))
    x = torch.from_numpy(lhs).to(dev)
    y = torch.zeros((m, N), device=dev)
    base = capi.Weight.upload(capi.Q4_K, blocks, N, K)
    weights = [base] + [capi.Weight.upload_device(capi.Q4_K, base.device_ptr, base.nbytes, N, K)
                        for _ in range(max(args.copies, 1) - 1)]
    stream = torch.cuda.current_stream()
    sh = stream.cuda_stream

    def enqueue(i0: int, count: int) -> None:
        for i in range(i0, i0 + count):
            weights[i % len(weights)].matmul_t_dev(m, x.data_ptr(), x.numel(), y.data_ptr(), y.numel(), sh)

    enqueue(0, args.warmup)
    torch.cuda.synchronize()

    # K steps are enqueued as one unit (a HIP graph holding the K launches, or K plain launches), the unit is
    # repeated back to back with an event between repetitions, and the reported time is the median
    # repetition: each sample is exactly K steps on a device that never idles, and a short run (K = 20)
    # no longer carries the graph's launch latency or a single slow repetition in its figure.
    steps = args.steps
    reps = args.replays if args.replays > 0 else int(min(400, max(5, np.ceil(30.0 / (steps * 0.008)))))
    mode = "stream"
    ms_graph = None
    if not args.no_graph:
        side = torch.cuda.Stream()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            sh_side = side.cuda_stream
            g.capture_begin()
            for i in range(steps):
                weights[i % len(weights)].matmul_t_dev(m, x.data_ptr(), x.numel(), y.data_ptr(), y.numel(), sh_side)
            g.capture_end()
        g.replay()
        torch.cuda.synchronize()
        rep_graph = _timed_replays(torch, stream, g.replay, reps)
        ms_graph = float(np.median(rep_graph))
    rep_stream = _timed_replays(torch, stream, lambda: enqueue(0, steps), reps)
    ms_stream = float(np.median(rep_stream))
    if ms_graph is not None and ms_graph < ms_stream:
        mode, ms_total, samples = "hipgraph", ms_graph, rep_graph
    else:
        ms_total, samples = ms_stream, rep_stream
    ms_per_step = ms_total / steps
    kernel = capi.last_kernel()

    # Cache-resident figure (one weight copy, 33 MB < Infinity Cache), labelled as such.
    ms_res = float(np.median(_timed_replays(
        torch, stream, lambda: [weights[0].matmul_t_dev(m, x.data_ptr(), x.numel(), y.data_ptr(), y.numel(), sh)
                                for _ in range(steps)], max(reps // 4, 3)))) / steps
    enqueue(0, 1)   # leave the result of a cold step in y for the check below
    torch.cuda.synchronize()

    # Parity spot check of the very buffers that were timed.
    import oracle
    want = oracle.matmul_t(12, (m, K, N), lhs, blocks, avx2=oracle.have_avx2())
    parity_ok = _close(y.cpu().numpy(), want)

    abytes = algorithmic_bytes(m)
    gbs = abytes / (ms_per_step * 1e-3) / 1e9
    out = {
        "metric": "Q4_K GEMV HBM GB/s (% of peak); decode tokens/s, 1 MI355X",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        # 4-bit weights x two int8 activation planes on every path (v_dot4 or int8 MFMA, int32 sums), f32 scales and result
        "dtype": "int8", "dtype_note": "integer dot products per 32-element sub-block (int4 weights x 15-bit fixed-point "
        "activations in two int8 planes), f32 scales and accumulation across sub-blocks" if m < 64 else
        "int8 MFMA GEMM (int4 weights unpacked to int8 x 15-bit fixed-point activations in two int8 planes, one scale per "
        "256-element run), int32 sums per 32-element sub-block, f32 scales and accumulation across sub-blocks",
        "data": "synthetic",
        "config": {"workload": f"Q4_K matmul_t {N}x{K} (Llama-3-8B FFN-up), M={m}, f32 activations N(0,1), "
                               f"weights N(0,0.02) quantized to Q4_K, {len(weights)} weight copies rotated (cold HBM)",
                   "launch": mode, "kernel": kernel},
        "timing": {"repetitions_of_the_k_steps": reps, "statistic": "median repetition / K",
                   "fastest_us_per_step": round(min(samples) / steps * 1e3, 3),
                   "slowest_us_per_step": round(max(samples) / steps * 1e3, 3)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC["bytes"] if (m == MEASURED_TRAFFIC["m"] and kernel == MEASURED_TRAFFIC["kernel"]) else None,
                     "algorithmic_bytes_per_launch": abytes, "kernel_us": round(ms_per_step * 1e3, 3)},
        "pct_of_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
        "cache_resident": {"value": round(abytes / (ms_res * 1e-3) / 1e9, 2), "unit": "GB/s",
                           "note": "one 33 MB weight copy reused every step (served by the 256 MB Infinity Cache)"},
        "stream_launch_ms_per_step": round(ms_stream / steps, 6),
        "graph_launch_ms_per_step": None if ms_graph is None else round(ms_graph / steps, 6),
        "parity_ok": parity_ok,
    }
    if args.cpu_seconds > 0:
        out["cpu_baseline"] = cpu_baseline(blocks, lhs, args.cpu_seconds)
    del weights, base
    torch.cuda.empty_cache()
    if args.extras:
        out["workloads"] = extra_workloads(min(max(steps, 100), 200), args.only, args.cpu_seconds)
        parity_ok = parity_ok and all(wl.get("parity_ok", True) for wl in out["workloads"].values())
    if args.decode:
        out["decode"] = decode_leg(args.prompt, args.new_tokens, args.cpu_seconds, bool(args.share_layers), args.prefill_parity)
        parity_ok = parity_ok and out["decode"].get("parity_ok", True)
    if args.plugin:
        out["plugin"] = plugin_leg(args.prompt, args.new_tokens, bool(args.share_layers))
    if args.plugin_moe > 0:
        out["plugin_moe"] = plugin_moe_leg(args.prompt, args.new_tokens, bool(args.share_layers), args.plugin_moe, args.cpu_seconds)
        parity_ok = parity_ok and out["plugin_moe"].get("parity_ok", True)
    elif args.plugin_moe < 0 and args.decode and args.extras and not args.only and args.m == 1:
        # the mixture-of-experts model rides along in a full run; a box without the room for its file is no failure
        import shutil
        import tempfile
        try:
            free = shutil.disk_usage(tempfile.gettempdir()).free
            if free < 25e9:
                out["plugin_moe"] = {"skipped": f"{free / 1e9:.0f} GB free in {tempfile.gettempdir()}, the model file takes 18.6"}
            else:
                out["plugin_moe"] = plugin_moe_leg(args.prompt, args.new_tokens, True, 48, args.cpu_seconds)
                parity_ok = parity_ok and out["plugin_moe"].get("parity_ok", True)
        except (OSError, MemoryError) as e:
            out["plugin_moe"] = {"skipped": repr(e)}
    print(json.dumps(out))
    return 0 if parity_ok else 1


if __name__ == "__main__":
    sys.exit(main())
