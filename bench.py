#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X: the Q4_K dequant-GEMV of a Llama-7B FFN projection.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-graph] [--skip-cpu]

A "step" is one pass of the hot path over one batch of synthetic input: one y = W.x product with the packed
weight already resident in HBM. Default workload (the configuration the metric is quoted on): W 11008x4096 ~ N(0, 0.02^2) quantised to GGUF
Q4_K (25 362 432 B), x ~ N(0, 1) fp32[4096], batch 1. Consecutive steps read DIFFERENT copies of the weight
(enough copies to exceed twice the 256 MB memory-side cache), so the reported rate is an HBM rate, not a cache rate;
the cache-warm figure (one copy) is reported next to it under "extra".

Prints ONE JSON line: metric/value (GB/s of algorithmic bytes = packed weight + x + y), the roofline object for
the GEMV kernel (HIP-event time over exactly K launches on the launch stream, median of several replays of the same
K-step graph) and the CPU baseline (the reference's own native C kernel, compiled from its sources into oracle/_ref,
timed on this host's cores: the reference's 4-participant row pool, and the same kernel over all host cores).

The default run also measures the two other parts of the headline metric in the same process and puts them under
"extra.headline": the Q4_K dequant-GEMM at M = 512 (TFLOP/s against the bf16 MFMA peak) and the synthetic
Llama-3-8B-shape decode (tokens/s, prefill time), each with its own parity flag. `--workload NAME` runs one workload
alone as the main line.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
LLC_BYTES = 256 << 20

# name -> (encoding, rows n, cols k, batch m)
WORKLOADS = {
    "q4k_gemv_11008x4096_b1": ("Q4_K", 11008, 4096, 1),
    "q4k_gemv_11008x4096_b4": ("Q4_K", 11008, 4096, 4),
    "q4k_gemv_11008x4096_b8": ("Q4_K", 11008, 4096, 8),
    "q8_0_gemv_4096x4096_b1": ("Q8_0", 4096, 4096, 1),
    "q6k_gemv_32000x4096_b1": ("Q6_K", 32000, 4096, 1),
    # the decoder's down projection: long rows, K split over the waves of a workgroup
    "q4k_gemv_4096x14336_b1": ("Q4_K", 4096, 14336, 1),
    # the other products of a Llama-3-8B decode step: fused gate/up, fused q/k/v, attention output, the Q6_K head
    "q4k_gemv_28672x4096_b1": ("Q4_K", 28672, 4096, 1),
    "q4k_gemv_6144x4096_b1": ("Q4_K", 6144, 4096, 1),
    "q4k_gemv_4096x4096_b1": ("Q4_K", 4096, 4096, 1),
    "q6k_gemv_128256x4096_b1": ("Q6_K", 128256, 4096, 1),
    # the remaining packed formats of the provider SPI, at the headline shape
    "q4_0_gemv_11008x4096_b1": ("Q4_0", 11008, 4096, 1),
    "q5_0_gemv_11008x4096_b1": ("Q5_0", 11008, 4096, 1),
    "q5_1_gemv_11008x4096_b1": ("Q5_1", 11008, 4096, 1),
    "q5k_gemv_11008x4096_b1": ("Q5_K", 11008, 4096, 1),
    # prefill: batch > 8 goes to the MFMA dequant-GEMM and is reported in TFLOP/s against the bf16 MFMA peak
    "q4k_gemm_512x4096x4096": ("Q4_K", 4096, 4096, 512),
    # short prompts and speculative batches: more rows than the GEMV kernels take, fewer than a 256-row tile
    "q4k_gemm_16x4096x4096": ("Q4_K", 4096, 4096, 16),
    "q4k_gemm_32x4096x4096": ("Q4_K", 4096, 4096, 32),
    "q4k_gemm_64x4096x4096": ("Q4_K", 4096, 4096, 64),
    "q4k_gemm_128x4096x4096": ("Q4_K", 4096, 4096, 128),
    "q4k_gemm_128x14336x4096": ("Q4_K", 14336, 4096, 128),
    "q6k_gemm_512x32000x4096": ("Q6_K", 32000, 4096, 512),
    "q4k_gemm_512x14336x4096": ("Q4_K", 14336, 4096, 512),
    # the other products of a Llama-3-8B prefill of 512 tokens: fused gate/up, fused q/k/v, down
    "q4k_gemm_512x28672x4096": ("Q4_K", 28672, 4096, 512),
    "q4k_gemm_512x6144x4096": ("Q4_K", 6144, 4096, 512),
    "q4k_gemm_512x4096x14336": ("Q4_K", 4096, 14336, 512),
    "q5k_gemm_512x4096x4096": ("Q5_K", 4096, 4096, 512),
    "q4_0_gemm_512x4096x4096": ("Q4_0", 4096, 4096, 512),
}
MFMA_BF16_PEAK_TFLOPS = 2500.0
ATTENTION_PREFILL_USES_MFMA = True    # the prompt-shape attention kernel runs bf16 operands on the matrix cores


def measured_traffic(workload, kernel):
    """HBM bytes per launch of the workload's dominant kernel as recorded by the last profiling session
    (profiles/traffic.json: rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE, scaled by what the same counters read for a plain
    copy of known size). A record belongs to a kernel: it is reported only while that kernel is the one that runs."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            rec = json.load(f)["workloads"].get(workload)
    except (OSError, ValueError, KeyError):
        return None
    if not rec or rec.get("kernel") != kernel:
        return None
    return rec.get("bytes_per_launch")


def algorithmic_bytes(enc, n, k, m):
    from skainet_amd.kernels import ENCODINGS
    _, bs, nb = ENCODINGS[enc]
    return n * (k // bs) * nb + 4 * k * m + 4 * n * m


def cpu_baseline(enc, n, k, m, packed, x, budget_s=12.0):
    """The reference's native row-major kernel (int8-activation path for K-quants, 4-participant row pool) on this
    host; protocol of the reference microbench: >= 20 warm-ups, median of >= 21 samples. m rows = m calls (the
    reference has no packed GEMM); for a prefill batch a bounded sample of rows is timed and scaled to the batch.
    Next to it ("all_cores"): the same kernel with the output rows split over every host core, one reference call per
    slice from a thread of its own (the calls release the interpreter lock), so the CPU figure is not held back by the
    reference's pool size."""
    m_full = m
    m = min(m, 16)
    from oracle import lib as L
    short = {"Q8_0": "q8_0", "Q4_K": "q4k", "Q6_K": "q6k", "Q4_0": "q4_0", "Q5_0": "q5_0", "Q5_1": "q5_1", "Q5_K": "q5k"}[enc]
    ref = L.ref()
    if ref is not None and hasattr(ref, f"skainet_{short}_matmul_rm"):
        fn, kind, cores, extra_args = getattr(ref, f"skainet_{short}_matmul_rm"), "reference", 4, ()
    elif enc in ("Q8_0", "Q4_K", "Q6_K"):
        fn, kind, cores, extra_args = getattr(L.oracle(fast=True), f"orc_native_{short}_matmul_rm"), "port", 1, ()
    else:                                          # the reference's scalar kernel restated, canonical order
        fn, kind, cores, extra_args = getattr(L.oracle(fast=True), f"orc_{short}_matmul"), "port", 1, (1,)
        short = f"scalar_{short}"
    y = np.empty((m, n), np.float32)

    def call():
        for r in range(m):
            fn(L.fp(x), r * k, L.u8(packed), 0, k, n, L.fp(y), r * n, *extra_args)

    def timed(fn_call, budget):
        t0 = time.perf_counter()
        fn_call()
        one = time.perf_counter() - t0
        warm = 20 if one * 41 < budget else 2
        samples_n = max(5, min(101, int((budget - warm * one) / max(one, 1e-6))))
        for _ in range(warm):
            fn_call()
        samples = []
        for _ in range(samples_n):
            t0 = time.perf_counter()
            fn_call()
            samples.append(time.perf_counter() - t0)
        return float(np.median(samples)), warm, samples_n

    med, warm, samples_n = timed(call, budget_s)

    # all host cores: row slices of at least 64 rows, one reference call per slice and thread
    all_cores = None
    from skainet_amd.kernels import ENCODINGS
    _, bs, nb = ENCODINGS[enc]
    ncores = max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)))
    if kind == "reference" and ncores > 1 and n >= 64 * 2:
        import concurrent.futures
        workers = min(ncores, n // 64)
        row_bytes = (k // bs) * nb
        bounds = [n * i // workers for i in range(workers + 1)]
        pool = concurrent.futures.ThreadPoolExecutor(max_workers=workers)

        def slice_call(i):
            r0, r1 = bounds[i], bounds[i + 1]
            for r in range(m):
                fn(L.fp(x), r * k, L.u8(packed), r0 * row_bytes, k, r1 - r0, L.fp(y), r * n + r0)

        def call_all():
            list(pool.map(slice_call, range(workers)))

        med_all, warm_all, n_all = timed(call_all, budget_s / 2)
        pool.shutdown()
        val = (2.0 * m * n * k / med_all / 1e12) if m_full > 8 else (algorithmic_bytes(enc, n, k, m) / med_all / 1e9)
        all_cores = {"value": round(val, 5 if m_full > 8 else 3), "unit": "TFLOP/s" if m_full > 8 else "GB/s", "cores": workers,
                     "sample": f"output rows split over {workers} threads (each thread's slice runs the reference's own pool of "
                               f"up to 4 participants when it has >= 512 rows), {warm_all} warm-ups + median of {n_all} "
                               f"({med_all * 1e3:.3f} ms)"}
    if m_full > 8:
        tflops = 2.0 * m * n * k / med / 1e12
        out = {"value": round(tflops, 5), "unit": "TFLOP/s", "cores": cores, "kind": kind,
               "sample": f"{m} of the {m_full} activation rows, one skainet_{short}_matmul_rm call per row, {warm} warm-ups + "
                         f"median of {samples_n} samples ({med / m * 1e3:.3f} ms/row -> {med / m * m_full * 1e3:.1f} ms/step, "
                         f"host has {os.cpu_count()} logical cores)"}
    else:
        gbs = algorithmic_bytes(enc, n, k, m) / med / 1e9
        out = {"value": round(gbs, 3), "unit": "GB/s", "cores": cores, "kind": kind,
               "sample": f"same workload, {warm} warm-ups + median of {samples_n} calls of skainet_{short}_matmul_rm "
                         f"({med * 1e3:.3f} ms/step, host has {os.cpu_count()} logical cores)"}
    if all_cores is not None:
        out["all_cores"] = all_cores
    return out


DECODER_WORKLOADS = {
    # name -> (config overrides, prompt tokens, layers with values of their own)
    "llama3_8b_decode": ({}, 512, 1),
    # a quarter-depth stack for quick runs; same per-layer shapes
    "llama3_8b_8layers_decode": ({"layers": 8}, 512, 1),
}
# The same stack driven through host arrays only (the unchanged kernel SPI): see measure_decoder_spi.
SPI_DECODER_WORKLOADS = {"llama3_8b_decode_spi": "llama3_8b_decode", "llama3_8b_8layers_decode_spi": "llama3_8b_8layers_decode"}
# The same stack written against the generic resident-activation ops class (one device entry per op, nothing fused by
# name): see measure_decoder_ops.
OPS_DECODER_WORKLOADS = {"llama3_8b_decode_ops": "llama3_8b_decode", "llama3_8b_8layers_decode_ops": "llama3_8b_8layers_decode"}


def cpu_baseline_decode(cfg, host, ctx):
    """Reference native kernels over one decoder layer's four Q4_K products and the Q6_K head, scaled to the stack:
    the CPU cost of the packed products of one decode step (attention, norms and RoPE left out, which favours the CPU)."""
    from oracle import lib as L
    ref = L.ref()
    if ref is not None:
        q4, q6, kind, cores = ref.skainet_q4k_matmul_rm, ref.skainet_q6k_matmul_rm, "reference", 4
    else:
        lib = L.oracle(fast=True)
        q4, q6, kind, cores = lib.orc_native_q4k_matmul_rm, lib.orc_native_q6k_matmul_rm, "port", 1
    rng = np.random.default_rng(1)
    shapes = [("l0.wqkv", cfg.q_dim + 2 * cfg.kv_dim, cfg.hidden), ("l0.wo", cfg.hidden, cfg.q_dim),
              ("l0.w_gate_up", 2 * cfg.ffn, cfg.hidden), ("l0.w_down", cfg.hidden, cfg.ffn)]
    xs = {k: rng.standard_normal(k).astype(np.float32) for k in {s[2] for s in shapes} | {cfg.hidden}}
    ys = {n: np.empty(n, np.float32) for n in {s[1] for s in shapes} | {cfg.vocab}}

    def layer():
        for name, n, k in shapes:
            q4(L.fp(xs[k]), 0, L.u8(host[name]), 0, k, n, L.fp(ys[n]), 0)

    def head():
        q6(L.fp(xs[cfg.hidden]), 0, L.u8(host["head"]), 0, cfg.hidden, cfg.vocab, L.fp(ys[cfg.vocab]), 0)

    def med(fn, reps):
        fn()
        t = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            t.append(time.perf_counter() - t0)
        return float(np.median(t))

    t_layer, t_head = med(layer, 41), med(head, 21)
    per_token = cfg.layers * t_layer + t_head
    return {"value": round(1.0 / per_token, 3), "unit": "tok/s", "cores": cores, "kind": kind,
            "sample": f"one layer's four Q4_K products (median of 41: {t_layer * 1e3:.2f} ms) x {cfg.layers} layers + the Q6_K head "
                      f"(median of 21: {t_head * 1e3:.2f} ms); attention, norms, RoPE not included; host has {os.cpu_count()} logical cores"}


ATTENTION_WORKLOADS = {
    # name -> (batch, seq_q, seq_kv); 32 query heads, 8 KV heads, head_dim 128, fp32, scale 1/sqrt(128), causal
    "sdpa_prefill_2048": (1, 2048, 2048),
    # the same prompt under a 512-key sliding window (a fourth field: the window)
    "sdpa_prefill_2048_w512": (1, 2048, 2048, 512),
    "sdpa_decode_576_b1": (1, 1, 576),
    "sdpa_decode_4096_b1": (1, 1, 4096),
    "sdpa_decode_4096_b8": (8, 1, 4096),
}
FP32_VECTOR_PEAK_TFLOPS = 157.3


def cpu_baseline_attention(batch, seq_q, seq_kv, heads, kv_heads, d, scale, window=0, budget_s=15.0):
    """The reference's skainet_f32_sdpa on this host. Prefill is sampled on one KV head's group (heads / kv_heads
    query heads) and scaled to all groups; decode runs the whole call."""
    from oracle import lib as L
    ref = L.ref()
    fn, kind = (ref.skainet_f32_sdpa, "reference") if ref is not None else (L.oracle(fast=True).orc_f32_sdpa, "port")
    h, hkv = (heads // kv_heads, 1) if seq_q > 1 else (heads, kv_heads)
    rng = np.random.default_rng(3)
    q = rng.standard_normal((batch, h, seq_q, d)).astype(np.float32)
    k = rng.standard_normal((batch, hkv, seq_kv, d)).astype(np.float32)
    v = rng.standard_normal((batch, hkv, seq_kv, d)).astype(np.float32)
    o = np.empty_like(q)

    def call():
        fn(L.fp(q), L.fp(k), L.fp(v), L.fp(o), batch, h, hkv, seq_q, seq_kv, d, scale, 1, window, 0, None, None, 0, 0, 0, 0)

    t0 = time.perf_counter()
    call()
    one = time.perf_counter() - t0
    reps = max(1, min(21, int(budget_s / max(one, 1e-6)) - 1))
    t = []
    for _ in range(reps):
        t0 = time.perf_counter()
        call()
        t.append(time.perf_counter() - t0)
    med = float(np.median(t)) * (heads // h)
    return med, kind, f"{'one KV head group (' + str(h) + ' query heads) scaled x' + str(heads // h) if seq_q > 1 else 'the whole call'}, " \
                      f"median of {reps} after 1 warm-up ({med * 1e3:.2f} ms per call, host has {os.cpu_count()} logical cores)"


DENSE_WORKLOADS = {   # name: (m, n, k, B given as [n, k] (x . W^T)); fp32 operands on the fp32 matrix instruction
    "dense_f32_4096x4096x4096": (4096, 4096, 4096, False),
    "dense_f32_wt_512x4096x4096": (512, 4096, 4096, True),
    "dense_f32_wt_2048x11008x4096": (2048, 11008, 4096, True),
}
MFMA_F32_PEAK_TFLOPS = 157.3


def bench_dense(a):
    """Dense fp32 matmul of the kernel SPI (Fp32MatmulKernel / Fp32MatmulWtKernel) on resident operands."""
    import torch
    from skainet_amd import _lib, kernels
    m, n, k, wt = DENSE_WORKLOADS[a.workload]
    steps = 20 if a.steps == 2000 else a.steps
    warmup = 3 if a.warmup == 200 else a.warmup
    gen = torch.Generator(device="cuda").manual_seed(20251125)
    x = torch.randn((m, k), device="cuda", generator=gen)
    w = torch.randn((n, k) if wt else (k, n), device="cuda", generator=gen)
    out = torch.empty((m, n), device="cuda")

    def call():
        if wt:
            kernels.fp32_matmul_wt_dev(x, 0, w, 0, out, 0, m, n, k)
        else:
            kernels.fp32_matmul_dev(x, 0, k, w, 0, n, out, 0, n, m, n, k)

    call()
    kernels.sync()
    kernel = kernels.last_kernel()

    def timed(count):
        if a.no_graph:
            with kernels.Timer() as t:
                for _ in range(count):
                    call()
            return t.ms
        with kernels.Graph() as g:
            for _ in range(count):
                call()
        g.launch(); g.sync()
        with kernels.Timer() as t:
            g.launch()
        g.close()
        return t.ms

    if warmup > 0:
        timed(warmup)
    t0 = time.perf_counter()
    ms_per_step = timed(steps) / steps
    wall = time.perf_counter() - t0
    rows = torch.arange(0, m, max(1, m // 64), device="cuda")
    want = x[rows].double() @ (w.double().T if wt else w.double())
    err = float(((out[rows].double() - want).abs().max() / want.abs().max()).cpu())
    tol = 1e-5
    flops = 2.0 * m * n * k
    tf = flops / (ms_per_step * 1e-3) / 1e12
    out_json = {
        "metric": "dense fp32 matmul TFLOP/s", "value": round(tf, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_per_step, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": a.workload, "m": m, "n": n, "k": k, "b_layout": "[n, k]" if wt else "[k, n]",
                   "launch": "host loop" if a.no_graph else "hip-graph replay"},
        "roofline": {"bound": "mfma", "achieved": round(tf, 2), "peak": MFMA_F32_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tf / MFMA_F32_PEAK_TFLOPS, 4), "traffic": None},
        "extra": {"flops_per_step": flops, "kernel": kernel, "wall_s_timed_region": round(wall, 4),
                  "max_err_over_max_vs_torch_fp64_on_sampled_rows": err, "device": _lib.hip().skainet_hip_device_name().decode()},
    }
    if err > tol:
        out_json["extra"]["PARITY_FAILED"] = True
    if not a.skip_cpu:
        # the reference's own C library on a bounded sample of the same product: the first rows of A, all of B
        from oracle import lib as L
        ref = L.ref()
        if ref is not None:
            ms_ = max(8, min(m, int(2.0e9 / (n * k)) or 1))
            xa = np.ascontiguousarray(x[:ms_].cpu().numpy())
            wa = np.ascontiguousarray(w.cpu().numpy())
            oa = np.empty((ms_, n), np.float32)
            fn = (lambda: ref.skainet_fp32_matmul_wt(L.fp(xa), 0, L.fp(wa), 0, L.fp(oa), 0, ms_, n, k)) if wt else \
                 (lambda: ref.skainet_fp32_matmul(L.fp(xa), 0, k, L.fp(wa), 0, n, L.fp(oa), 0, n, ms_, n, k))
            fn()
            ts = []
            t_end = time.perf_counter() + 10.0
            while len(ts) < 3 or (time.perf_counter() < t_end and len(ts) < 20):
                t1 = time.perf_counter(); fn(); ts.append(time.perf_counter() - t1)
            med = float(np.median(ts))
            out_json["cpu_baseline"] = {"value": round(2.0 * ms_ * n * k / med / 1e12, 4), "unit": "TFLOP/s", "cores": 4, "kind": "reference",
                                        "sample": f"the first {ms_} rows of A against all of B, median of {len(ts)} calls of the reference's C entry ({med * 1e3:.1f} ms)"}
    print(json.dumps(out_json).replace("NaN", "null"))
    sys.exit(0 if err <= tol else 1)


def bench_attention(a):
    rec, ok = measure_attention(a.workload, a.steps, a.warmup, a.no_graph, a.skip_cpu)
    print(json.dumps(rec).replace("NaN", "null"))
    sys.exit(0 if ok else 1)


def measure_attention(workload, steps_arg, warmup_arg, no_graph, skip_cpu):
    """Fused causal GQA attention, fp32 operands: prefill at 2048 (MFMA-class, flops counted dense as the reference's
    scenarios do) and one-token decode against a 4096-long KV cache (HBM-bound: K and V are read once). Returns
    (record, ok)."""
    import torch
    from types import SimpleNamespace
    from skainet_amd import _lib, kernels
    a = SimpleNamespace(workload=workload, steps=steps_arg, warmup=warmup_arg, no_graph=no_graph, skip_cpu=skip_cpu)
    batch, sq, skv = ATTENTION_WORKLOADS[a.workload][:3]
    window = ATTENTION_WORKLOADS[a.workload][3] if len(ATTENTION_WORKLOADS[a.workload]) > 3 else 0
    heads, kvh, d = 32, 8, 128
    scale = float(1.0 / np.sqrt(d))
    decode = sq == 1
    steps = (2000 if decode else 20) if a.steps == 2000 else a.steps
    warmup = (200 if decode else 3) if a.warmup == 200 else a.warmup
    gen = torch.Generator(device="cuda").manual_seed(20251125)
    q = torch.randn((batch, heads, sq, d), device="cuda", generator=gen)
    kv_bytes = 2 * batch * kvh * skv * d * 4
    copies = max(2, -(-2 * LLC_BYTES // kv_bytes) + 1) if decode else 1
    ks = [torch.randn((batch, kvh, skv, d), device="cuda", generator=gen) for _ in range(copies)]
    vs = [torch.randn((batch, kvh, skv, d), device="cuda", generator=gen) for _ in range(copies)]
    out = torch.empty_like(q)

    def call(i):
        kernels.sdpa_dev(q, ks[i % copies], vs[i % copies], out, batch, heads, kvh, sq, skv, d, scale, True, window)

    call(0)                                   # sizes the library's scratch before any capture
    kernels.sync()

    def timed(n):
        if a.no_graph:
            with kernels.Timer() as t:
                for i in range(n):
                    call(i)
            return t.ms
        with kernels.Graph() as g:
            for i in range(n):
                call(i)
        g.launch(); g.sync()
        with kernels.Timer() as t:
            g.launch()
        g.close()
        return t.ms

    if warmup > 0:
        timed(warmup)
    t0 = time.perf_counter()
    ms = timed(steps)
    wall = time.perf_counter() - t0
    ms_per_step = ms / steps
    # sanity: torch's fp32 attention on the same operands (textbook softmax(QK^T)V with the causal rule)
    call(0)
    kernels.sync()
    kk, vv = ks[0].repeat_interleave(heads // kvh, 1), vs[0].repeat_interleave(heads // kvh, 1)
    sc = torch.matmul(q.double(), kk.double().transpose(-1, -2)) * scale
    if not decode:
        keep = torch.ones(sq, skv, dtype=torch.bool, device="cuda").tril(skv - sq)
        if window > 0:
            keep &= torch.ones(sq, skv, dtype=torch.bool, device="cuda").triu(skv - sq - window + 1)
        sc = sc.masked_fill(~keep, -1e30)
    want = torch.matmul(torch.softmax(sc, -1), vv.double())
    err = float(((out.double() - want).abs().max() / want.abs().max()).cpu())
    tol = 2e-2
    del sc, kk, vv, want
    flops_dense = 4.0 * batch * heads * sq * skv * d
    alg_bytes = kv_bytes + 2 * q.numel() * 4
    if decode:
        gbs = alg_bytes / (ms_per_step * 1e-3) / 1e9
        value, unit, metric = gbs, "GB/s", "decode attention GB/s"
        roof = {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": measured_traffic(a.workload, kernels.last_kernel())}
    else:
        tf = flops_dense / (ms_per_step * 1e-3) / 1e12
        # attended (query, key) pairs under the causal rule and the window: what a kernel that skips the rest has to do
        useful_pairs = sum(min(qi + skv - sq + 1, window if window > 0 else skv) for qi in range(sq))
        value, unit, metric = tf, "TFLOP/s", "prefill attention TFLOP/s (dense-counted)"
        peak = MFMA_BF16_PEAK_TFLOPS if ATTENTION_PREFILL_USES_MFMA else FP32_VECTOR_PEAK_TFLOPS
        roof = {"bound": "mfma", "achieved": round(tf, 2), "peak": peak, "unit": "TFLOP/s", "frac": round(tf / peak, 4),
                "traffic": measured_traffic(a.workload, kernels.last_kernel())}
    out_json = {
        "metric": metric, "value": round(value, 2), "unit": unit, "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_per_step, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if decode or not ATTENTION_PREFILL_USES_MFMA else "bf16 x bf16 -> f32", "data": "synthetic",
        "config": {"workload": a.workload, "batch": batch, "heads": heads, "kv_heads": kvh, "head_dim": d, "seq_q": sq,
                   "seq_kv": skv, "causal": True, "window": window, "kv_copies_rotated": copies,
                   "launch": "host loop" if a.no_graph else "hip-graph replay"},
        "roofline": roof,
        "extra": {"algorithmic_bytes_per_step": alg_bytes, "flops_dense_per_step": flops_dense,
                  "flops_causal_useful_per_step": flops_dense if decode else 4.0 * batch * heads * d * useful_pairs,
                  "wall_s_timed_region": round(wall, 4), "max_err_over_max_vs_torch_fp64": err,
                  "device": _lib.hip().skainet_hip_device_name().decode()},
    }
    if err > tol:
        out_json["extra"]["PARITY_FAILED"] = True
    if not a.skip_cpu:
        med, kind, sample = cpu_baseline_attention(batch, sq, skv, heads, kvh, d, scale, window)
        cpu_val = alg_bytes / med / 1e9 if decode else flops_dense / med / 1e12
        # the reference threads its attention rows over at most 4 pool participants once there are >= 512 rows
        cores = 4 if (kind == "reference" and not decode) else 1
        out_json["cpu_baseline"] = {"value": round(cpu_val, 4), "unit": unit, "cores": cores, "kind": kind, "sample": sample}
    del ks, vs, q, out
    torch.cuda.empty_cache()
    return out_json, err <= tol


def measure_decoder(workload, steps, warmup, no_graph, skip_cpu):
    """Synthetic Llama-3-8B-shape stack: prefill of 512 random token ids, then greedy decode; a step = one decoded token.
    Returns (record, ok)."""
    from dataclasses import replace
    from skainet_amd import _lib, kernels
    from skainet_amd.decoder import LLAMA3_8B, LlamaDecoder, LlamaWeights
    overrides, prompt_len, distinct = DECODER_WORKLOADS[workload]
    cfg = replace(LLAMA3_8B, **overrides)
    t0 = time.perf_counter()
    w = LlamaWeights(cfg, seed=20251125, keep_host=not skip_cpu, distinct_layers=distinct)
    t_weights = time.perf_counter() - t0
    dec = LlamaDecoder(w, max_prefill=prompt_len)
    prompt = np.random.default_rng(7).integers(0, cfg.vocab, prompt_len)
    dec.prefill(prompt)                      # warm-up pass: sizes the library's scratch
    kernels.sync()
    with kernels.Timer() as t:
        first = dec.prefill(prompt)
    prefill_ms = t.ms
    toks = [first] + [int(x) for x in dec.decode(max(1, warmup), use_graph=not no_graph)]
    kernels.sync()
    pos0 = dec.position()
    if pos0 + steps > cfg.ctx_max:
        raise SystemExit(f"bench.py: {steps} decode steps from position {pos0} would pass the context limit {cfg.ctx_max}")

    def timed_steps(count):
        with kernels.Timer() as tm:          # HIP events on the launch stream around exactly `count` decode steps
            dec.run_steps(count, use_graph=not no_graph)
        return tm.ms

    t0 = time.perf_counter()
    ms = timed_steps(steps)
    wall = time.perf_counter() - t0
    assert dec.position() == pos0 + steps
    generated = dec.generated_tokens()
    ms_per_tok = ms / steps
    ctx_mid = pos0 + steps // 2
    alg = w.decode_bytes_per_token(ctx_mid)
    gbs = alg / (ms_per_tok * 1e-3) / 1e9
    # sanity of the timed path: the last emitted token is the first arg-max of the logits left on the device
    logits = dec.last_logits()
    ok = bool(np.isfinite(logits).all()) and int(np.argmax(logits)) == int(generated[-1])
    # the same step at the far end of the context: walk the cache up to the limit, time the last steps
    late = min(steps, 64)
    gap = cfg.ctx_max - late - dec.position()
    late_ms = None
    if gap >= 0:
        if gap > 0:
            timed_steps(gap)
        late_pos0 = dec.position()
        late_ms = timed_steps(late) / late
        ok = ok and dec.position() == late_pos0 + late == cfg.ctx_max
        lg = dec.last_logits()
        ok = ok and bool(np.isfinite(lg).all()) and int(np.argmax(lg)) == int(dec.generated_tokens()[-1])
    rec = {
        "metric": "decode tok/s", "value": round(1e3 / ms_per_tok, 2), "unit": "tok/s", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": round(ms_per_tok, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32 (packed Q4_K / Q6_K weights)", "data": "synthetic",
        "config": {"workload": workload, "layers": cfg.layers, "hidden": cfg.hidden, "heads": cfg.heads,
                   "kv_heads": cfg.kv_heads, "head_dim": cfg.head_dim, "ffn": cfg.ffn, "vocab": cfg.vocab, "batch": 1,
                   "prompt_tokens": prompt_len, "decoded_tokens": steps, "context_at_end": pos0 + steps,
                   "weights": f"random init N(0, 0.02^2), Q4_K linears + Q6_K head; {distinct} layer(s) of distinct values, "
                              f"every layer in its own HBM allocation",
                   "launch": "host loop" if no_graph else "hip-graph replay of one decode step"},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None},
        "extra": {"algorithmic_bytes_per_token": alg, "packed_weight_bytes": w.packed_bytes(),
                  "prefill_ms": round(prefill_ms, 3), "prefill_tok_per_s": round(prompt_len / (prefill_ms * 1e-3), 1),
                  "hbm_bound_ms_per_token": round(alg / (HBM_PEAK_GBS * 1e9) * 1e3, 5),
                  "ms_per_token_at_context_limit": None if late_ms is None else round(late_ms, 5),
                  "context_limit": cfg.ctx_max,
                  "wall_s_timed_region": round(wall, 4), "weight_build_s": round(t_weights, 1),
                  "first_tokens": toks[:8], "device": _lib.hip().skainet_hip_device_name().decode()},
    }
    if not ok:
        rec["extra"]["PARITY_FAILED"] = True
    if not skip_cpu:
        rec["cpu_baseline"] = cpu_baseline_decode(cfg, w.host, ctx_mid)
    dec.close()
    return rec, ok


def measure_decoder_spi(workload, steps, warmup):
    """The decode step of `measure_decoder` with every operand a host array: each linear is one call of the library's
    host-array product (upload, launch, download, wait), attention and the norms go through the SPI's host kernels, the
    rest runs in numpy. The prompt is prefilled by the resident decoder and its KV cache handed over, so the timed
    steps run at the same context. A step = one decoded token, timed on the host clock (every call ends in a wait)."""
    from dataclasses import replace
    from skainet_amd import _lib, kernels
    from skainet_amd.decoder import LLAMA3_8B, LlamaDecoder, LlamaWeights
    from skainet_amd.spi_decoder import SpiDecoder
    overrides, prompt_len, distinct = DECODER_WORKLOADS[SPI_DECODER_WORKLOADS[workload]]
    cfg = replace(LLAMA3_8B, **overrides)
    w = LlamaWeights(cfg, seed=20251125, distinct_layers=distinct)
    dec = LlamaDecoder(w, max_prefill=prompt_len)
    prompt = np.random.default_rng(7).integers(0, cfg.vocab, prompt_len)
    first = dec.prefill(prompt)
    spi = SpiDecoder(w)
    shape = (cfg.layers, cfg.kv_heads, cfg.ctx_max, cfg.head_dim)
    spi.k_cache[...] = dec.k_cache.download(np.float32, int(np.prod(shape))).reshape(shape)
    spi.v_cache[...] = dec.v_cache.download(np.float32, int(np.prod(shape))).reshape(shape)
    spi.pos, spi.token = prompt_len, first
    # parity of the timed route: same token in, logits within the fp32 bar of the resident decoder's
    resident_next = int(dec.decode(1, use_graph=False)[0])
    spi.step(first)
    ref = dec.last_logits().astype(np.float64)
    err = float(np.abs(spi.logits[0] - ref).max() / np.abs(ref).max())
    ok = err < 1e-3 and bool(np.isfinite(spi.logits).all())
    spi.token = resident_next
    for _ in range(max(0, warmup - 1)):
        spi.step(spi.token)
    spi.matmul_seconds, spi.attention_seconds, spi.matmul_calls, spi.calls = 0.0, 0.0, 0, 0
    pos0 = spi.pos
    t0 = time.perf_counter()
    spi.decode(steps)
    wall = time.perf_counter() - t0
    ms_per_tok = wall * 1e3 / steps
    # the resident decoder at the same context, for the comparison
    dec.decode(max(1, warmup), use_graph=True)
    with kernels.Timer() as tm:
        dec.run_steps(64)
    resident_ms = tm.ms / 64
    linears = 4 * cfg.layers + 1
    us_call = spi.matmul_seconds / spi.matmul_calls * 1e6
    alg = w.decode_bytes_per_token(pos0 + steps // 2)
    gbs = alg / (ms_per_tok * 1e-3) / 1e9
    rec = {
        "metric": "decode tok/s", "value": round(1e3 / ms_per_tok, 2), "unit": "tok/s", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": round(ms_per_tok, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32 (packed Q4_K / Q6_K weights)", "data": "synthetic",
        "config": {"workload": workload, "layers": cfg.layers, "hidden": cfg.hidden, "heads": cfg.heads,
                   "kv_heads": cfg.kv_heads, "head_dim": cfg.head_dim, "ffn": cfg.ffn, "vocab": cfg.vocab, "batch": 1,
                   "prompt_tokens": prompt_len, "decoded_tokens": steps, "context_at_end": pos0 + steps,
                   "route": "kernel SPI with host arrays: weights resident, activations / KV cache / results on the host; "
                            "driven from Python over ctypes"},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None},
        "extra": {"boundary_calls_per_token": spi.calls // steps, "linear_calls_per_token": linears,
                  "us_per_linear_call": round(us_call, 2),
                  "ms_per_token_in_linears": round(spi.matmul_seconds * 1e3 / steps, 4),
                  "ms_per_token_in_attention_calls": round(spi.attention_seconds * 1e3 / steps, 4),
                  "resident_ms_per_token_same_context": round(resident_ms, 5),
                  "us_per_linear_resident_upper_bound": round(resident_ms * 1e3 / linears, 2),
                  "host_overhead_us_per_linear": round(us_call - resident_ms * 1e3 / linears, 2),
                  "logits_err_vs_resident": err, "device": _lib.hip().skainet_hip_device_name().decode()},
    }
    if not ok:
        rec["extra"]["PARITY_FAILED"] = True
    spi.close()
    dec.close()
    return rec, ok


def measure_decoder_ops(workload, steps, warmup, no_graph):
    """The decode step of `measure_decoder` through skainet_amd.ops.HipOps alone: what a model built with the NN DSL costs
    when its TensorOps keeps activations resident -- 17 device entries per layer instead of the fused decoder's 5, every
    intermediate a device tensor, the step recorded into a HIP graph. The fused decoder runs beside it on the same
    weights: same prompt, logits compared, and its time per token at the same context for the comparison."""
    from dataclasses import replace
    from skainet_amd import _lib, kernels
    from skainet_amd.decoder import LLAMA3_8B, LlamaDecoder, LlamaWeights
    from skainet_amd.ops_decoder import OpsLlamaDecoder, OpsLlamaWeights
    overrides, prompt_len, distinct = DECODER_WORKLOADS[OPS_DECODER_WORKLOADS[workload]]
    cfg = replace(LLAMA3_8B, **overrides)
    w = LlamaWeights(cfg, seed=20251125, distinct_layers=distinct)
    ow = OpsLlamaWeights(w)
    prompt = np.random.default_rng(7).integers(0, cfg.vocab, prompt_len)
    fused = LlamaDecoder(w, max_prefill=prompt_len)
    first_fused = fused.prefill(prompt)
    dec = OpsLlamaDecoder(ow, max_prefill=prompt_len)
    dec.prefill(prompt)                      # warm-up pass: sizes the library's scratch
    kernels.sync()
    with kernels.Timer() as t:
        first = dec.prefill(prompt)
    prefill_ms = t.ms
    ref = fused.last_logits().astype(np.float64)
    err = float(np.abs(dec.last_logits() - ref).max() / np.abs(ref).max())       # both prefills run the bf16 MFMA GEMM
    ok = err < 2e-2 and bool(np.isfinite(dec.last_logits()).all())
    dec.decode(max(1, warmup), use_graph=not no_graph)
    fused.decode(max(1, warmup), use_graph=not no_graph)
    pos0 = dec.position()
    with kernels.Timer() as tm:
        dec.run_steps(steps, use_graph=not no_graph)
    ms_per_tok = tm.ms / steps
    with kernels.Timer() as tm:
        fused.run_steps(steps, use_graph=not no_graph)
    fused_ms = tm.ms / steps
    lg = dec.last_logits()
    ok = ok and bool(np.isfinite(lg).all()) and dec.position() == pos0 + steps
    alg = w.decode_bytes_per_token(pos0 + steps // 2)
    gbs = alg / (ms_per_tok * 1e-3) / 1e9
    rec = {
        "metric": "decode tok/s", "value": round(1e3 / ms_per_tok, 2), "unit": "tok/s", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": round(ms_per_tok, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32 (packed Q4_K / Q6_K weights)", "data": "synthetic",
        "config": {"workload": workload, "layers": cfg.layers, "hidden": cfg.hidden, "heads": cfg.heads,
                   "kv_heads": cfg.kv_heads, "head_dim": cfg.head_dim, "ffn": cfg.ffn, "vocab": cfg.vocab, "batch": 1,
                   "prompt_tokens": prompt_len, "decoded_tokens": steps, "context_at_end": pos0 + steps,
                   "route": "generic resident-activation ops class (HipOps): one device entry per tensor op, activations "
                            "and KV cache resident, nothing fused by name",
                   "launch": "host loop" if no_graph else "hip-graph replay of one decode step"},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None},
        "extra": {"device_entries_per_token": dec.launches_per_token(), "prefill_ms": round(prefill_ms, 3),
                  "fused_decoder_ms_per_token_same_context": round(fused_ms, 5),
                  "prefill_logits_err_vs_fused_decoder": err, "first_token_equals_fused": bool(first == first_fused),
                  "algorithmic_bytes_per_token": alg, "device": _lib.hip().skainet_hip_device_name().decode()},
    }
    if not ok:
        rec["extra"]["PARITY_FAILED"] = True
    dec.close()
    fused.close()
    return rec, ok


UPLOAD_WORKLOADS = {"weight_upload_q4k_528mb": ("Q4_K", 229376, 4096)}   # name: (encoding, rows, cols)
PCIE_PEAK_GBS = 64.0   # PCIe 5.0 x16, one direction, before protocol overhead


def bench_upload(a):
    """Host -> device rate of skainet_hip_weight_upload on one large packed weight (the bytes are never interpreted, so
    they are random): from pageable memory through the library's page-locked chunks at the default setting and with the
    staging off (one blocking copy), and from page-locked memory. A step is one upload; the best of `steps` is reported
    (the host's page cache and clocks make the first calls slower), and the device copy is compared byte for byte."""
    from skainet_amd import _lib, kernels
    enc, rows, cols = UPLOAD_WORKLOADS[a.workload]
    bs, nb = {"Q4_K": (256, 144)}[enc]
    nbytes = rows * (cols // bs) * nb
    steps = 6 if a.steps == 2000 else a.steps
    src = np.random.default_rng(3).integers(0, 256, nbytes, dtype=np.uint8)
    back = np.empty(nbytes, np.uint8)

    def rate(arr, check):
        best, ok = float("inf"), True
        for i in range(steps):
            t0 = time.perf_counter()
            w = kernels.DeviceWeight.upload(enc, arr, rows, cols)
            best = min(best, time.perf_counter() - t0)
            if check and i == 0:
                assert _lib.hip().skainet_hip_memcpy_d2h(back.ctypes.data, w.data_ptr, nbytes) == 0
                ok = bool(np.array_equal(back, src))
            w.close()
        return nbytes / best / 1e9, best, ok

    staged, best, ok = rate(src, True)
    kernels.set_tuning("upload_chunk_mib", 0)
    blocking, _, _ = rate(src, False)
    kernels.set_tuning("upload_chunk_mib", 8)
    pinned = kernels.PinnedBytes(nbytes)
    pinned.array[:] = src
    locked, _, ok2 = rate(pinned.array, True)
    pinned.close()
    t0 = time.perf_counter()
    back[:] = src
    host_copy = nbytes / (time.perf_counter() - t0) / 1e9
    rec = {
        "metric": "weight upload GB/s (pageable source)", "value": round(staged, 2), "unit": "GB/s", "n_gpus": 1, "steps": steps,
        "warmup": 0, "ms_per_step": round(best * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "config": {"workload": a.workload, "encoding": enc, "rows": rows, "cols": cols, "bytes": nbytes,
                   "timing": f"best of {steps} uploads, host clock around the call (it returns when the bytes are on the device)"},
        "roofline": {"bound": "pcie", "achieved": round(staged, 2), "peak": PCIE_PEAK_GBS, "unit": "GB/s",
                     "frac": round(staged / PCIE_PEAK_GBS, 4), "traffic": None},
        "extra": {"one_blocking_copy_GBps": round(blocking, 2), "page_locked_source_GBps": round(locked, 2),
                  "host_memcpy_one_core_GBps": round(host_copy, 2), "device": _lib.hip().skainet_hip_device_name().decode()},
    }
    if not (ok and ok2):
        rec["extra"]["PARITY_FAILED"] = True
    print(json.dumps(rec))
    sys.exit(0 if ok and ok2 else 1)


def bench_decoder(a):
    if a.workload in OPS_DECODER_WORKLOADS:
        rec, ok = measure_decoder_ops(a.workload, 64 if a.steps == 2000 else a.steps, 4 if a.warmup == 200 else a.warmup, a.no_graph)
        print(json.dumps(rec).replace("NaN", "null"))
        sys.exit(0 if ok else 1)
    if a.workload in SPI_DECODER_WORKLOADS:
        rec, ok = measure_decoder_spi(a.workload, 32 if a.steps == 2000 else a.steps, 4 if a.warmup == 200 else a.warmup)
        print(json.dumps(rec).replace("NaN", "null"))
        sys.exit(0 if ok else 1)
    steps = 128 if a.steps == 2000 else a.steps
    warmup = 8 if a.warmup == 200 else a.warmup
    rec, ok = measure_decoder(a.workload, steps, warmup, a.no_graph, a.skip_cpu)
    print(json.dumps(rec).replace("NaN", "null"))
    sys.exit(0 if ok else 1)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000, help="timed steps (default 2000; 200 for the GEMM workloads)")
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", default="q4k_gemv_11008x4096_b1", choices=sorted(WORKLOADS) + sorted(DECODER_WORKLOADS) + sorted(SPI_DECODER_WORKLOADS) + sorted(OPS_DECODER_WORKLOADS) + sorted(ATTENTION_WORKLOADS) + sorted(DENSE_WORKLOADS) + sorted(UPLOAD_WORKLOADS))
    ap.add_argument("--no-graph", action="store_true", help="launch from the host loop instead of replaying a HIP graph")
    ap.add_argument("--skip-cpu", action="store_true", help="omit the CPU baseline (profiling runs)")
    ap.add_argument("--hbm-only", action="store_true", help="skip the cache-warm pass and the read probe, so every launch of the "
                    "kernel in a profile is one of the rotating-copy (HBM) kind")
    ap.add_argument("--no-headline", action="store_true", help="default workload only: skip the GEMM and decoder measurements "
                    "that the default run adds under extra.headline")
    ap.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE", help="launch-shape knob (skainet_hip_set_tuning)")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this backend is a single-GPU kernel library (no collectives); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from skainet_amd import _lib, kernels
    if not kernels.is_available():
        print("bench.py: HIP backend unavailable: " + _lib.last_error(), file=sys.stderr)
        sys.exit(1)
    for kv in a.tune:
        key, _, val = kv.partition("=")
        _lib.check(_lib.hip().skainet_hip_set_tuning(key.encode(), int(val)), "set_tuning")

    if a.workload in DECODER_WORKLOADS or a.workload in SPI_DECODER_WORKLOADS or a.workload in OPS_DECODER_WORKLOADS:
        bench_decoder(a)
    if a.workload in UPLOAD_WORKLOADS:
        return bench_upload(a)
    if a.workload in DENSE_WORKLOADS:
        return bench_dense(a)
    if a.workload in ATTENTION_WORKLOADS:
        return bench_attention(a)
    default_run = a.workload == "q4k_gemv_11008x4096_b1" and not a.no_headline
    out, ok = measure_matmul(a.workload, a.steps, a.warmup, not a.no_graph, a.hbm_only, a.skip_cpu)
    if default_run:
        # the other two parts of the headline metric, same process, same device
        headline = {}
        g_steps, g_warm = (200, 20) if a.steps == 2000 else (a.steps, a.warmup)
        rec, g_ok = measure_matmul("q4k_gemm_512x4096x4096", g_steps, g_warm, not a.no_graph, True, True)
        headline["q4k_gemm_512x4096x4096"] = {
            "metric": rec["metric"], "value": rec["value"], "unit": rec["unit"], "ms_per_step": rec["ms_per_step"],
            "steps": rec["steps"], "frac_of_bf16_mfma_peak": rec["roofline"]["frac"], "traffic": rec["roofline"]["traffic"],
            "dtype": rec["dtype"], "parity_ok": g_ok, "max_err_over_max": rec["extra"]["max_normalized_err_vs_fp64_decode_matmul"],
            "kernel": rec["extra"]["kernel"]}
        # the config's own 128 decoded tokens, whatever --steps says (a shorter run is a different workload)
        rec, d_ok = measure_decoder("llama3_8b_decode", 128, 8, a.no_graph, True)
        headline["llama3_8b_decode"] = {
            "metric": rec["metric"], "value": rec["value"], "unit": rec["unit"], "ms_per_token": rec["ms_per_step"],
            "steps": rec["steps"], "frac_of_hbm_peak": rec["roofline"]["frac"], "prefill_ms": rec["extra"]["prefill_ms"],
            "prefill_tok_per_s": rec["extra"]["prefill_tok_per_s"], "context_at_end": rec["config"]["context_at_end"],
            "ms_per_token_at_context_limit": rec["extra"]["ms_per_token_at_context_limit"],
            "context_limit": rec["extra"]["context_limit"], "dtype": rec["dtype"], "self_check_ok": d_ok,
            "weights": rec["config"]["weights"]}
        ok = ok and g_ok and d_ok
        # the remaining configurations of the baseline, each with the parity flag of its own fp64 check
        short = a.steps != 2000
        for wl in ("q8_0_gemv_4096x4096_b1", "q4k_gemv_11008x4096_b4", "q4k_gemv_11008x4096_b8", "q6k_gemm_512x32000x4096"):
            gemm = WORKLOADS[wl][3] > 8
            st, wu = ((100, 10) if gemm else (1000, 100)) if not short else (a.steps, a.warmup)
            rec, w_ok = measure_matmul(wl, st, wu, not a.no_graph, True, True)
            headline[wl] = {"metric": rec["metric"], "value": rec["value"], "unit": rec["unit"], "ms_per_step": rec["ms_per_step"],
                            "steps": rec["steps"], "frac": rec["roofline"]["frac"], "bound": rec["roofline"]["bound"],
                            "traffic": rec["roofline"]["traffic"], "dtype": rec["dtype"], "kernel": rec["extra"]["kernel"],
                            "parity_ok": w_ok, "max_err": rec["extra"]["max_normalized_err_vs_fp64_decode_matmul"]}
            ok = ok and w_ok
        for wl in ("sdpa_prefill_2048", "sdpa_decode_4096_b1", "sdpa_decode_4096_b8"):
            decode = ATTENTION_WORKLOADS[wl][1] == 1
            st, wu = ((1000, 100) if decode else (20, 3)) if not short else (a.steps, a.warmup)
            rec, w_ok = measure_attention(wl, st, wu, a.no_graph, True)
            headline[wl] = {"metric": rec["metric"], "value": rec["value"], "unit": rec["unit"], "ms_per_step": rec["ms_per_step"],
                            "steps": rec["steps"], "frac": rec["roofline"]["frac"], "bound": rec["roofline"]["bound"],
                            "traffic": rec["roofline"]["traffic"], "dtype": rec["dtype"], "parity_ok": w_ok,
                            "max_err": rec["extra"]["max_err_over_max_vs_torch_fp64"]}
            ok = ok and w_ok
        out["extra"]["headline"] = headline
    print(json.dumps(out).replace("NaN", "null"))
    sys.exit(0 if ok else 1)


def measure_matmul(workload, steps, warmup, graph, hbm_only, skip_cpu):
    """One packed-weight product workload (GEMV for batch <= 8, the MFMA dequant-GEMM above); returns (record, ok)."""
    import torch
    from skainet_amd import _lib, kernels
    enc, n, k, m = WORKLOADS[workload]
    rng = np.random.default_rng(20251125)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    packed = kernels.quantize(enc, w)
    del w
    alg = algorithmic_bytes(enc, n, k, m)

    copies = max(2, -(-2 * LLC_BYTES // packed.size) + 1)
    base = torch.from_numpy(packed).cuda()
    store = [base] + [base.clone() for _ in range(copies - 1)]
    weights = [kernels.DeviceWeight.wrap(enc, t, n, k) for t in store]
    xd = torch.from_numpy(x).cuda()
    yd = torch.empty((m, n), dtype=torch.float32, device="cuda")
    kind = 0 if m <= 8 else 1
    is_gemm = kind == 1
    if is_gemm and steps == 2000:
        steps, warmup = 200, 20
    weights[0].matmul(xd, m, yd, kind)      # sizes the library's scratch before any stream capture
    torch.cuda.synchronize()
    kernel = kernels.last_kernel()
    replays = 5 if steps <= 500 else 3

    def run(ws, iters):
        torch.cuda.synchronize()
        ms = kernels.matmul_repeat(ws, xd, m, yd, iters, kind, graph, replays)
        torch.cuda.synchronize()
        return ms

    if warmup > 0:
        run(weights, warmup)
    t0 = time.perf_counter()
    ms = run(weights, steps)                # exactly K steps per timed pass, HIP events on the launch stream, median of 5 passes
    wall = time.perf_counter() - t0
    ms_probe = float("nan")
    if hbm_only:
        ms_warm = float("nan")
    else:
        ms_warm = run(weights[:1], steps)     # same K steps on one copy: served by the memory-side cache
    # ceiling for a read-once pass over the same rotating copies: a kernel that only loads (no arithmetic)
    probe_iters = min(max(steps, 100), 500)
    if not hbm_only:
        ms_probe = min(kernels.read_probe(store, packed.size, probe_iters, g) for g in (256, 512, 2048))
    gbs_probe = packed.size / (ms_probe / probe_iters * 1e-3) / 1e9
    ms_per_step = ms / steps
    gbs = alg / (ms_per_step * 1e-3) / 1e9
    gbs_warm = alg / (ms_warm / steps * 1e-3) / 1e9

    # sanity: the timed path computed the right thing -- compare with the device decode (bit-exact kernel) times x in fp64
    dense = torch.empty((n, k), dtype=torch.float32, device="cuda")
    weights[0].dequantize(dense)
    want = (dense.double() @ xd[0].double()).cpu().numpy()
    got = yd[0].cpu().numpy()
    floor = 1.0 if is_gemm else 1e-2        # bf16 operands: error taken against the largest output
    err = float((np.abs(got - want) / np.maximum(np.abs(want), floor * np.abs(want).max())).max())
    tol = 2e-2 if is_gemm else 1e-3
    del dense

    flops = 2.0 * m * n * k
    tflops = flops / (ms_per_step * 1e-3) / 1e12
    traffic = measured_traffic(workload, kernel)
    out = {
        "metric": f"{enc} GEMM TFLOP/s" if is_gemm else f"{enc} GEMV GB/s",
        "value": round(tflops if is_gemm else gbs, 2), "unit": "TFLOP/s" if is_gemm else "GB/s", "n_gpus": 1,
        "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_per_step, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 x bf16 -> f32" if is_gemm else ("i8 x i8 -> i32 -> f32" if kernel == "q4k_gemv_mfma_kernel" else "f32"),
        "data": "synthetic",
        "config": {"workload": workload, "encoding": enc, "rows": n, "cols": k, "batch": m,
                   "weight_copies_rotated": copies, "launch": "hip-graph replay" if graph else "host loop",
                   "timing": f"median of {replays} timed passes of {steps} steps each, inside one chain of launches behind 400 untimed ones"},
        "roofline": ({"bound": "mfma", "achieved": round(tflops, 2), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                      "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": traffic}
                     if is_gemm else
                     {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                      "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": traffic}),
        "extra": {"algorithmic_bytes_per_step": alg, "kernel": kernel, "cache_warm_GBps": round(gbs_warm, 2),
                  "cache_warm_ms_per_step": round(ms_warm / steps, 6), "pct_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2),
                  "read_only_probe_GBps_same_buffers": round(gbs_probe, 2),
                  "frac_of_read_only_probe": round(gbs / gbs_probe, 4),
                  "wall_s_timed_region": round(wall, 4), "max_normalized_err_vs_fp64_decode_matmul": err,
                  "device": _lib.hip().skainet_hip_device_name().decode()},
    }
    if is_gemm:
        out["extra"]["flops_per_step"] = flops
        out["extra"]["step_includes"] = "every launch of the product: activation pass (if any), dequant-GEMM kernel, split sum (if any)"
    if err > tol:
        out["extra"]["PARITY_FAILED"] = True
    if not skip_cpu:
        out["cpu_baseline"] = cpu_baseline(enc, n, k, m, packed, x)
    for t in store:
        del t
    del store, weights, base
    torch.cuda.empty_cache()
    return out, err <= tol


if __name__ == "__main__":
    main()
