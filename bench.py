#!/usr/bin/env python3
"""Headline benchmark: Q4_K batch-1 matvec 4096 x 11008 on one MI355X, effective HBM GB/s.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra]

A step is one matvec  y = deq(W) . x  through the C ABI (skn_matvec_q) on device-resident inputs.  The
weight of step i is copy i mod 24 of 24 distinct seeded 25.4 MB tensors (609 MB in all), so that no step
finds its weights in the 256 MB last-level cache: the figure is an HBM figure.

Output: ONE JSON line.
  value            algorithmic bytes of K steps / wall time of K steps (launch gaps included), GB/s
  roofline         algorithmic bytes of one launch / mean kernel duration (per-launch HIP events on the
                   stream the kernel runs on), against the 8 TB/s HBM peak
  cpu_baseline     the CPU oracle (C, OpenMP) on the same workload, timed on this box's host cores
  extra            the other benchmark shapes, cache-hot figures, attention and decode throughput
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from skainet_amd import runtime, synth, traffic  # noqa: E402

HBM_PEAK_GBS = 8000.0
Q8_0, Q4_K, Q6_K = 8, 12, 14
N_COPIES = 24


def matvec_bytes(qtype, n, k):
    be, bb = synth.BLOCK[qtype]
    return n * (k // be) * bb + 4 * k + 4 * n


def bench_matvec(ctx, qtype, n, k, steps, warmup, copies=N_COPIES, seed=1234):
    """-> dict with wall and per-kernel timing of `steps` matvecs rotating over `copies` weight tensors."""
    be, bb = synth.BLOCK[qtype]
    w_bytes = n * (k // be) * bb
    weights = []
    sums = []
    for c in range(copies):
        raw = synth.weight(qtype, n, k, seed=seed + c)
        if c == 0:
            sums.append(synth.checksum(raw))
        weights.append(ctx.to_device(raw))
    x = ctx.to_device(synth.activation_f32(k, seed=seed + 999))
    y = ctx.alloc(4 * n)
    for i in range(warmup):
        ctx.matvec_q(qtype, weights[i % copies], n, k, x, y)
    ctx.sync()
    # (1) wall clock over exactly `steps` steps, synchronised on both sides
    t0 = time.perf_counter()
    for i in range(steps):
        ctx.matvec_q(qtype, weights[i % copies], n, k, x, y)
    ctx.sync()
    wall = time.perf_counter() - t0
    # (2) the same steps again with per-launch start/stop events: kernel durations without launch gaps
    ctx.prof_start(steps)
    for i in range(steps):
        ctx.matvec_q(qtype, weights[i % copies], n, k, x, y)
    kernel_ms, launches = ctx.prof_stop()
    # (3) cache-hot: one weight copy only
    hot_steps = min(steps, 200)
    ctx.prof_start(hot_steps)
    for i in range(hot_steps):
        ctx.matvec_q(qtype, weights[0], n, k, x, y)
    hot_ms, hot_n = ctx.prof_stop()
    nbytes = matvec_bytes(qtype, n, k)
    res = {
        "bytes_per_launch": nbytes,
        "wall_s": wall,
        "ms_per_step": wall / steps * 1e3,
        "wall_gbs": nbytes * steps / wall / 1e9,
        "kernel_us": kernel_ms / launches * 1e3,
        "kernel_gbs": nbytes / (kernel_ms / launches * 1e-3) / 1e9,
        "hot_kernel_us": hot_ms / hot_n * 1e3,
        "hot_kernel_gbs": nbytes / (hot_ms / hot_n * 1e-3) / 1e9,
        "weight_bytes": w_bytes,
        "copies": copies,
        "checksum_copy0": sums[0],
    }
    for wbuf in weights:
        wbuf.free()
    x.free()
    y.free()
    return res


def bench_attention(ctx, steps, warmup):
    """8 sequences x 32 heads x 128 dims, 256-token pages: append one token per sequence, attend over 4096."""
    n_seq, n_head, dim, n_ctx = 8, 32, 128, 4096
    kv = ctx.kv_cache(n_seq, n_head, dim, 256, 8192)
    for s in range(n_seq):
        k = ctx.to_device(synth.kv_f16((n_ctx - 1, n_head, dim), seed=50 + s))
        v = ctx.to_device(synth.kv_f16((n_ctx - 1, n_head, dim), seed=70 + s))
        kv.append_run(s, k, v, n_ctx - 1)
        k.free()
        v.free()
    k1 = ctx.to_device(synth.kv_f16((n_seq, n_head, dim), seed=90))
    v1 = ctx.to_device(synth.kv_f16((n_seq, n_head, dim), seed=91))
    q = ctx.to_device(np.random.default_rng(92).standard_normal((n_seq, n_head, dim)).astype(np.float32))
    out = ctx.alloc(4 * n_seq * n_head * dim)
    kv.append(k1, v1, list(range(n_seq)))
    scale = 1.0 / np.sqrt(dim)
    lens = [n_ctx] * n_seq
    for _ in range(warmup):
        kv.attn_decode(q, out, scale, n_ctx=lens)
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        kv.attn_decode(q, out, scale, n_ctx=lens)
    ctx.sync()
    wall = time.perf_counter() - t0
    ctx.prof_start(4 * steps)
    for _ in range(steps):
        kv.attn_decode(q, out, scale, n_ctx=lens)
    kernel_ms, launches = ctx.prof_stop()
    nbytes = n_seq * n_head * n_ctx * dim * 2 * 2 + 2 * 4 * n_seq * n_head * dim
    kv.free()
    per_step_us = kernel_ms / steps * 1e3
    # what the memory system gives a plain stream of the same size: the dense F16 matvec over 32768 x 8192 (536 870 912
    # weight bytes, twice the last-level cache, so every launch reads memory)
    rn, rk = 32768, 8192
    wbig = ctx.alloc(2 * rn * rk)
    ctx.memset(wbig, 0x3c, 2 * rn * rk)
    xb, yb = ctx.to_device(synth.activation_f32(rk, seed=5)), ctx.alloc(4 * rn)
    for _ in range(3):
        ctx.matvec_q(1, wbig, rn, rk, xb, yb)
    ctx.prof_start(20)
    for _ in range(20):
        ctx.matvec_q(1, wbig, rn, rk, xb, yb)
    rms, rl = ctx.prof_stop()
    for b in (wbig, xb, yb):
        b.free()
    read_us = rms / rl * 1e3
    read_gbs = (2 * rn * rk + 4 * rk + 4 * rn) / (read_us * 1e-6) / 1e9
    return {
        "read_rate_same_bytes_us": read_us,
        "read_rate_same_bytes_frac": read_gbs / HBM_PEAK_GBS,
        "frac_of_read_rate": nbytes / (per_step_us * 1e-6) / 1e9 / read_gbs,
        "bytes_per_step": nbytes,
        "kernel_us_per_step": per_step_us,
        "kernel_gbs": nbytes / (per_step_us * 1e-6) / 1e9,
        "frac_hbm_peak": nbytes / (per_step_us * 1e-6) / 1e9 / HBM_PEAK_GBS,
        "wall_us_per_step": wall / steps * 1e6,
        "launches_per_step": launches / steps,
    }


MFMA_F16_PEAK_TFLOPS = 2500.0


def bench_attention_prefill(ctx, reps=20):
    """Causal attention of a 512-token prompt, 32 heads x 128 dims: 4 * T^2 / 2 * heads * dim flops of the two
    products (each done twice, on fp16 hi + lo pairs) against the dense fp16 matrix-core peak."""
    n_tok, n_head, dim = 512, 32, 128
    kv = ctx.kv_cache(1, n_head, dim, 256, 1024)
    k = ctx.to_device(synth.kv_f16((n_tok, n_head, dim), seed=150))
    v = ctx.to_device(synth.kv_f16((n_tok, n_head, dim), seed=170))
    kv.append_run(0, k, v, n_tok)
    q = ctx.to_device(np.random.default_rng(192).standard_normal((n_tok, n_head, dim)).astype(np.float32))
    out = ctx.alloc(4 * n_tok * n_head * dim)
    scale = 1.0 / np.sqrt(dim)
    for _ in range(3):
        kv.attn_prefill(0, q, n_tok, out, scale)
    ctx.sync()
    ctx.prof_start(4 * reps)
    for _ in range(reps):
        kv.attn_prefill(0, q, n_tok, out, scale)
    ms, launches = ctx.prof_stop()
    for buf in (k, v, q, out):
        buf.free()
    kv.free()
    us = ms / reps * 1e3
    flops = 4.0 * n_tok * (n_tok + 1) / 2 * n_head * dim
    return {"us_per_call": round(us, 1), "launches_per_call": launches // reps, "tflops_useful": round(flops / us / 1e6, 1),
            "frac_mfma_f16_peak": round(flops / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4)}


def bench_gemm(ctx, qtype, m, n, k, reps=20, expanded=False):
    """Prefill GEMM C[m,n] = A[m,k] . deq(W)[n,k]^T (A bf16): summed kernel time of one call (activation
    preparation included), 2mnk flops against the dense fp16 matrix-core peak.  expanded: the weight pass of the
    formats other than Q4_K done once beforehand (skn_gemm_expand, 4 bytes per weight kept on the device)."""
    w = ctx.to_device(synth.weight(qtype, n, k, seed=3))
    a = ctx.to_device(synth.activation_bf16((m, k), seed=4))
    c = ctx.alloc(4 * m * n)
    kept = ctx.gemm_expand(qtype, w, n, k) if expanded else None

    def call():
        if expanded:
            ctx.gemm_expanded(kept, n, k, a, m, c)
        else:
            ctx.gemm_q(qtype, w, n, k, a, m, c)

    for _ in range(3):
        call()
    ctx.sync()
    ctx.prof_start(8 * reps)
    for _ in range(reps):
        call()
    ms, launches = ctx.prof_stop()
    for buf in (w, a, c) + ((kept,) if expanded else ()):
        buf.free()
    us = ms / reps * 1e3
    tflops = 2.0 * m * n * k / us / 1e6
    return {"us_per_gemm": round(us, 1), "launches_per_gemm": launches // reps, "tflops": round(tflops, 1),
            "frac_mfma_f16_peak": round(tflops / MFMA_F16_PEAK_TFLOPS, 4)}


def matvec_timeline(ctx, n, k, reps=20, queued=12):
    """In-kernel timeline of the headline kernel (its measuring build, skn_test_matvec_q4k_stamps): `queued` launches back
    to back over rotating weight copies, the stamps of the last one; percentiles over its wavefronts, averaged over
    `reps` such launches.  Times in microseconds after the first wavefront of the launch started (100 MHz clock)."""
    ws = [ctx.to_device(synth.weight(Q4_K, n, k, seed=1234 + c)) for c in range(N_COPIES)]
    x = ctx.to_device(synth.activation_f32(k, seed=5))
    y = ctx.alloc(4 * n)
    stamps = ctx.alloc(8 * 8 * n)
    names = ["wavefront starts", "x and step-0 weights requested", "x stored to LDS", "barrier passed", "step 0 done",
             "step 1 done", "step 2 done"]
    acc = np.zeros((7, 5))
    end_by_block = np.zeros(n // 8)
    end_by_xcc = {}
    for r in range(reps):
        for j in range(queued):
            ctx.test_matvec_q4k_stamps(ws[(r * queued + j) % N_COPIES], n, k, x, y, stamps)
        ctx.sync()
        t = stamps.download(np.uint64, 8 * n).reshape(n, 8)
        rel = (t[:, :7] - t[:, 0].min()).astype(np.float64) * 0.01
        for e in range(7):
            v = np.sort(rel[:, e])
            acc[e] += [v[0], v[n // 10], v[n // 2], v[n * 9 // 10], v[-1]]
        end_by_block += rel[:, 6].reshape(n // 8, 8).mean(axis=1)
        xcc = (t[:, 7] >> np.uint64(32)).astype(np.int64) & 7
        for q in range(8):
            if np.any(xcc == q):
                end_by_xcc.setdefault(q, []).append(float(rel[xcc == q, 6].mean()))
    acc /= reps
    end_by_block /= reps
    half = (n // 8) // 2
    out = {"mode": "timeline", "workload": f"Q4_K matvec N={n} K={k}", "wavefronts": n, "launches_averaged": reps,
           "queued_back_to_back": queued, "columns": ["min", "p10", "median", "p90", "max"],
           "events_us": {names[e]: [round(float(a), 2) for a in acc[e]] for e in range(7)},
           "mean_end_us_first_half_of_workgroups": round(float(end_by_block[:half].mean()), 2),
           "mean_end_us_second_half_of_workgroups": round(float(end_by_block[half:].mean()), 2),
           "mean_end_us_by_xcd": {str(q): round(float(np.mean(v)), 2) for q, v in sorted(end_by_xcc.items())}}
    for b in ws + [x, y, stamps]:
        b.free()
    return out


def matvec_split_figures(ctx, n, k, steps=600, warmup=50):
    """The headline matvec with k split across workgroups (option q4k.split) beside the default kernel, and beside the
    dense F16 matvec over the same weight bytes: kernel durations from per-launch events, cold weights."""
    out = {"mode": "ksplit", "workload": f"Q4_K matvec N={n} K={k}"}
    r = bench_matvec(ctx, Q4_K, n, k, steps, warmup)
    out["default_whole_rows_per_wavefront"] = {"kernel_us": round(r["kernel_us"], 3), "wall_us": round(r["ms_per_step"] * 1e3, 3)}
    for split, rows, name in ((1, 1, "ticket_merge_1_row"), (1, 2, "ticket_merge_2_rows"), (2, 1, "atomic_add_1_row"), (2, 2, "atomic_add_2_rows")):
        ctx.set_option("q4k.split", split)
        ctx.set_option("q4k.rows", rows)
        try:
            r = bench_matvec(ctx, Q4_K, n, k, steps, warmup)
        finally:
            ctx.set_option("q4k.split", 0)
            ctx.set_option("q4k.rows", 0)
        # (with atomic adds every step is a fill of y and the kernel: the per-launch figure averages both)
        out[name] = {"mean_us_per_launch": round(r["kernel_us"], 3), "wall_us_per_step": round(r["ms_per_step"] * 1e3, 3)}
    rd = bench_matvec(ctx, 1, n, (n * (k // 256) * 144) // (2 * n), steps, warmup, seed=8100)
    out["f16_matvec_same_weight_bytes"] = {"kernel_us": round(rd["kernel_us"], 3)}
    return out


def gemm_expanded_rows(ctx):
    """The Q6_K shapes of the GEMM leg with their expanded weights kept between calls."""
    return {f"q6_k_expanded_{mm}x{nn}x{kk}": bench_gemm(ctx, Q6_K, mm, nn, kk, expanded=True)
            for mm, nn, kk in ((512, 4096, 4096), (512, 14336, 4096))}


def bench_dequant(ctx, qtype, n, k, reps=20):
    """Block dequantization to fp32: bytes read + bytes written per launch against the HBM peak."""
    w = ctx.to_device(synth.weight(qtype, n, k, seed=17))
    out = ctx.alloc(4 * n * k)
    for _ in range(3):
        ctx.dequant(qtype, w, n * k, out)
    ctx.prof_start(reps)
    for _ in range(reps):
        ctx.dequant(qtype, w, n * k, out)
    ms, launches = ctx.prof_stop()
    be, bb = synth.BLOCK[qtype]
    nbytes = n * (k // be) * bb + 4 * n * k
    w.free()
    out.free()
    us = ms / launches * 1e3
    return {"kernel_us": round(us, 1), "gbs": round(nbytes / us / 1e3, 1), "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}


def bench_kv(ctx, steps=200):
    """Paged KV cache, 8 sequences x 32 heads x 128: appending one token per sequence (131 072 bytes written per
    step) and gathering 4096 tokens of one sequence back (64 MiB moved)."""
    n_seq, n_head, dim, n_ctx = 8, 32, 128, 4096
    kv = ctx.kv_cache(n_seq, n_head, dim, 256, 8192)
    k1 = ctx.to_device(synth.kv_f16((n_seq, n_head, dim), seed=90))
    v1 = ctx.to_device(synth.kv_f16((n_seq, n_head, dim), seed=91))
    seqs = list(range(n_seq))
    for _ in range(20):
        kv.append(k1, v1, seqs)
    ctx.prof_start(4 * steps)
    for _ in range(steps):
        kv.append(k1, v1, seqs)
    ms, launches = ctx.prof_stop()
    append_us = ms / steps * 1e3
    run_k = ctx.to_device(synth.kv_f16((n_ctx, n_head, dim), seed=92))
    run_v = ctx.to_device(synth.kv_f16((n_ctx, n_head, dim), seed=93))
    kv.reset(0)
    kv.append_run(0, run_k, run_v, n_ctx)
    gk, gv = ctx.alloc(n_ctx * n_head * dim * 2), ctx.alloc(n_ctx * n_head * dim * 2)
    kv.gather(0, 0, n_ctx, gk, gv)
    ctx.prof_start(40)
    for _ in range(10):
        kv.gather(0, 0, n_ctx, gk, gv)
    gms, gl = ctx.prof_stop()
    gather_us = gms / 10 * 1e3
    moved = 2 * 2 * n_ctx * n_head * dim * 2  # K and V, read and written
    kv.free()
    return {"append_us_per_step": round(append_us, 2), "append_launches_per_step": launches / steps,
            "append_bytes_per_step": 2 * n_seq * n_head * dim * 2, "gather_4096_tokens_us": round(gather_us, 1),
            "gather_gbs": round(moved / gather_us / 1e3, 1)}


def cpu_baseline(qtype, n, k, budget_s=10.0):
    """The CPU oracle (C, OpenMP over rows) on the headline workload; a bounded number of repetitions."""
    from oracle import oracle_c  # the checker, timed as the "port" CPU baseline -- never the product path

    raw = synth.weight(qtype, n, k, seed=1234)
    x = synth.activation_f32(k, seed=2233)
    cores = oracle_c.num_threads()
    oracle_c.matvec_q(qtype, raw, n, k, x)  # warm
    reps, t0 = 0, time.perf_counter()
    while True:
        oracle_c.matvec_q(qtype, raw, n, k, x)
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s or reps >= 20000:
            break
    per = dt / reps
    # the reference's own algorithm for such a weight (dequantize to fp64, transpose, i-outer loop), one thread
    t1 = time.perf_counter()
    oracle_c.matvec_q(qtype, raw, n, k, x, reference_algorithm=True)
    ref_alg = time.perf_counter() - t1
    # the same oracle on one thread
    oracle_c.set_num_threads(1)
    try:
        t2 = time.perf_counter()
        for _ in range(3):
            oracle_c.matvec_q(qtype, raw, n, k, x)
        single = (time.perf_counter() - t2) / 3
    finally:
        oracle_c.set_num_threads(cores)
    nbytes = matvec_bytes(qtype, n, k)
    # The reference is Kotlin: were a JVM and a Kotlin compiler on this box, its CPU restatement
    # (bindings/kotlin/common/CpuQuantReference.kt) could be timed beside the oracle.  Probed, never required.
    import shutil

    jvm = {tool: shutil.which(tool) for tool in ("java", "kotlinc")}
    kotlin = ("absent (no " + " / ".join(t for t, path in jvm.items() if not path) + " on this box)" if not all(jvm.values())
              else "java and kotlinc present; the Kotlin restatement is not compiled or run by this script")
    return {
        "value": nbytes / per / 1e9,
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{reps} repetitions of the full Q4_K {n}x{k} matvec ({dt:.1f} s), fp64 accumulation, OpenMP over rows",
        "ms_per_matvec": per * 1e3,
        "single_thread_ms": single * 1e3,
        "single_thread_gbs": nbytes / single / 1e9,
        "reference_algorithm_1thread_ms": ref_alg * 1e3,
        "kotlin_cpu_reference": kotlin,
    }


def bench_other_formats(ctx):
    """The further formats: matvec at 4096 x 4096 and 4096 x 11008, kernel time and GB/s of block bytes."""
    out = {}
    for nn, kk in ((4096, 4096), (4096, 11008)):
        res = {}
        for name, qt in (("q4_0", 2), ("q4_1", 3), ("q5_0", 6), ("q5_1", 7), ("q2_k", 10), ("q3_k", 11), ("q5_k", 13),
                         ("q8_k", 15), ("iq4_nl", 20), ("iq4_xs", 23), ("tq1_0", 34), ("tq2_0", 35), ("f16", 1)):
            r = bench_matvec(ctx, qt, nn, kk, 200, 20, copies=24, seed=7000 + qt)
            res[name] = {"kernel_us": round(r["kernel_us"], 2), "kernel_gbs": round(r["kernel_gbs"], 1)}
        out[f"{nn}x{kk}"] = res
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary shapes")
    ap.add_argument("--mode", choices=["bench", "copy", "decode", "attention", "gemm", "formats", "timeline", "ksplit"], default="bench",
                    help="decode / attention / gemm: only that leg (for kernel traces).  timeline: the headline kernel's in-kernel time stamps.  ksplit: the headline matvec with k split across workgroups beside the default.  copy: run --steps plain device copies of the headline weight size instead (the known-size "
                         "workload that hardware traffic counters are calibrated against)")
    ap.add_argument("--set", action="append", default=[], metavar="KEY=VALUE",
                    help="a tuning option of the library (skn_set_option) for this run, e.g. --set attn.splits=2 or --set llama.attn_wide=0; repeatable")
    ap.add_argument("--no-graph", action="store_true",
                    help="decode without the captured step graph (kernel tracers that cannot follow graph launches)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    ctx = runtime.Context(0)
    info = ctx.device_info()
    if args.no_graph:
        ctx.set_option("llama.graph", 0)
    for kv in args.set:
        key, _, val = kv.partition("=")
        ctx.set_option(key, int(val))
    n, k = 4096, 11008
    if args.mode == "timeline":
        print(json.dumps(matvec_timeline(ctx, n, k)))
        ctx.close()
        return
    if args.mode == "ksplit":
        print(json.dumps(matvec_split_figures(ctx, n, k, min(args.steps, 600), min(args.warmup, 50))))
        ctx.close()
        return
    if args.mode == "copy":
        nbytes = n * (k // 256) * 144
        srcs = [ctx.to_device(synth.weight(Q4_K, n, k, seed=1234 + c)) for c in range(N_COPIES)]
        dst = ctx.alloc(nbytes)
        ctx.prof_start(args.steps)
        for i in range(args.steps):
            ctx.copy(dst, srcs[i % N_COPIES], nbytes)
        ms, launches = ctx.prof_stop()
        print(json.dumps({"mode": "copy", "bytes_read": nbytes, "bytes_written": nbytes, "launches": launches,
                          "kernel": "copy16_kernel", "kernel_us": round(ms / launches * 1e3, 3),
                          "read_plus_write_gbs": round(2 * nbytes / (ms / launches * 1e-3) / 1e9, 1)}))
        ctx.close()
        return
    if args.mode == "decode":
        from skainet_amd import llama_bench
        print(json.dumps({"mode": "decode", **llama_bench.run(ctx, steps=min(args.steps, 128))}))
        ctx.close()
        return
    gemm_shapes = [("q4_k", Q4_K, 512, 4096, 4096), ("q4_k", Q4_K, 512, 14336, 4096), ("q4_k", Q4_K, 512, 4096, 11008),
                   ("q6_k", Q6_K, 512, 4096, 4096), ("q6_k", Q6_K, 512, 14336, 4096)]
    if args.mode == "attention":
        print(json.dumps({"mode": "attention", **bench_attention(ctx, min(args.steps, 200), 10)}))
        ctx.close()
        return
    if args.mode == "formats":
        print(json.dumps({"mode": "formats", **bench_other_formats(ctx)}))
        ctx.close()
        return
    if args.mode == "gemm":
        print(json.dumps({"mode": "gemm", **gemm_expanded_rows(ctx), **{f"{nm}_{mm}x{nn}x{kk}": bench_gemm(ctx, qt, mm, nn, kk)
                                             for nm, qt, mm, nn, kk in gemm_shapes}}))
        ctx.close()
        return
    head = bench_matvec(ctx, Q4_K, n, k, args.steps, args.warmup)
    # What this machine streams at the headline's byte count with next to no arithmetic: the dense F16 matvec of the
    # library over a weight of the same bytes (4096 x 3096 x 2 = the 25 362 432 bytes of the Q4_K blocks), cold like the
    # headline (24 rotating copies).  The headline's fraction of the published peak stands beside its fraction of this.
    rd = bench_matvec(ctx, 1, 4096, 3096, min(args.steps, 600), min(args.warmup, 50), copies=N_COPIES, seed=8100)

    extra = {"device": info["name"], "compute_units": info["compute_units"]}
    if not args.no_extra:
        es, ew = min(args.steps, 600), min(args.warmup, 50)
        shapes = [("q4_k_4096x4096", Q4_K, 4096, 4096, 64), ("q4_k_11008x4096", Q4_K, 11008, 4096, 24),
                  ("q8_0_4096x4096", Q8_0, 4096, 4096, 32), ("q6_k_4096x4096", Q6_K, 4096, 4096, 40)]
        for name, qt, nn, kk, copies in shapes:
            r = bench_matvec(ctx, qt, nn, kk, es, ew, copies=copies, seed=4000 + nn + kk + qt)
            extra[name] = {key: (round(r[key], 3) if isinstance(r[key], float) else r[key])
                           for key in ("kernel_us", "kernel_gbs", "hot_kernel_us", "hot_kernel_gbs", "wall_gbs")}
            extra[name]["frac_hbm_peak"] = round(r["kernel_gbs"] / HBM_PEAK_GBS, 4)
        # the smallest shape beside the dense F16 matvec over its weight bytes (4096 x 1152 x 2 = 9 437 184), as the
        # headline stands beside its own: at 9.4 MB a launch is mostly its fixed cost, for any kernel
        rs = bench_matvec(ctx, 1, 4096, 1152, es, ew, copies=64, seed=8200)
        extra["q4_k_4096x4096"]["read_rate_same_bytes"] = {"kernel": "dense F16 matvec 4096 x 1152", "kernel_us": round(rs["kernel_us"], 3),
                                                          "frac": round(rs["kernel_gbs"] / HBM_PEAK_GBS, 4)}
        extra["q4_k_4096x4096"]["frac_of_read_rate"] = round(extra["q4_k_4096x4096"]["kernel_gbs"] / rs["kernel_gbs"], 4)
        other = bench_other_formats(ctx)["4096x4096"]
        extra["other_formats_4096x4096"] = other
        extra["dequant_4096x4096"] = {name: bench_dequant(ctx, qt, 4096, 4096)
                                      for name, qt in (("q8_0", Q8_0), ("q4_k", Q4_K), ("q6_k", Q6_K))}
        extra["kv_cache_8x32x128"] = bench_kv(ctx)
        att = bench_attention(ctx, min(args.steps, 200), 10)
        extra["attention_8x32x128_ctx4096"] = {key: round(val, 4) for key, val in att.items()}
        extra["prompt_attention_512x32x128"] = bench_attention_prefill(ctx)
        extra["prefill_gemm"] = {f"{nm}_{mm}x{nn}x{kk}": bench_gemm(ctx, qt, mm, nn, kk)
                                 for nm, qt, mm, nn, kk in gemm_shapes}
        extra["prefill_gemm"].update(gemm_expanded_rows(ctx))
        try:
            from skainet_amd import llama_bench
            extra["decode_7b_q4_k"] = llama_bench.run(ctx)
            # the same shape as mixed quantizations have it: Q6_K value and down projections in every second layer
            mix = {f"l{i}.{m}": Q6_K for i in range(0, 32, 2) for m in ("wv", "w_down")}
            r = llama_bench.run(ctx, steps=64, matrix_types=mix)
            extra["decode_7b_q4_k_q6_k_mix"] = {key: r[key] for key in ("decode_tok_s", "ms_per_token", "prefill_ms", "weight_bytes_per_token")}
            ctx.set_option("llama.expand_weights", 1)  # the Q6_K matrices keep their expanded copies: 4 GB more
            try:
                r = llama_bench.run(ctx, steps=8, matrix_types=mix)
                extra["decode_7b_q4_k_q6_k_mix"]["prefill_ms_expanded_weights"] = r["prefill_ms"]
            finally:
                ctx.set_option("llama.expand_weights", 0)
        except Exception as e:  # the decoder leg reports its own absence instead of failing the headline
            extra["decode_7b_q4_k"] = {"error": f"{type(e).__name__}: {e}"}

    traffic_rec = traffic.load_current(os.path.join(ROOT, "profiles", "matvec_q4k_4096x11008_traffic.json"))
    out = {
        "metric": "Q4_K matvec effective HBM GB/s (% peak); decode tok/s, 7B-shape Q4_K",
        "value": round(head["wall_gbs"], 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(head["ms_per_step"], 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "q4_k x f32 -> f32",
        "data": "synthetic",
        "config": {
            "workload": "Q4_K matvec batch 1, N=4096 K=11008 (BASELINE configs[1])",
            "weight_copies_rotated": head["copies"],
            "weight_bytes": head["weight_bytes"],
            "algorithmic_bytes_per_step": head["bytes_per_launch"],
            "weight_checksum_copy0": head["checksum_copy0"],
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(head["kernel_gbs"], 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(head["kernel_gbs"] / HBM_PEAK_GBS, 4),
            # HBM bytes of one launch from hardware counters (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE, one run
            # each, scaled by what the same counters read for a copy kernel of this size), as recorded in
            # profiles/ by skainet_amd/traffic.py -- null when that record was taken on other kernel sources
            "traffic": traffic_rec["traffic_bytes"] if traffic_rec else None,
            "traffic_record": "profiles/matvec_q4k_4096x11008_traffic.json" if traffic_rec else "none for these kernel sources",
            "kernel": "matvec_q4k_kernel",
            "kernel_us": round(head["kernel_us"], 3),
            "cache_hot_gbs": round(head["hot_kernel_gbs"], 2),
            "read_rate_same_bytes": {
                "kernel": "dense F16 matvec 4096 x 3096 (skn_matvec_q), the same weight bytes, cold",
                "bytes_per_launch": rd["bytes_per_launch"],
                "kernel_us": round(rd["kernel_us"], 3),
                "gbs": round(rd["kernel_gbs"], 2),
                "frac": round(rd["kernel_gbs"] / HBM_PEAK_GBS, 4),
            },
            "frac_of_read_rate": round(head["kernel_gbs"] / rd["kernel_gbs"], 4),
        },
        "extra": extra,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(Q4_K, n, k)
    ctx.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
