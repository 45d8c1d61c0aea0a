#!/usr/bin/env python3
"""Benchmark of the fused-block path on one MI355X.

A "step" is one call of the Llama-3-8B-shaped fused SwiGLU FFN
(X [2048, 4096], W_gate/W_up [4096, 14336], W_down [14336, 4096], fp16 in HBM,
fp32 accumulation): the gate/up GEMM with the SwiGLU epilogue followed by the
down projection, both launched through the C ABI of libtrinity_amd.so.  Inputs
are synthetic, seeded and resident in HBM before the timed region.

One JSON line is printed: the headline value (TFLOP/s of the whole FFN step),
`roofline` for the dominant kernel (the gate/up GEMM, timed per launch with
events on the launch stream inside the timed region), `cpu_baseline` (the CPU
oracle on a bounded row sample, on this box's host cores) and `blocks`: µs per
call and fraction of roofline for every other benchmark configuration
(RMSNorm, Falcon GELU FFN, the five attention variants), each timed as 100
replays of a captured HIP graph after 10 warm-up calls.
"""
import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0  # MI355X dense fp16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E


def _gen(seed=42):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def _randn(g, *shape, std=1.0, mean=0.0, dev="cuda:0"):
    return (torch.randn(*shape, generator=g) * std + mean).to(torch.float16).to(dev)


def progress(msg):
    """One line on stderr per stage, flushed: a long run shows where it is."""
    sys.stderr.write("[bench] %s\n" % msg)
    sys.stderr.flush()


REPLAYS = 100  # graph replays per block (lowered with --replays for counter-collection runs)


def graph_time_us(fn, warmup=10, replays=None, inner=1):
    """10 warm-up calls, capture `inner` back-to-back calls in a HIP graph, mean
    over 100 replays.  `inner` > 1 is used for kernels of a few microseconds,
    where the gap between two graph launches would otherwise be what is timed."""
    replays = REPLAYS if replays is None else replays
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(warmup):
            fn()
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(inner):
                fn()
    stream.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with torch.cuda.stream(stream):
        graph.replay()
        start.record()
        for _ in range(replays):
            graph.replay()
        end.record()
    stream.synchronize()
    return start.elapsed_time(end) / (replays * inner) * 1e3


def attn_flops(S, N, Hq, Hkv, D, causal=True):
    proj = 2.0 * S * N * (Hq + 2 * Hkv) * D
    attn = 4.0 * D * Hq * (S * (S + 1) / 2.0 if causal else float(S) * S)
    return proj, attn


def bench_blocks(ext, dev, quick=False, only=None):
    """µs/call of every other benchmark configuration (`only`: just the attention blocks whose name contains it)."""
    out = []
    g = _gen(42)
    want = lambda name: not only or only in name
    if want("rmsnorm_4096x4096"):
        _rmsnorm_block(ext, dev, g, out)
    if want("ffn_gelu_falcon7b_T2048"):
        _gelu_block(ext, dev, g, out)
    if not quick and want("ffn_swiglu_llama3_8b_T2048_bf16"):
        _bf16_block(ext, dev, g, out)
    return _attention_blocks(ext, dev, g, out, quick, only)


def _rmsnorm_block(ext, dev, g, out):
    # ---- standalone RMSNorm, X [4096, 4096]
    progress("rmsnorm")
    x = _randn(g, 4096, 4096)
    w = _randn(g, 4096, std=0.1, mean=1.0)
    y = torch.empty_like(x)
    nbytes = 2 * 4096 * 4096 * 2 + 4096 * 2
    # HBM figure: the 50 calls of a replay walk a ring of 20 x / y pairs (1.34 GB), so that no call finds its rows
    # in the 256 MB Infinity Cache; every x holds its own random data
    ring = 20
    xs = [x] + [_randn(g, 4096, 4096) for _ in range(ring - 1)]
    ys = [torch.empty_like(x) for _ in range(ring)]
    turn = [0]

    def ring_call():
        i = turn[0] % ring
        turn[0] += 1
        ext.rmsnorm(xs[i], w, ys[i], 1e-5)

    us = graph_time_us(ring_call, warmup=ring, inner=2 * ring + 10)
    # the same kernel on one x / y pair replayed back to back: its 64 MB then stay in the Infinity Cache
    us_cached = graph_time_us(lambda: ext.rmsnorm(x, w, y, 1e-5), inner=50)
    out.append({"block": "rmsnorm_4096x4096", "us": us, "GBps": nbytes / us * 1e-3, "frac_hbm": nbytes / us * 1e-3 / PEAK_HBM_GBS,
                "buffers": "ring of %d x/y pairs, %.2f GB (no reuse out of the Infinity Cache)" % (ring, ring * 2 * 4096 * 4096 * 2 / 1e9),
                "us_cache_resident": us_cached, "GBps_cache_resident": nbytes / us_cached * 1e-3})
    del x, y, xs, ys


def _gelu_block(ext, dev, g, out):
    # ---- Falcon-7B GELU FFN
    progress("falcon gelu ffn")
    T, N, F = 2048, 4544, 18176
    x = _randn(g, T, N)
    w1, w2 = _randn(g, N, F, std=0.02), _randn(g, F, N, std=0.02)
    hid = torch.empty(T, F, dtype=torch.float16, device=dev)
    o = torch.empty(T, N, dtype=torch.float16, device=dev)
    ws_bytes = ext.ffn_workspace_bytes(T, N, F)   # the second product runs split over K when given room
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    us = graph_time_us(lambda: ext.ffn_gelu(x, w1, w2, hid, o, workspace=ws))
    fl = 2.0 * 2 * T * N * F
    out.append({"block": "ffn_gelu_falcon7b_T2048", "us": us, "TFLOPs": fl / us * 1e-6, "frac_mfma": fl / us * 1e-6 / PEAK_FP16_TFLOPS})
    del x, w1, w2, hid, o, ws


def _bf16_block(ext, dev, g, out):
    # ---- bf16 copy of the step (outside the benchmark configuration; same kernels compiled for bf16)
    progress("llama swiglu ffn, bf16")
    T, N, F = 2048, 4096, 14336
    bf = torch.bfloat16
    xb = _randn(g, T, N).to(bf)
    wgb, wub, wdb = _randn(g, N, F, std=0.02).to(bf), _randn(g, N, F, std=0.02).to(bf), _randn(g, F, N, std=0.02).to(bf)
    hb = torch.empty(T, F, dtype=bf, device=dev)
    ob = torch.empty(T, N, dtype=bf, device=dev)
    us = graph_time_us(lambda: ext.ffn_swiglu(xb, wgb, wub, wdb, hb, ob))
    fl = 3.0 * 2 * T * N * F
    out.append({"block": "ffn_swiglu_llama3_8b_T2048_bf16", "us": us, "TFLOPs": fl / us * 1e-6, "frac_mfma": fl / us * 1e-6 / PEAK_FP16_TFLOPS})
    del xb, wgb, wub, wdb, hb, ob


def _attention_blocks(ext, dev, g, out, quick, only):
    def attn_case(name, S, N, Hq, Hkv, D, variant, prenorm=False, qknorm=False, kcontig=False, zero_x=False):
        if only and only not in name:
            return
        x = _randn(g, S, N)
        if zero_x:  # Q = K = V = 0: the same instruction streams without switching activity in the data paths
            x.zero_()
        wq, wk, wv = _randn(g, N, Hq * D, std=0.02), _randn(g, N, Hkv * D, std=0.02), _randn(g, N, Hkv * D, std=0.02)
        if kcontig:  # the same matrices stored K-contiguous (stride[0] == 1), the layout of torch.nn.Linear.weight
            wq, wk, wv = (w.t().contiguous().t() for w in (wq, wk, wv))
        nw = _randn(g, N, std=0.1, mean=1.0) if prenorm else None
        p = ext.attn_params(Hq, Hkv, D, S, scale=1.0 / math.sqrt(D), causal=True, rms_eps=1e-5, prenorm=prenorm,
                            qknorm=qknorm, tau=1.0, noise_seed=42)
        scratch = torch.empty(ext.qkv_scratch_bytes(p, N), dtype=torch.uint8, device=dev)
        o = torch.empty(S, Hq * D, dtype=torch.float16, device=dev)
        if variant == "vanilla":
            fn = lambda: ext.qkv_attention(x, nw, wq, wk, wv, None, None, scratch, None, o, p)
        elif variant == "keyformer":
            sc = torch.empty(Hq, S, dtype=torch.float32, device=dev)
            fn = lambda: ext.keyformer(x, nw, wq, wk, wv, None, None, scratch, None, o, sc, p)
        else:
            s1 = torch.empty(Hq, S, dtype=torch.float32, device=dev)
            s2 = torch.empty(Hq, S, dtype=torch.float32, device=dev)
            fn = lambda: ext.roco(x, nw, wq, wk, wv, None, None, scratch, o, s1, s2, p, as_mean_var=True)
        progress(name)
        us = graph_time_us(fn)
        proj, attn = attn_flops(S, N, Hq, Hkv, D)
        fl = proj + attn  # algorithmic minimum: the score path's recomputed QK^T is not counted
        rec = {"block": name, "us": us, "TFLOPs": fl / us * 1e-6, "frac_mfma": fl / us * 1e-6 / PEAK_FP16_TFLOPS}
        if not quick:
            # `us` follows the reference's protocol (one call per graph), so it holds the gap between two graph
            # launches; ten calls per graph show the call without it
            rec["us_ten_calls_per_graph"] = graph_time_us(fn, replays=max(1, REPLAYS // 10), inner=10)
        out.append(rec)

    seqs = [1024] if quick else [1024, 4096]
    for S in seqs:
        attn_case("vanilla_llama3_8b_S%d" % S, S, 4096, 32, 8, 128, "vanilla")
    if not quick:  # (outside the benchmark configuration: its weights are row-major, as the reference's X.W)
        attn_case("vanilla_llama3_8b_S4096_wT", 4096, 4096, 32, 8, 128, "vanilla", kcontig=True)
        # (not a benchmark configuration either: what the block takes when the board's power limit does not bind)
        attn_case("vanilla_llama3_8b_zero_inputs_S4096", 4096, 4096, 32, 8, 128, "vanilla", zero_x=True)
    for S in seqs:
        attn_case("prenorm_falcon7b_S%d" % S, S, 4544, 71, 1, 64, "vanilla", prenorm=True)
        attn_case("qknorm_falcon7b_S%d" % S, S, 4544, 71, 1, 64, "vanilla", qknorm=True)
    for S in ([2048] if quick else [2048, 4096]):
        attn_case("keyformer_llama3_8b_S%d" % S, S, 4096, 32, 8, 128, "keyformer")
        attn_case("roco_llama3_8b_S%d" % S, S, 4096, 32, 8, 128, "roco")
    return out


def bench_reference_shapes(ext, dev):
    """The reference's own evaluation shapes (M = 16 new tokens, P = 1024 cached keys, as many KV heads as
    query heads, no mask, no softmax scale, KeyFormer noise as a tensor with tau = 1.5;
    evaluation/llama_configs.json, falcon_configs.json, ffn/*/tensor_configs.json).  These calls are bound by
    streaming the weights once: bytes = weights + the cache rows read + inputs and outputs."""
    out = []
    g = _gen(42)
    for model, (M, D, N, P, H) in (("llama", (16, 128, 4096, 1024, 32)), ("falcon", (16, 64, 4544, 1024, 71))):
        progress("reference shapes: " + model)
        L = P + M
        x = _randn(g, M, N, std=0.01)
        wq, wk, wv = (_randn(g, N, H * D, std=0.01) for _ in range(3))
        kc, vc = _randn(g, H, L, D, std=0.01), _randn(g, H, L, D, std=0.01)
        noise = _randn(g, H, M, L)
        o = torch.empty(M, H * D, dtype=torch.float16, device=dev)
        sc1 = torch.empty(H, L, dtype=torch.float32, device=dev)
        sc2 = torch.empty(H, L, dtype=torch.float32, device=dev)
        base_bytes = 3 * N * H * D * 2 + 2 * H * L * D * 2 + 2 * M * N * 2 + 2 * H * M * D * 2
        for variant, kw in (("vanilla", {}), ("prenorm", {"prenorm": True}), ("qknorm", {"qknorm": True}),
                            ("keyformer", {}), ("roco", {})):
            p = ext.attn_params(H, H, D, M, kv_prefix=P, scale=1.0, causal=False, rms_eps=0.0, tau=1.5, **kw)
            scratch = torch.empty(ext.qkv_scratch_bytes(p, N), dtype=torch.uint8, device=dev)
            nbytes = base_bytes
            if variant == "keyformer":
                fn = lambda: ext.keyformer(x, None, wq, wk, wv, kc, vc, scratch, noise, o, sc1, p)
                nbytes += H * M * L * 2 + H * L * 4
            elif variant == "roco":
                fn = lambda: ext.roco(x, None, wq, wk, wv, kc, vc, scratch, o, sc1, sc2, p)
                nbytes += 2 * H * L * 4
            else:
                fn = lambda: ext.qkv_attention(x, None, wq, wk, wv, kc, vc, scratch, None, o, p)
            us = graph_time_us(fn)
            out.append({"block": "%s_%s_M16_P1024" % (variant, model), "us": us, "GBps": nbytes / us * 1e-3,
                        "frac_hbm": nbytes / us * 1e-3 / PEAK_HBM_GBS})
        if model == "llama":
            # the same call with the caches held as fp8 (e4m3): append quantises, the attention kernel reads fp8 rows
            kc8 = (kc.float() / 0.001).clamp(-448, 448).to(torch.float8_e4m3fn)
            vc8 = (vc.float() / 0.001).clamp(-448, 448).to(torch.float8_e4m3fn)
            p = ext.attn_params(H, H, D, M, kv_prefix=P, scale=1.0, causal=False, kv_fp8=True, k_scale=0.001, v_scale=0.001)
            scratch = torch.empty(ext.qkv_scratch_bytes(p, N), dtype=torch.uint8, device=dev)
            us = graph_time_us(lambda: ext.qkv_attention(x, None, wq, wk, wv, kc8, vc8, scratch, None, o, p))
            nbytes = base_bytes - 2 * H * L * D
            out.append({"block": "vanilla_llama_M16_P1024_fp8kv", "us": us, "GBps": nbytes / us * 1e-3,
                        "frac_hbm": nbytes / us * 1e-3 / PEAK_HBM_GBS})
            del kc8, vc8, scratch
        del x, wq, wk, wv, kc, vc, noise
    # the same 16 new tokens against a long cache with the benchmark configuration's heads (Llama-3-8B: 32 query heads
    # over 8 KV heads, causal, 1/sqrt(D)): the looping key-split kernel; fp16 and fp8 (e4m3) caches
    M, D, N, P, Hq, Hkv = 16, 128, 4096, 32768, 32, 8
    L = P + M
    x = _randn(g, M, N, std=0.01)
    wq, wk, wv = _randn(g, N, Hq * D, std=0.01), _randn(g, N, Hkv * D, std=0.01), _randn(g, N, Hkv * D, std=0.01)
    o = torch.empty(M, Hq * D, dtype=torch.float16, device=dev)
    for fp8 in (False, True):
        kc, vc = _randn(g, Hkv, L, D, std=0.5), _randn(g, Hkv, L, D, std=0.5)
        if fp8:
            kc, vc = kc.to(torch.float8_e4m3fn), vc.to(torch.float8_e4m3fn)
        p = ext.attn_params(Hq, Hkv, D, M, kv_prefix=P, scale=1.0 / math.sqrt(D), causal=True, kv_fp8=fp8, k_scale=1.0, v_scale=1.0)
        scratch = torch.empty(ext.qkv_scratch_bytes(p, N), dtype=torch.uint8, device=dev)
        us = graph_time_us(lambda: ext.qkv_attention(x, None, wq, wk, wv, kc, vc, scratch, None, o, p))
        nbytes = N * (Hq + 2 * Hkv) * D * 2 + 2 * Hkv * L * D * (1 if fp8 else 2) + 2 * M * N * 2 + 2 * Hq * M * D * 2
        out.append({"block": "vanilla_llama_gqa_M16_P32768" + ("_fp8kv" if fp8 else ""), "us": us, "GBps": nbytes / us * 1e-3,
                    "frac_hbm": nbytes / us * 1e-3 / PEAK_HBM_GBS})
        del kc, vc, scratch
    del x, wq, wk, wv, o
    for model, (M, N, F, tail) in (("llama", (16, 4096, 14336, False)), ("falcon", (16, 4544, 4544, True))):
        o2, x = _randn(g, M, N, std=0.01), _randn(g, M, N, std=0.01)
        wo, a, b, w2 = _randn(g, N, N, std=0.01), _randn(g, N, F, std=0.01), _randn(g, N, F, std=0.01), _randn(g, F, N, std=0.01)
        attn = torch.empty(M, N, dtype=torch.float16, device=dev)
        rs = torch.empty(M, dtype=torch.float32, device=dev)
        ff1 = torch.empty(M, F, dtype=torch.float16, device=dev)
        ff2 = torch.empty(M, N, dtype=torch.float16, device=dev)
        onorm = torch.empty(M, N, dtype=torch.float16, device=dev) if tail else None
        ws = torch.empty(max(16, ext.ffn_workspace_bytes(M, N, F)), dtype=torch.uint8, device=dev)
        us = graph_time_us(lambda: ext.ffn_block(o2, wo, x, a, b, w2, attn, rs, ff1, ff2, onorm, workspace=ws))
        nbytes = (N * N + 3 * N * F) * 2 + 4 * M * N * 2 + M * F * 2
        out.append({"block": "ffn_block_%s_M16" % model, "us": us, "GBps": nbytes / us * 1e-3,
                    "frac_hbm": nbytes / us * 1e-3 / PEAK_HBM_GBS})
        del o2, x, wo, a, b, w2
    return out


def _median(xs):
    ys = sorted(xs)
    n = len(ys)
    return ys[n // 2] if n % 2 else 0.5 * (ys[n // 2 - 1] + ys[n // 2])


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _best_of(fn, budget_s, max_iters):
    """Best wall time of fn() over at most max_iters runs within about budget_s seconds (at least one run)."""
    best, spent, n = float("inf"), 0.0, 0
    while n < max_iters and (n == 0 or spent + best <= budget_s):
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        best, spent, n = min(best, dt), spent + dt, n + 1
    return best, n


def cpu_baseline(T, N, F, sample_rows):
    """The CPU oracle (a port of the reference's eager math: baseline/ffn_ref.py:37-50 for the FFN,
    baseline/ref_rms.py:101-102 and :44-82 for RMSNorm and Vanilla attention; the eager path
    run_baseline.py:162-311 times) on this box's host cores.  Bounded: about 25 s in all."""
    import oracle

    g = _gen(42)
    x = (torch.randn(sample_rows, N, generator=g)).half()
    wg = (torch.randn(N, F, generator=g) * 0.02).half()
    wu = (torch.randn(N, F, generator=g) * 0.02).half()
    wd = (torch.randn(F, N, generator=g) * 0.02).half()
    threads = torch.get_num_threads()
    progress("cpu baseline: ffn, %d threads" % threads)
    oracle.ffn_swiglu(x[:8], wg, wu, wd)  # warm-up (thread pool, allocator)
    best, n = _best_of(lambda: oracle.ffn_swiglu(x, wg, wu, wd), 10.0, 24)
    flops = 3.0 * 2 * sample_rows * N * F
    res = {
        "value": flops / best * 1e-12,
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "port",
        "sample": "%d of %d token rows of the same FFN (fp16 tensors, fp32 math, torch CPU), best of %d runs, %.2f s each"
        % (sample_rows, T, n, best),
        "cpu_model": _cpu_model(),
        "os_cpu_count": os.cpu_count(),
    }
    # the same math on one thread, on a row sample small enough for a single core
    rows1 = min(64, sample_rows)
    progress("cpu baseline: one thread")
    torch.set_num_threads(1)
    try:
        b1, n1 = _best_of(lambda: oracle.ffn_swiglu(x[:rows1], wg, wu, wd), 4.0, 5)
    finally:
        torch.set_num_threads(threads)
    res["one_thread"] = {"value": 3.0 * 2 * rows1 * N * F / b1 * 1e-12, "unit": "TFLOP/s",
                         "sample": "%d rows, best of %d runs, %.2f s each" % (rows1, n1, b1)}
    # fp16 tensors multiplied as fp16 tensors (what the reference's eager modules do when run on the CPU)
    # (where the CPU has no fp16 matrix units torch falls back to a scalar loop, orders of magnitude slower: probe with
    # two rows, then size the sample for about two seconds)
    progress("cpu baseline: fp16 tensors")
    t0 = time.perf_counter()
    oracle.ffn_swiglu(x[:2], wg, wu, wd, compute=torch.float16)
    probe = time.perf_counter() - t0
    rows16 = int(max(2, min(256, sample_rows, 2.0 / max(probe, 1e-4) * 2)))
    if rows16 > 2:
        b16, n16 = _best_of(lambda: oracle.ffn_swiglu(x[:rows16], wg, wu, wd, compute=torch.float16), 4.0, 5)
    else:
        b16, n16 = probe, 1
    res["fp16_tensors"] = {"value": 3.0 * 2 * rows16 * N * F / b16 * 1e-12, "unit": "TFLOP/s", "cores": threads,
                           "sample": "%d rows, torch CPU half matmul, best of %d runs, %.2f s each" % (rows16, n16, b16)}
    del x, wg, wu, wd
    # RMSNorm 4096 x 4096 and Vanilla attention, Llama-3-8B heads, S = 1024 (oracle, four heads at a time)
    progress("cpu baseline: rmsnorm, attention")
    xr = torch.randn(4096, 4096, generator=g).half()
    wr = (torch.randn(4096, generator=g) * 0.1 + 1.0).half()
    br, nr = _best_of(lambda: oracle.rmsnorm(xr, wr, 1e-5), 2.0, 10)
    res["rmsnorm_4096x4096"] = {"us": br * 1e6, "GBps": (2 * 4096 * 4096 * 2 + 4096 * 2) / br * 1e-9, "cores": threads,
                                "sample": "best of %d runs" % nr}
    del xr
    S, Na, Hq, Hkv, D = 1024, 4096, 32, 8, 128
    xa = torch.randn(S, Na, generator=g).half()
    wq = (torch.randn(Na, Hq * D, generator=g) * 0.02).half()
    wk = (torch.randn(Na, Hkv * D, generator=g) * 0.02).half()
    wv = (torch.randn(Na, Hkv * D, generator=g) * 0.02).half()
    ba, na = _best_of(lambda: oracle.qkv_attention(xa, wq, wk, wv, n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D,
                                                   scale=1.0 / math.sqrt(D), causal=True), 4.0, 10)
    proj, attn = attn_flops(S, Na, Hq, Hkv, D)
    res["vanilla_llama3_8b_S1024"] = {"us": ba * 1e6, "TFLOPs": (proj + attn) / ba * 1e-12, "cores": threads,
                                      "sample": "best of %d runs" % na}
    return res


def _traffic_from_profile():
    """HBM-side bytes per gate/up launch as measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE, scaled by a plain
    copy): read from the committed summary, so that the figure and its provenance travel together."""
    import re

    path = os.path.join(ROOT, "profiles", "gemm_swiglu_gateup_llama_ffn.md")
    try:
        text = open(path).read()
    except OSError:
        return None, None
    m = re.search(r"^traffic_bytes_per_launch:\s*([0-9.]+e?[0-9]*)\s*$", text, re.M)
    tag = re.search(r"^measured_at_commit:\s*(\S+)\s*$", text, re.M)
    if not m:
        return None, None
    return float(m.group(1)), "profiles/gemm_swiglu_gateup_llama_ffn.md" + (" @ " + tag.group(1) if tag else "")


def issue_model(ext):
    """What a SIMD needs for a group of one MFMA and n vector instructions, fitted on the issue probe (two waves
    per SIMD, shader-clock ticks): an MFMA alone takes `mfma` ticks; `free` vector instructions issue under it at no
    cost, every further one adds `valu` ticks, a transcendental one `trans` more."""
    ext.issue_probe(True, 4, 0, 2)  # warm-up
    tick = lambda mf, nv, nt: min(ext.issue_probe(mf, nv, nt, 2)[0] for _ in range(3)) / 2.0   # per group and SIMD
    a, b, c, d = tick(1, 0, 0), tick(1, 8, 0), tick(1, 16, 0), tick(1, 8, 2)
    valu = max((c - b) / 8.0, 1e-3)
    return {"mfma": a, "valu": valu, "free": max(0.0, 8.0 - (b - a) / valu), "trans": max(0.0, (d - b) / 2.0),
            "probe_ticks": {"mfma": a, "mfma_8_fma": b, "mfma_16_fma": c, "mfma_8_fma_2_exp": d},
            "note": "ticks per group and SIMD, two waves per SIMD; bound = (mfma * M + valu * max(0, V - free * M) + "
                    "trans * T) / 1024 SIMDs / clock"}


def power_model(ext):
    """What the instructions of the softmax kernels cost at the board's power limit, fitted on the power probe: long
    loops of one MFMA on random fp16 operands with LDS reads, v_fma_f32 and v_exp_f32 beside it, two waves per SIMD.
    The pure MFMA loop already runs at the limit (the clock it settles at is reported), so the time a group takes -
    ns of one SIMD - is the energy it draws, and what an instruction adds to the group is its cost.  The same
    streams on zero operands run at the full clock: their ticks are the issue limits."""
    # (ds_read_b128 per two groups, global -> LDS loads per eight groups, v_fma_f32, v_exp_f32)
    cfgs = {"mfma": (0, 0, 0, 0), "mfma_1_lds": (2, 0, 0, 0), "mfma_2_lds": (4, 0, 0, 0), "mfma_4_fma": (0, 0, 4, 0),
            "mfma_4_fma_1_exp": (0, 0, 4, 1), "mfma_quarter_dma": (0, 2, 0, 0), "mfma_half_dma": (0, 4, 0, 0),
            # the mix of the attention kernel per MFMA, and of the GEMMs
            "mfma_1_lds_quarter_dma_3_fma_1_exp": (2, 2, 3, 1), "mfma_half_lds_quarter_dma_3_fma_1_exp": (1, 2, 3, 1),
            "mfma_half_lds_quarter_dma": (1, 2, 0, 0)}
    probe = {}
    for rnd in (1, 0):
        for name, (nl, ng, nv, nt) in cfgs.items():
            ticks, ns, ghz = ext.power_probe(nl, ng, nv, nt, rnd)
            probe[name + ("" if rnd else "_zero_operands")] = {"ns": round(ns, 3), "ticks": round(ticks, 2), "clock_ghz": round(ghz, 3)}
    ns = lambda k: probe[k]["ns"]
    mfma = ns("mfma")
    return {"mfma_ns": mfma, "lds_read_ns": max(0.0, (ns("mfma_2_lds") - mfma) / 2.0),
            "valu_ns": max(0.0, (ns("mfma_4_fma") - mfma) / 4.0),
            "trans_ns": max(0.0, ns("mfma_4_fma_1_exp") - ns("mfma_4_fma")),
            # (from the GEMM-like mix, which stays at the power limit; the MFMA with nothing but such loads beside it
            # waits for them instead)
            "dma_load_ns": max(0.0, (ns("mfma_half_lds_quarter_dma") - mfma - (ns("mfma_2_lds") - mfma) / 4.0) * 4.0),
            "gemm_mix_TFLOPs_at_power_limit": 32768.0 * 1024 / ns("mfma_half_lds_quarter_dma") * 1e-3,
            "attention_mix_TFLOPs_at_power_limit": 32768.0 * 1024 / ns("mfma_1_lds_quarter_dma_3_fma_1_exp") * 1e-3,
            # the matrix pipe's rate on random operands at the power limit: 32768 flop per MFMA on each of 1024 SIMDs
            "mfma_TFLOPs_at_power_limit": 32768.0 * 1024 / mfma * 1e-3,
            "probe": probe,
            "note": "ns of one SIMD per wave instruction at the power limit (random operands); bound = (mfma_ns * M + "
                    "lds_read_ns * L + valu_ns * V + trans_ns * T + dma_load_ns * M / 4) / 1024 SIMDs (the kernels "
                    "bring 256 bytes of K / V tiles into LDS per MFMA: a quarter of a wave's load)"}


def _issue_inputs():
    """Per-kernel instruction counts of the softmax blocks (rocprofv3 --pmc, per dispatch), from the committed
    summary: lines `issue_model: block=... kind=proj|attn|score us=... clock_ghz=... insts_mfma=... insts_valu=...
    insts_trans=...`."""
    import re

    path = os.path.join(ROOT, "profiles", "mfma_utilisation_attention_kernels.md")
    out = {}
    try:
        text = open(path).read()
    except OSError:
        return out
    for line in re.findall(r"^issue_model: (.*)$", text, re.M):
        kv = dict(f.split("=", 1) for f in line.split())
        out.setdefault(kv["block"], []).append({k: (v if k in ("block", "kind") else float(v)) for k, v in kv.items()})
    return out


def add_issue_bounds(blocks, model):
    """issue_bound_us per softmax block: what its attention and score kernels would take if they were bound by
    nothing but instruction issue (the fitted probe model on their counted MFMA, vector and transcendental
    instructions, at the clock they ran at, capped at 2.4 GHz), plus the measured time of the block's projection
    (a GEMM, bound by the matrix pipe and the memory system, not by vector issue)."""
    inputs = _issue_inputs()
    for rec in blocks:
        kernels = inputs.get(rec["block"])
        if not kernels:
            continue
        bound, measured, parts = 0.0, 0.0, {}
        for k in kernels:
            measured += k["us"]
            if k["kind"] == "proj":
                us = k["us"]
            else:
                m, v, t = k["insts_mfma"], k["insts_valu"] - k["insts_mfma"], k["insts_trans"]
                ticks = model["mfma"] * m + model["valu"] * max(0.0, v - model["free"] * m) + model["trans"] * t
                us = ticks / 1024.0 / min(k["clock_ghz"], 2.4) * 1e-3
            parts[k["kind"]] = round(us, 1)
            bound += us
        rec["issue_bound_us"] = bound
        rec["issue_bound_parts_us"] = parts
        # against the sum of the kernels' own durations under the counters (the block's `us` also holds launch gaps)
        rec["frac_of_issue_bound"] = bound / measured
        rec["kernels_us_under_counters"] = measured


def add_power_bounds(blocks, model):
    """power_bound_us per softmax block: what its kernels (projection, attention, score pass) would take if their
    counted MFMA, LDS, vector and transcendental instructions cost what the power probe says they cost at the
    board's power limit - every LDS instruction priced as a 16-byte-per-lane read, a quarter of a global -> LDS
    load added per MFMA - and nothing else took time.  The fraction is taken against the block's own time."""
    inputs = _issue_inputs()
    for rec in blocks:
        kernels = inputs.get(rec["block"])
        if not kernels or any("insts_lds" not in k for k in kernels):
            continue
        bound, parts = 0.0, {}
        for k in kernels:
            m, v, t, l = k["insts_mfma"], k["insts_valu"] - k["insts_mfma"] - k["insts_trans"], k["insts_trans"], k["insts_lds"]
            us = (model["mfma_ns"] * m + model["lds_read_ns"] * l + model["valu_ns"] * max(0.0, v) + model["trans_ns"] * t +
                  model["dma_load_ns"] * m / 4.0) / 1024.0 * 1e-3
            parts[k["kind"]] = round(us, 1)
            bound += us
        rec["power_bound_us"] = bound
        rec["power_bound_parts_us"] = parts
        rec["frac_of_power_bound"] = bound / rec["us"]


def power_legs(ext, dev, x, wg, wu, wd, hid, out):
    """Two measurements that say what limits the two products of the step on this box: the same products through the
    vendor library (torch.matmul -> hipBLASLt; plain GEMMs, no SwiGLU), and this library's gate/up launch on all-zero
    operands (same instructions, no switching activity in the multipliers)."""
    T, N = x.shape
    F = wg.shape[1]
    res = {}
    progress("vendor GEMMs")
    w_cat = torch.cat([wg, wu], dim=1)               # [N, 2F]: the vendor's gate/up product in one call
    o_cat = torch.empty(T, 2 * F, dtype=torch.float16, device=dev)
    us_gu = graph_time_us(lambda: torch.matmul(x, w_cat, out=o_cat))
    us_dn = graph_time_us(lambda: torch.matmul(hid, wd, out=out))
    res["vendor_gemm_us"] = {"gateup_plain": us_gu, "down_proj": us_dn,
                             "gateup_TFLOPs": 2.0 * 2 * T * N * F / us_gu * 1e-6, "down_TFLOPs": 2.0 * T * F * N / us_dn * 1e-6,
                             "note": "torch.matmul on the same tensors, row-major [K,N] weights, graph replays; no activation pass"}
    del o_cat
    # K-contiguous weights (the layout the vendor's fastest kernel wants): same products, weights stored transposed
    progress("vendor GEMMs, K-contiguous weights")
    w_cat_t = w_cat.t().contiguous().t()
    o_cat = torch.empty(T, 2 * F, dtype=torch.float16, device=dev)
    res["vendor_gemm_us"]["gateup_plain_wT"] = graph_time_us(lambda: torch.matmul(x, w_cat_t, out=o_cat))
    del o_cat, w_cat, w_cat_t
    wd_t = wd.t().contiguous().t()
    res["vendor_gemm_us"]["down_proj_wT"] = graph_time_us(lambda: torch.matmul(hid, wd_t, out=out))
    del wd_t
    progress("gate/up on random and on zero data")
    # this library on K-contiguous weights (same values, W stored as W^T [N][K]; stride[0] == 1 at the boundary)
    wg_t, wu_t, wd_t = wg.t().contiguous().t(), wu.t().contiguous().t(), wd.t().contiguous().t()
    us_gu_t = graph_time_us(lambda: ext.gateup_swiglu(x, wg_t, wu_t, None, hid))
    us_dn_t = graph_time_us(lambda: ext.matmul(hid, wd_t, None, out))
    us_ffn_t = graph_time_us(lambda: ext.ffn_swiglu(x, wg_t, wu_t, wd_t, hid, out))
    fl = 3.0 * 2 * T * N * F
    res["ffn_swiglu_llama3_8b_T2048_wT"] = {
        "us": us_ffn_t, "TFLOPs": fl / us_ffn_t * 1e-6, "frac_mfma": fl / us_ffn_t * 1e-6 / PEAK_FP16_TFLOPS,
        "gateup_swiglu_us": us_gu_t, "down_proj_us": us_dn_t,
        "gateup_frac_mfma": 2.0 * 2 * T * N * F / us_gu_t * 1e-6 / PEAK_FP16_TFLOPS,
        "note": "the step's FFN with W_gate / W_up / W_down stored K-contiguous (graph replays)"}
    del wg_t, wu_t, wd_t
    us_rand = graph_time_us(lambda: ext.gateup_swiglu(x, wg, wu, None, hid))
    zx, zg, zu = torch.zeros_like(x), torch.zeros_like(wg), torch.zeros_like(wu)
    us_zero = graph_time_us(lambda: ext.gateup_swiglu(zx, zg, zu, None, hid))
    res["gateup_random_data_us"] = us_rand
    res["gateup_zero_data_us"] = us_zero
    res["gateup_zero_over_random"] = us_zero / us_rand
    return res


def vendor_only(dev, T, N, F, calls=3):
    """Only the vendor library's kernels for the two products of the step, a few eager calls each: the program
    whose hipBLASLt counter columns `rocprofv3 --pmc ... -- python3 bench.py --only-vendor` collects."""
    g = _gen(42)
    x = _randn(g, T, N)
    w_cat = torch.cat([_randn(g, N, F, std=0.02), _randn(g, N, F, std=0.02)], dim=1)
    wd = _randn(g, F, N, std=0.02)
    hid = _randn(g, T, F, std=0.3)
    o_cat = torch.empty(T, 2 * F, dtype=torch.float16, device=dev)
    out = torch.empty(T, N, dtype=torch.float16, device=dev)
    legs = {}
    for name, a, w, o in (("gateup_plain", x, w_cat, o_cat), ("down_proj", hid, wd, out),
                          ("gateup_plain_wT", x, w_cat.t().contiguous().t(), o_cat),
                          ("down_proj_wT", hid, wd.t().contiguous().t(), out)):
        progress("vendor " + name)
        for _ in range(2):
            torch.matmul(a, w, out=o)
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(calls):
            torch.matmul(a, w, out=o)
        end.record()
        torch.cuda.synchronize()
        legs[name] = start.elapsed_time(end) / calls * 1e3
    return {"vendor_gemm_us": legs, "note": "torch.matmul (hipBLASLt), eager calls, no activation pass"}


def microbench(ext):
    """The issue probe: what a group of one MFMA, n v_fma_f32 and t v_exp_f32 costs a SIMD, with one and with two
    waves per SIMD, one workgroup on each of 256 CUs.  ns and shader-clock ticks per group and wave."""
    rows = []
    ext.issue_probe(True, 4, 0, 2)  # warm-up (clock, code load)
    for waves in (1, 2):
        for mfma, nv, nt in ((1, 0, 0), (0, 4, 0), (0, 8, 0), (0, 12, 0), (0, 16, 0), (0, 0, 2), (0, 0, 4),
                             (1, 2, 0), (1, 4, 0), (1, 6, 0), (1, 8, 0), (1, 12, 0), (1, 16, 0),
                             (1, 0, 1), (1, 0, 2), (1, 4, 1), (1, 8, 1), (1, 8, 2), (1, 16, 4)):
            best = min((ext.issue_probe(mfma, nv, nt, waves) for _ in range(3)), key=lambda r: r[1])
            rows.append({"waves_per_simd": waves, "mfma": mfma, "v_fma": nv, "v_exp": nt,
                         "ticks_per_group": round(best[0], 2), "ns_per_group": round(best[1], 3),
                         # a SIMD serves `waves` waves: its time per group of ONE wave
                         "ns_per_group_per_simd": round(best[1] / waves, 3)})
    # three and four waves per SIMD, the groups that show most what a further wave buys
    for waves in (3, 4):
        for mfma, nv, nt in ((0, 16, 0), (1, 8, 0), (1, 16, 0), (1, 8, 2), (1, 16, 4)):
            best = min((ext.issue_probe(mfma, nv, nt, waves) for _ in range(3)), key=lambda r: r[1])
            rows.append({"waves_per_simd": waves, "mfma": mfma, "v_fma": nv, "v_exp": nt,
                         "ticks_per_group": round(best[0], 2), "ns_per_group": round(best[1], 3),
                         "ns_per_group_per_simd": round(best[1] / waves, 3)})
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-blocks", action="store_true", help="skip the per-block table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-power-legs", action="store_true",
                    help="skip the vendor-GEMM, zero-data and K-contiguous-weight legs of the step's two products")
    ap.add_argument("--quick", action="store_true", help="smaller block table (one sequence length each)")
    ap.add_argument("--replays", type=int, default=100, help="graph replays per block of the tables")
    ap.add_argument("--only-block", default=None,
                    help="of the tables, run only the blocks whose name contains this (for profiling one block)")
    ap.add_argument("--no-step", action="store_true",
                    help="with --only-block: skip the headline step as well (nothing but that block's kernels run)")
    ap.add_argument("--only-reference-shapes", action="store_true",
                    help="of the tables, run only the reference-shape one (M = 16, P = 1024)")
    ap.add_argument("--only-vendor", action="store_true",
                    help="run nothing but the vendor library's products of the step (torch.matmul: gate/up and down, row-major and "
                         "K-contiguous weights), a few eager calls each - the program to put after `rocprofv3 --pmc ... --`")
    ap.add_argument("--microbench", action="store_true",
                    help="run only the issue microbenchmark (one MFMA followed by n vector instructions, one and two waves per SIMD)")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy (a kernel of known traffic to scale rocprofv3 byte counters by)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU's share of the path; run with --gpus 1 "
                 "(nothing on this path communicates between GPUs)")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    global REPLAYS
    REPLAYS = max(1, args.replays)
    from trinity_amd import ext

    ext.lib()  # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    T, N, F = 2048, 4096, 14336
    if args.only_block and args.no_step:
        print(json.dumps({"blocks": bench_blocks(ext, dev, quick=args.quick, only=args.only_block)}))
        return
    if args.only_vendor:
        print(json.dumps(vendor_only(dev, T, N, F)))
        return
    if args.microbench:
        print(json.dumps({"issue_probe": microbench(ext), "power_probe": power_model(ext)}))
        return
    g = _gen(42)
    x = _randn(g, T, N)
    wg, wu = _randn(g, N, F, std=0.02), _randn(g, N, F, std=0.02)
    wd = _randn(g, F, N, std=0.02)
    hid = torch.empty(T, F, dtype=torch.float16, device=dev)
    out = torch.empty(T, N, dtype=torch.float16, device=dev)

    def step(events=None):
        if events is not None:
            events[0].record()
        ext.gateup_swiglu(x, wg, wu, None, hid)
        if events is not None:
            events[1].record()
        ext.matmul(hid, wd, None, out)
        if events is not None:
            events[2].record()

    def run_tables():
        res = {}
        if not args.no_blocks:
            # (the small reference shapes first: the tables then end on the large blocks, whose kernels load the
            # device as the step's do)
            if not args.only_block:
                res["reference_shape_blocks"] = bench_reference_shapes(ext, dev)
            torch.cuda.empty_cache()
            if not args.only_reference_shapes:
                res["issue_model"] = issue_model(ext)
                res["power_model"] = power_model(ext)
                res["blocks"] = bench_blocks(ext, dev, quick=args.quick, only=args.only_block)
                add_issue_bounds(res["blocks"], res["issue_model"])
                add_power_bounds(res["blocks"], res["power_model"])
            torch.cuda.empty_cache()
        return res

    if args.pmc_calibration:
        ca = torch.ones(256 << 20, dtype=torch.uint8, device=dev)
        cb = torch.empty_like(ca)
        for _ in range(3):
            cb.copy_(ca)
        torch.cuda.synchronize()
        del ca, cb
    def timed_steps():
        """W untimed steps, then exactly K timed ones between two synchronisations: wall-clock ms per step and the
        per-step event times (us) of the two launches and of the step, in launch order."""
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            step(evs[i])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        return (dt / args.steps * 1e3, [e[0].elapsed_time(e[1]) * 1e3 for e in evs],
                [e[1].elapsed_time(e[2]) * 1e3 for e in evs], [e[0].elapsed_time(e[2]) * 1e3 for e in evs])

    # The headline: the W + K steps are the process's first GPU work, nothing runs before them.  (A fresh process
    # finds the device at its idle clocks and these steps - some 20 ms - end before it has left them: the series
    # shows the launch times falling; the same steps are timed once more after the block tables, see below.)
    progress("step: %d warm-up + %d timed" % (args.warmup, args.steps))
    ms_per_step, gateup_series, down_series, step_series = timed_steps()
    gateup_ms = sum(gateup_series) / args.steps * 1e-3
    down_ms = sum(down_series) / args.steps * 1e-3
    assert torch.isfinite(out).all()
    # the same step timed as the reference times its modules (convert_eval_rms.py:253-275): 10 warm-up calls on a
    # side stream, one captured graph, 100 replays between two events
    progress("step: graph replays")
    step_graph_us = graph_time_us(step)
    gateup_graph_us = graph_time_us(lambda: ext.gateup_swiglu(x, wg, wu, None, hid))
    down_graph_us = graph_time_us(lambda: ext.matmul(hid, wd, None, out))

    traffic, traffic_src = _traffic_from_profile()
    flops_step = 3.0 * 2 * T * N * F
    flops_gateup = 2.0 * 2 * T * N * F
    achieved = flops_gateup / (gateup_ms * 1e-3) * 1e-12
    frac_of = lambda us: flops_gateup / us * 1e-6 / PEAK_FP16_TFLOPS
    rnd = lambda xs: [round(v, 1) for v in xs]
    result = {
        "metric": "TFLOP/s of one fused SwiGLU FFN call (us/call in ms_per_step; % of fp16 MFMA peak in roofline)",
        "value": flops_step / (ms_per_step * 1e-3) * 1e-12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "Llama-3-8B fused SwiGLU FFN, X [2048,4096] fp16, W_gate/W_up [4096,14336], W_down [14336,4096], fp32 accumulate"},
        "roofline": {
            "bound": "mfma",
            "kernel": "tri::gemm_epi_kernel<DmaTile<256,256,2,2>, DmaTile<256,128,2,2>, 2> (gate/up GEMM + SwiGLU epilogue, one launch)",
            "achieved": achieved,
            "peak": PEAK_FP16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / PEAK_FP16_TFLOPS,
            "avg_launch_us": gateup_ms * 1e3,
            # the same launch by three other readings: median and minimum of the timed steps' event times, and the
            # mean of 100 graph replays after 10 warm-up calls (the reference's timing protocol)
            "median_launch_us": _median(gateup_series),
            "min_launch_us": min(gateup_series),
            "graph_launch_us": gateup_graph_us,
            "frac_median": frac_of(_median(gateup_series)),
            "frac_graph": frac_of(gateup_graph_us),
            # FETCH_SIZE x 2.0 + WRITE_SIZE of this launch on this workload (rocprofv3 --pmc, scaled by a plain
            # 256 MiB copy; the summary is under profiles/)
            "traffic": traffic,
            "traffic_source": traffic_src,
            # event times of every timed step, in launch order (us)
            "series_us": {"gateup_swiglu": rnd(gateup_series), "down_proj": rnd(down_series), "step": rnd(step_series)},
            "step_us": {"wall_mean": ms_per_step * 1e3, "event_mean": sum(step_series) / args.steps,
                        "event_median": _median(step_series), "event_min": min(step_series), "graph": step_graph_us,
                        "frac_mfma_wall_mean": flops_step / ms_per_step * 1e-9 / PEAK_FP16_TFLOPS,
                        "frac_mfma_event_median": flops_step / _median(step_series) * 1e-6 / PEAK_FP16_TFLOPS,
                        "frac_mfma_graph": flops_step / step_graph_us * 1e-6 / PEAK_FP16_TFLOPS},
        },
        "kernels_us": {"gateup_swiglu": gateup_ms * 1e3, "down_proj": down_ms * 1e3,
                       "gateup_swiglu_median": _median(gateup_series), "down_proj_median": _median(down_series),
                       "gateup_swiglu_graph": gateup_graph_us, "down_proj_graph": down_graph_us},
        "step_graph_us": step_graph_us,
    }
    if not args.no_power_legs:
        result.update(power_legs(ext, dev, x, wg, wu, wd, hid, out))
    tables = run_tables()
    result.update(tables)
    if tables:
        # the same W + K eager steps once more, now that the device has been busy for a while: not the headline
        progress("step: %d warm-up + %d timed, after the tables" % (args.warmup, args.steps))
        ms2, gu2, dn2, st2 = timed_steps()
        result["roofline"]["after_tables"] = {
            "ms_per_step": ms2, "value_TFLOPs": flops_step / (ms2 * 1e-3) * 1e-12,
            "avg_launch_us": sum(gu2) / len(gu2), "median_launch_us": _median(gu2),
            "frac": frac_of(sum(gu2) / len(gu2)), "frac_median": frac_of(_median(gu2)),
            "series_us": {"gateup_swiglu": rnd(gu2), "down_proj": rnd(dn2), "step": rnd(st2)}}
    del x, wg, wu, wd, hid, out
    torch.cuda.empty_cache()
    if "power_model" in result:
        # the published peak assumes 2.4 GHz; on random operands the matrix pipe alone already holds the board at
        # its power limit at a lower clock - the rate of the pure MFMA loop of the power probe
        lim = result["power_model"]["mfma_TFLOPs_at_power_limit"]
        result["roofline"]["mfma_TFLOPs_at_power_limit"] = lim
        result["roofline"]["frac_of_power_limit"] = achieved / lim
        result["roofline"]["frac_graph_of_power_limit"] = flops_gateup / gateup_graph_us * 1e-6 / lim
        # ... and with half an LDS read and a quarter of a global -> LDS load per MFMA beside it, which no GEMM
        # on 256 x 256 tiles does without
        result["roofline"]["gemm_mix_TFLOPs_at_power_limit"] = result["power_model"]["gemm_mix_TFLOPs_at_power_limit"]
        # (the fitted costs once more inside `roofline`: ns of a SIMD per wave instruction at the power limit)
        result["roofline"]["power_model_ns"] = {k: round(result["power_model"][k], 3) for k in
                                                ("mfma_ns", "lds_read_ns", "valu_ns", "trans_ns", "dma_load_ns")}
        result["roofline"]["frac_graph_of_gemm_mix_at_power_limit"] = (
            flops_gateup / gateup_graph_us * 1e-6 / result["power_model"]["gemm_mix_TFLOPs_at_power_limit"])
    # every block's us and fraction of its roofline once more inside `roofline`, in a compact form
    table = {}
    for rec in result.get("blocks", []) + result.get("reference_shape_blocks", []):
        table[rec["block"]] = [round(rec["us"], 1), round(rec.get("frac_mfma", rec.get("frac_hbm", 0.0)), 4)]
        if "issue_bound_us" in rec:   # [us, fraction of roofline, issue-bound us, issue bound / kernel time, ...
            table[rec["block"]] += [round(rec["issue_bound_us"], 1), round(rec["frac_of_issue_bound"], 3)]
        if "power_bound_us" in rec:   # ... power-bound us, power bound / block time]
            table[rec["block"]] += [round(rec["power_bound_us"], 1), round(rec["frac_of_power_bound"], 3)]
    if "ffn_swiglu_llama3_8b_T2048_wT" in result:
        r = result["ffn_swiglu_llama3_8b_T2048_wT"]
        table["ffn_swiglu_llama3_8b_T2048_wT"] = [round(r["us"], 1), round(r["frac_mfma"], 4)]
    if table:
        result["roofline"]["blocks_us_frac"] = table
    if "vendor_gemm_us" in result:
        result["roofline"]["vendor_gemm_us"] = {k: round(v, 1) for k, v in result["vendor_gemm_us"].items()
                                                 if isinstance(v, float) and not k.endswith("TFLOPs")}
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(T, N, F, sample_rows=T)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
