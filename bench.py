#!/usr/bin/env python3
"""Benchmark of the quantized GGUF matmul hot path on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input: marmot_linear with a Q4_K weight of
4096 x 14336 (Llama-3-8B FFN down projection, marmot M x K) and one fp32 activation row — activation
quantization to Q8_K on the device followed by the decode matvec. Weights rotate over enough distinct
copies to exceed the 256 MB Infinity Cache, so the figure is an HBM figure, not a cache figure.

Prints ONE JSON line (see README / the driver contract): `value` is whole-op GB/s (algorithmic bytes of the
op / wall time per step, inputs resident in HBM), `roofline` describes the dominant kernel (the matvec,
timed alone with HIP events on the library's stream), `cpu_baseline` is the CPU oracle timed on the host.
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
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "Q4_K matvec GB/s (% HBM peak) + prefill GEMM TOPS (% MFMA peak)"
HBM_PEAK_GBPS = 8000.0
MALL_BYTES = 256 << 20
# HBM bytes per launch of the Q4_K 4096x14336 N=1 matvec kernels (rocprofv3 FETCH_SIZE + WRITE_SIZE scaled by a plain
# copy kernel, profiles/matvec_q4_k_4096x14336_n1.md): the resident-share kernel with the activation quantization
# inside (k_matvec_rows2_q4k) and the streaming kernel on pre-packed activations (k_matvec_ls)
TRAFFIC_FUSED = 33_667_000
TRAFFIC_PREPACKED = 33_288_000


def algorithmic_bytes(kind_row_bytes: int, M: int, K: int, N: int) -> int:
    """Compulsory traffic of one linear: weights at true block bytes + fp32 activations in + fp32 outputs out."""
    return M * kind_row_bytes + N * K * 4 + N * M * 4


def random_blocks(rng, kind: int, rows: int, k: int) -> np.ndarray:
    """Synthetic weights: arbitrary block payloads with finite, small fp16 super-block scales."""
    from marmot_amd import block_bytes, block_values

    nb = (k + block_values(kind) - 1) // block_values(kind)
    bb = block_bytes(kind)
    raw = rng.integers(0, 256, size=(rows * nb, bb), dtype=np.uint8)
    offs = {1: [0], 2: [0, 2], 3: [0], 4: [0, 2], 5: [0], 6: [0, 2], 7: [80, 82], 8: [108], 9: [0, 2], 10: [0, 2], 11: [208]}[kind]
    for off in offs:
        h = raw[:, off:off + 2].copy().view(np.uint16)
        h = (h & 0x83FF) | 0x2000  # exponent field 8: magnitudes around 2^-7
        raw[:, off:off + 2] = h.view(np.uint8)
    return raw.reshape(rows, nb * bb)


# statistics of the most recent time_steps_graph call (the headline leg copies them into its JSON line)
LAST_TIMING: dict = {}


def time_steps_graph(hip, fn, steps: int, warmup: int, chunk: int = 500, repeats: int = 7, settle_ms: float = 50.0):
    """Like time_steps, but the timed steps are replayed from HIP graphs, so the host's launch rate does not enter the
    figure. A graph holds up to `chunk` steps and never more nodes than the library allows per graph (the node count of
    one step is measured by capturing one). The EXACTLY `steps` timed steps are bracketed by two time-stamp kernels
    recorded INSIDE the captured graphs (first node of the first graph, last node of the last one; they store the
    device's 100 MHz counter, HIP events cannot be read back from graph nodes on this runtime), so the submission of a
    graph is not in the figure and a repeat of 20 steps reads like one of 2000; the interval includes one launch gap
    and the first stamp kernel's run more than the steps need (about 1.5 us per repeat, on the slow side). Before
    anything is timed the graphs are replayed until `settle_ms` of GPU time have passed (the clocks need tens of
    milliseconds under load to settle); then `repeats` replays are timed one by one. Returns the MEDIAN repeat in ms
    per step; min / max / repeats go to LAST_TIMING."""
    import ctypes as C

    for i in range(warmup):
        fn(i)
    hip.synchronize()
    probe = hip.graph_capture(lambda: fn(warmup))
    per_step = max(1, hip.graph_last_capture_nodes())
    hip.graph_destroy(probe)
    # Under rocprofv3 (it exports ROCPROF_* / ROCP_* variables to the program it starts) the steps are replayed twice
    # only (no settling, one timed repeat), from graphs of 100 steps that are synchronized one by one: the queue
    # interception of its kernel trace ends in a segmentation fault inside hipGraphLaunch once about ten thousand
    # kernels of one process have gone through graph launches (observed: after 96 replays of 100-step graphs; 2200
    # such kernels per call of this function are fine). The profiler's own per-kernel durations are what such a run is
    # for, not this function's figure.
    profiled = any(k.startswith(("ROCPROF", "ROCP_")) for k in os.environ)
    if profiled:
        chunk, repeats, settle_ms = min(chunk, 100), 1, 0.0
    chunk = max(1, min(chunk, (hip.graph_max_nodes() - 2) // per_step))
    stamps = hip.alloc(16)
    n_graphs = -(-steps // chunk)
    graphs = []
    done = 0
    while done < steps:
        n = min(chunk, steps - done)
        base = warmup + done
        first, last = len(graphs) == 0, len(graphs) == n_graphs - 1

        def body():
            if first:
                hip.lib.marmot_hip_timestamp(hip.dev, C.c_void_p(stamps.ptr))
            for j in range(n):
                fn(base + j)
            if last:
                hip.lib.marmot_hip_timestamp(hip.dev, C.c_void_p(stamps.ptr + 8))

        graphs.append(hip.graph_capture(body))
        done += n

    def replay_ms():
        for g in graphs:
            hip.graph_launch(g)
            if profiled:
                hip.synchronize()
        hip.synchronize()
        t = stamps.download(np.uint64, (2,))
        return float(int(t[1]) - int(t[0])) * 1e-5  # 10 ns ticks -> ms

    # ---- settle: untimed replays until settle_ms of GPU time have passed
    once_ms = max(replay_ms(), 1e-3)
    settle_replays = min(20000, int(settle_ms / once_ms) + 1) if settle_ms > 0 else 0
    for _ in range(settle_replays):
        for g in graphs:
            hip.graph_launch(g)
            if profiled:
                hip.synchronize()
    hip.synchronize()
    # ---- timed repeats
    per_repeat = sorted(replay_ms() / steps for _ in range(repeats))
    for g in graphs:
        hip.graph_destroy(g)
    stamps.free()
    mid = len(per_repeat) // 2
    med = per_repeat[mid] if len(per_repeat) % 2 else 0.5 * (per_repeat[mid - 1] + per_repeat[mid])
    LAST_TIMING.clear()
    LAST_TIMING.update({"repeats": repeats, "ms_per_step_min": per_repeat[0], "ms_per_step_max": per_repeat[-1],
                        "settle_replays": settle_replays, "steps_per_repeat": steps})
    return med


def time_steps(hip, fn, steps: int, warmup: int):
    """Runs fn(i) for warmup + steps launches; returns (ms per step by HIP events, ms per step by host clock)."""
    for i in range(warmup):
        fn(i)
    hip.synchronize()
    e0, e1 = hip.event(), hip.event()
    t0 = time.perf_counter()
    hip.record(e0)
    for i in range(steps):
        fn(warmup + i)
    hip.record(e1)
    hip.synchronize()
    t1 = time.perf_counter()
    ev_ms = hip.elapsed_ms(e0, e1)
    return ev_ms / steps, (t1 - t0) * 1e3 / steps


def cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(kind, blocks, x, M, K, nbytes, ref_out, budget_s: float):
    """The CPU oracle (a restatement of the reference's CPU path) on the host cores, same workload: rows split over
    T = every core this process may run on (the reference's own default is a topology-derived count), and T = 1."""
    from oracle.pyoracle import Oracle

    oracle = Oracle()
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    out = oracle.matmul(kind, blocks, x, M, threads=cores)  # warm-up, and the parity check of the GPU result
    rms = float(np.sqrt(np.mean(out.astype(np.float64) ** 2)))
    err = float(np.max(np.abs(ref_out - out) / np.maximum(np.abs(out), 1e-3 * rms)))
    times = []
    t_end = time.perf_counter() + budget_s
    while time.perf_counter() < t_end and len(times) < 2000:
        t0 = time.perf_counter()
        oracle.matmul(kind, blocks, x, M, threads=cores)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    t1 = []
    for _ in range(3):
        t0 = time.perf_counter()
        oracle.matmul(kind, blocks, x, M, threads=1)
        t1.append(time.perf_counter() - t0)
    return {
        "value": round(nbytes / med / 1e9, 3),
        "unit": "GB/s",
        "cores": cores,
        "cpu_model": cpu_model(),
        "kind": "port",
        "sample": f"{len(times)} runs of the same Q4_K {M}x{K} N={x.shape[0]} linear (median), threads split over "
                  f"weight rows with the reference's grain rule",
        "ms_per_step": round(med * 1e3, 4),
        "single_thread_gbps": round(nbytes / float(np.median(t1)) / 1e9, 3),
    }, err


def read_calibration(hip, nbytes: int, steps: int, warmup: int):
    """The read-only streaming kernel (16-byte loads, nothing written) over `nbytes` per launch, dependent launches
    replayed from a HIP graph, rotating over copies larger than twice the Infinity Cache like the matvec's weights:
    the read bandwidth this box delivers to one launch of that size."""
    nbytes = (nbytes + 255) & ~255
    copies = max(2, -(-2 * MALL_BYTES // nbytes) + 1)
    buf = hip.alloc(nbytes * copies)
    hip.lib.marmot_hip_memset(hip.dev, buf.ptr, 0xFF, nbytes * copies)
    sink = hip.alloc(1024)
    ms = time_steps_graph(hip, lambda i: hip.read_probe_d(buf, nbytes, sink, offset=(i % copies) * nbytes), steps, warmup)
    buf.free()
    sink.free()
    return {"calibration": "read-only 16-byte streaming kernel, one dependent launch per step", "bytes_per_launch": nbytes,
            "copies": copies, "us_per_launch": round(ms * 1e3, 3), "gbps": round(nbytes / ms / 1e6, 1)}


def prefill_gemm(hip, tokens: int, steps: int, warmup: int):
    """Q4_K prefill GEMM leg: marmot_linear with fp16 activations [tokens, 4096] and a 4096 x 4096 Q4_K weight."""
    from marmot_amd import DT_F16, DT_F32, capi, row_bytes

    M = K = 4096
    kind = capi.KIND_Q4_K
    blocks = random_blocks(np.random.Generator(np.random.PCG64(30)), kind, M, K)
    x = np.random.Generator(np.random.PCG64(31)).standard_normal((tokens, K), dtype=np.float32).astype(np.float16)
    d_w, d_x = hip.to_device(blocks), hip.to_device(x)
    d_out = hip.alloc(tokens * M * 4)

    def step(i):
        hip.linear_d(kind, d_w, d_x, DT_F16, tokens, K, M, d_out, DT_F32)

    ms = time_steps_graph(hip, step, steps, warmup, chunk=50)
    flops = 2.0 * tokens * M * K
    out = {
        "workload": f"Q4_K prefill GEMM, weight {M}x{K}, {tokens} tokens fp16, fp32 out (fp16 MFMA, fp32 accumulate)",
        "route": hip.last_route(),
        "ms_per_step": round(ms, 5),
        "tflops": round(flops / (ms * 1e-3) / 1e12, 2),
        "peak_tflops": 2500.0,
        "frac_of_mfma_peak": round(flops / (ms * 1e-3) / 1e12 / 2500.0, 4),
        "tokens_per_s": round(tokens / (ms * 1e-3), 1),
        "steps": steps,
        "includes": "every kernel of the op (512 tokens: one launch, sub-block sums computed inside; K-split partials and their reduction only below half a chip of tiles)",
    }
    for b in (d_w, d_x, d_out):
        b.free()
    return out


def prefill_int8(hip, tokens: int, steps: int, warmup: int):
    """Q4_K prefill with fp32 activations (what marmot's own graph feeds): the reference's integer path, i.e. the
    activations are quantized to Q8_K (one launch) and the tiled int8 GEMM follows; weight 4096 x 4096."""
    from marmot_amd import DT_F32, capi

    M = K = 4096
    kind = capi.KIND_Q4_K
    blocks = random_blocks(np.random.Generator(np.random.PCG64(32)), kind, M, K)
    x = np.random.Generator(np.random.PCG64(33)).standard_normal((tokens, K), dtype=np.float32)
    d_w, d_x = hip.to_device(blocks), hip.to_device(x)
    d_out = hip.alloc(tokens * M * 4)
    ms = time_steps_graph(hip, lambda i: hip.linear_d(kind, d_w, d_x, DT_F32, tokens, K, M, d_out, DT_F32), steps,
                          warmup, chunk=20)
    ops = 2.0 * tokens * M * K
    out = {
        "workload": f"Q4_K prefill, weight {M}x{K}, {tokens} tokens fp32 -> Q8_K on device, fp32 out (int8 MFMA, "
                    f"exact integer block sums, fp32 accumulate over blocks)",
        "route": hip.last_route(),
        "ms_per_step": round(ms, 5),
        "tops": round(ops / (ms * 1e-3) / 1e12, 2),
        "peak_tops": 5000.0,
        "frac_of_int8_mfma_peak": round(ops / (ms * 1e-3) / 1e12 / 5000.0, 4),
        "tokens_per_s": round(tokens / (ms * 1e-3), 1),
        "steps": steps,
        "includes": "activation quantization launch and the GEMM kernel",
    }
    for b in (d_w, d_x, d_out):
        b.free()
    return out


def sweep(hip, steps: int, warmup: int, only=("C1", "C2", "C3", "C4", "C4P", "BRANCH", "C5", "QKV", "OPS", "ATTN", "LAYER", "LOGITS", "Q5K", "LEGACY", "Q23K", "PREFILL32", "PREFILLFMT")):
    """Every benchmark configuration (C1..C5, C4P, BRANCH, QKV, OPS, ATTN, LAYER, LOGITS, Q5K, LEGACY, Q23K, PREFILL32, PREFILLFMT) on the device, one JSON line each (documentation runs, not the
    driver's line): weights rotate over copies larger than twice the Infinity Cache; times are HIP-graph replays."""
    from marmot_amd import DT_F16, DT_F32, capi, row_bytes

    rng = np.random.Generator(np.random.PCG64(7))
    names = {capi.KIND_Q4_K: "Q4_K", capi.KIND_Q5_K: "Q5_K", capi.KIND_Q6_K: "Q6_K", capi.KIND_Q8_0: "Q8_0",
             capi.KIND_Q4_0: "Q4_0", capi.KIND_Q4_1: "Q4_1", capi.KIND_Q5_0: "Q5_0", capi.KIND_Q5_1: "Q5_1",
             capi.KIND_Q2_K: "Q2_K", capi.KIND_Q3_K: "Q3_K"}

    def emit(rec):
        print(json.dumps(rec), flush=True)

    def linear_case(config, kind, M, K, N):
        rb = row_bytes(kind, K)
        stride = (M * rb + 255) & ~255
        copies = max(2, -(-2 * MALL_BYTES // stride) + 1)
        blocks = random_blocks(rng, kind, M, K)
        d_w = hip.alloc(stride * copies)
        for c in range(copies):
            d_w.upload(blocks, offset=c * stride)
        d_x = hip.to_device(rng.standard_normal((N, K), dtype=np.float32))
        d_out = hip.alloc(N * M * 4)
        ms = time_steps_graph(hip, lambda i: hip.linear_d(kind, d_w, d_x, DT_F32, N, K, M, d_out, DT_F32,
                                                          weight_offset=(i % copies) * stride), steps, warmup)
        nbytes = algorithmic_bytes(rb, M, K, N)
        emit({"config": config, "workload": f"{names[kind]} {M}x{K} N={N}", "route": hip.last_route(),
              "us": round(ms * 1e3, 2), "GB/s": round(nbytes / ms / 1e6, 1),
              "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4), "tokens_per_s": round(N / ms * 1e3)})
        for b in (d_w, d_x, d_out):
            b.free()

    if "C1" in only:
        linear_case("C1", capi.KIND_Q8_0, 5632, 2048, 1)
    for kind in (capi.KIND_Q4_K, capi.KIND_Q6_K):
        for (M, K) in ((14336, 4096), (4096, 14336)):
            for N in (1, 4, 8):
                if "C2" in only:
                    linear_case("C2", kind, M, K, N)
    for tokens in (64, 128, 512, 2048) if "C3" in only else ():
        r = prefill_gemm(hip, tokens, max(100, steps // 2), max(20, steps // 20))
        emit({"config": "C3", "workload": f"Q4_K 4096x4096 N={tokens} fp16", "route": r["route"],
              "us": round(r["ms_per_step"] * 1e3, 2), "TFLOP/s": r["tflops"],
              "frac_of_mfma_peak": r["frac_of_mfma_peak"], "tokens_per_s": round(r["tokens_per_s"])})

    if "Q5K" in only:
        # the C2 shapes with Q5_K weights (the feed-forward matrices of a Q5_K_M file), decode and small batch
        for (M, K) in ((14336, 4096), (4096, 14336)):
            for N in (1, 4, 8, 16):
                linear_case("Q5K", capi.KIND_Q5_K, M, K, N)
    if "PREFILL32" in only:
        # prefill with fp32 activations: the reference's integer path (Q8_K activations), small-batch MFMA kernel in
        # passes of 32 rows (Q4_K, Q5_K) or 16 rows (Q6_K); one weight copy (the passes re-read it from the caches)
        for kind in (capi.KIND_Q4_K, capi.KIND_Q5_K, capi.KIND_Q6_K):
            for N in (32, 128, 512):
                M = K = 4096
                d_w = hip.to_device(random_blocks(rng, kind, M, K))
                d_x = hip.to_device(rng.standard_normal((N, K), dtype=np.float32))
                d_out = hip.alloc(N * M * 4)
                step = lambda i: hip.linear_d(kind, d_w, d_x, DT_F32, N, K, M, d_out, DT_F32)
                if os.environ.get("MARMOT_BENCH_EAGER"):  # plain launches (for kernel traces), host rate included
                    ms, _ = time_steps(hip, step, max(40, steps // 20), 10)
                else:
                    ms = time_steps_graph(hip, step, max(40, steps // 20), 10, chunk=20)
                emit({"config": "PREFILL32", "workload": f"{names[kind]} {M}x{K} N={N} fp32 activations",
                      "route": hip.last_route(), "us": round(ms * 1e3, 1),
                      "TOP/s": round(2.0 * N * M * K / ms / 1e9, 1), "tokens_per_s": round(N / ms * 1e3)})
                for b in (d_w, d_x, d_out):
                    b.free()
    if "PREFILLFMT" in only:
        # prefill for the other formats: the 32-value formats and Q2_K / Q3_K with fp32 activations (integer path) and
        # fp16 activations (direct route: decoded weights on the fp16 matrix cores)
        from marmot_amd import DT_F16
        for kind, dt in ((capi.KIND_Q8_0, DT_F32), (capi.KIND_Q4_0, DT_F32), (capi.KIND_Q4_1, DT_F32),
                         (capi.KIND_Q5_0, DT_F32), (capi.KIND_Q5_1, DT_F32), (capi.KIND_Q2_K, DT_F32),
                         (capi.KIND_Q3_K, DT_F32), (capi.KIND_Q8_0, DT_F16), (capi.KIND_Q4_0, DT_F16),
                         (capi.KIND_Q6_K, DT_F16), (capi.KIND_Q5_K, DT_F16), (capi.KIND_Q4_1, DT_F16)):
            for N in (16, 128, 512):
                M = K = 4096
                d_w = hip.to_device(random_blocks(rng, kind, M, K))
                x = rng.standard_normal((N, K), dtype=np.float32)
                d_x = hip.to_device(x if dt == DT_F32 else x.astype(np.float16))
                d_out = hip.alloc(N * M * 4)
                step = lambda i: hip.linear_d(kind, d_w, d_x, dt, N, K, M, d_out, DT_F32)
                ms = time_steps_graph(hip, step, max(40, steps // 20), 10, chunk=20)
                emit({"config": "PREFILLFMT",
                      "workload": f"{names[kind]} {M}x{K} N={N} {'fp32' if dt == DT_F32 else 'fp16'} activations",
                      "route": hip.last_route(), "us": round(ms * 1e3, 1),
                      "TOP/s": round(2.0 * N * M * K / ms / 1e9, 1), "tokens_per_s": round(N / ms * 1e3)})
                for b in (d_w, d_x, d_out):
                    b.free()
    if "Q23K" in only:
        # the low-bit K formats on the dot-product matvec (four lanes per block), decode and small batch
        for kind in (capi.KIND_Q2_K, capi.KIND_Q3_K):
            for N in (1, 4, 8):
                linear_case("Q23K", kind, 14336, 4096, N)
    if "LEGACY" in only:
        # the 32-value formats on the dot-product matvec (one lane per block), decode sizes
        for kind in (capi.KIND_Q4_0, capi.KIND_Q4_1, capi.KIND_Q5_0, capi.KIND_Q5_1, capi.KIND_Q8_0):
            for N in (1, 4):
                linear_case("LEGACY", kind, 14336, 4096, N)
    if "C4" in only:
        sweep_layer_stack(hip, rng, emit, steps)
    if "C4P" in only:
        sweep_layer_stack(hip, rng, emit, steps, N=512, config="C4P")
    if "BRANCH" in only:
        sweep_branches(hip, rng, emit, steps)
    if "C5" in only:
        sweep_moe(hip, rng, emit, steps)
    if "QKV" in only:
        sweep_qkv(hip, rng, emit, steps, warmup)
    if "OPS" in only:
        sweep_ops(hip, rng, emit, steps, warmup)
    if "ATTN" in only:
        sweep_attention(hip, rng, emit, steps)
    if "LAYER" in only:
        sweep_whole_layer(hip, rng, emit, steps)
    if "LOGITS" in only:
        # the vocabulary-sized matvec at the end of a decode step (Llama-3 vocabulary, 128256 rows of 4096)
        for kind in (capi.KIND_Q6_K, capi.KIND_Q4_K):
            for N in (1, 4):
                linear_case("LOGITS", kind, 128256, 4096, N)


def sweep_ops(hip, rng, emit, steps: int, warmup: int):
    """The operations between the linears at decode and prefill sizes of a Llama-3-8B layer: RMS normalization and
    residual add over [T, 4096], SwiGLU over [T, 14336], rotary embedding of the q rows [T x 32, 128] (FLOAT32 and
    FLOAT16). Inputs and outputs rotate over copies larger than twice the Infinity Cache, so every figure is an HBM
    rate; inside a layer the producer's output is usually still cache-resident and the operations run faster."""
    import ctypes as C

    from marmot_amd import DT_F16, DT_F32, capi

    lib, dev = hip.lib, hip.dev
    vp = C.c_void_p

    def rotating(nbytes, fill=None):
        stride = (nbytes + 255) & ~255
        copies = max(2, -(-2 * MALL_BYTES // stride) + 1)
        buf = hip.alloc(stride * copies)
        if fill is not None:
            for c in range(copies):
                buf.upload(fill, offset=c * stride)
        return buf, stride, copies

    def run(name, T, nbytes, step, copies):
        ms = time_steps_graph(hip, step, steps, warmup)
        emit({"config": "OPS", "workload": f"{name} T={T}", "us": round(ms * 1e3, 2),
              "GB/s": round(nbytes / ms / 1e6, 1), "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4),
              "copies": copies})

    for T in (16, 512):
        H, F, heads, D = 4096, 14336, 32, 128
        x = rng.standard_normal((T, H), dtype=np.float32)
        d_x, sx, cx = rotating(x.nbytes, x)
        d_r, _, _ = rotating(x.nbytes, x)
        d_y, sy, cy = rotating(x.nbytes)
        d_w = hip.to_device(np.ones(H, np.float32))
        run("rms_norm [T,4096] fp32 with residual and weight", T, 3 * x.nbytes + H * 4,
            lambda i: capi.check(lib.marmot_hip_rms_norm(dev, vp(d_x.ptr + (i % cx) * sx), vp(d_r.ptr + (i % cx) * sx),
                                                         vp(d_w.ptr), 0.0, 1e-5, T, H, vp(d_y.ptr + (i % cy) * sy))), cx)
        run("add [T,4096] fp32", T, 3 * x.nbytes,
            lambda i: capi.check(lib.marmot_hip_add(dev, vp(d_x.ptr + (i % cx) * sx), vp(d_r.ptr + (i % cx) * sx),
                                                    T * H, vp(d_y.ptr + (i % cy) * sy))), cx)
        pos = np.repeat(np.arange(T, dtype=np.int32) + 1000, heads)
        freqs, scale, hd = hip.rope_frequencies(D, head_dim=D, theta=500000.0)
        d_p, d_f = hip.to_device(pos), hip.to_device(freqs)
        arg = capi.Rope(d_p.ptr, capi.DT_I32, d_f.ptr, scale, hd, 0, 0, 0)
        for rope_type in (0, 1):
            arg.rope_type = rope_type
            run(f"rope q rows [T x 32,128] fp32 {'neox' if rope_type else 'norm'}", T, 2 * x.nbytes + pos.nbytes,
                lambda i: capi.check(lib.marmot_hip_rope(dev, vp(d_x.ptr + (i % cx) * sx), DT_F32, T * heads, D, D, D,
                                                         C.byref(arg), vp(d_y.ptr + (i % cy) * sy))), cx)
        arg.rope_type = 0
        run("rope q rows [T x 32,128] fp16 norm", T, x.nbytes + pos.nbytes,
            lambda i: capi.check(lib.marmot_hip_rope(dev, vp(d_x.ptr + (i % cx) * sx), DT_F16, T * heads, D, D, D,
                                                     C.byref(arg), vp(d_y.ptr + (i % cy) * sy))), cx)
        for b in (d_x, d_r, d_y, d_w, d_p, d_f):
            b.free()
        g = rng.standard_normal((T, F), dtype=np.float32)
        d_g, sg, cg = rotating(g.nbytes, g)
        d_u, _, _ = rotating(g.nbytes, g)
        d_o, so, co = rotating(g.nbytes)
        run("swiglu [T,14336] fp32", T, 3 * g.nbytes,
            lambda i: capi.check(lib.marmot_hip_glu(dev, 0, vp(d_g.ptr + (i % cg) * sg), vp(d_u.ptr + (i % cg) * sg),
                                                    T, F, F, F, F, vp(d_o.ptr + (i % co) * so))), cg)
        for b in (d_g, d_u, d_o):
            b.free()


def sweep_qkv(hip, rng, emit, steps: int, warmup: int):
    """Fused Q/K/V projection (three 4096 x 4096 weights of one scheme, one input) against three separate linears on
    the same buffers; weight copies rotate as in the other configurations."""
    from marmot_amd import DT_F32, capi, row_bytes

    M = K = 4096
    names = {capi.KIND_Q4_K: "Q4_K", capi.KIND_Q6_K: "Q6_K"}
    for kind in (capi.KIND_Q4_K, capi.KIND_Q6_K):
        rb = row_bytes(kind, K)
        stride = (M * rb + 255) & ~255
        copies = max(2, -(-2 * MALL_BYTES // (3 * stride)) + 1)
        d_w = []
        for _ in range(3):
            blocks = random_blocks(rng, kind, M, K)
            buf = hip.alloc(stride * copies)
            for c in range(copies):
                buf.upload(blocks, offset=c * stride)
            d_w.append(buf)
        for N in (1, 4, 16):
            d_x = hip.to_device(rng.standard_normal((N, K), dtype=np.float32))
            d_o = [hip.alloc(N * M * 4) for _ in range(3)]
            fused = time_steps_graph(hip, lambda i: hip.linear_qkv_d(kind, *d_w, d_x, DT_F32, N, K, M, *d_o,
                                                                     weight_offset=(i % copies) * stride),
                                     steps, warmup, chunk=50)
            route = hip.last_route()

            def three(i):
                for w, o in zip(d_w, d_o):
                    hip.linear_d(kind, w, d_x, DT_F32, N, K, M, o, DT_F32, weight_offset=(i % copies) * stride)

            separate = time_steps_graph(hip, three, steps, warmup, chunk=50)
            nbytes = 3 * M * rb + N * K * 4 + 3 * N * M * 4
            emit({"config": "QKV", "workload": f"{names[kind]} q,k,v 3 x {M}x{K} N={N}", "route": route,
                  "us": round(fused * 1e3, 2), "us_three_linears": round(separate * 1e3, 2),
                  "GB/s": round(nbytes / fused / 1e6, 1),
                  "frac_of_hbm_peak": round(nbytes / fused / 1e6 / HBM_PEAK_GBPS, 4),
                  "tokens_per_s": round(N / fused * 1e3)})
            for b in [d_x] + d_o:
                b.free()
        for b in d_w:
            b.free()


def sweep_layer_stack(hip, rng, emit, steps: int, N: int = 16, config: str = "C4"):
    """C4: the seven linears of one layer at 16 tokens; 4 copies of the 139 MB of weights rotate. C4P: the same layer
    at 512 tokens of a prompt (fp32 activations: the tiled int8 GEMMs)."""
    from marmot_amd import DT_F32, capi, row_bytes

    specs = [(capi.KIND_Q4_K, 4096, 4096), (capi.KIND_Q4_K, 1024, 4096), (capi.KIND_Q6_K, 1024, 4096),
             (capi.KIND_Q4_K, 4096, 4096), (capi.KIND_Q4_K, 14336, 4096), (capi.KIND_Q4_K, 14336, 4096),
             (capi.KIND_Q6_K, 4096, 14336)]
    copies = 4
    layers = []
    total = 0
    for kind, M, K in specs:
        rb = row_bytes(kind, K)
        stride = (M * rb + 255) & ~255
        blocks = random_blocks(rng, kind, M, K)
        d_w = hip.alloc(stride * copies)
        for c in range(copies):
            d_w.upload(blocks, offset=c * stride)
        layers.append((kind, M, K, stride, d_w, hip.to_device(rng.standard_normal((N, K), dtype=np.float32)),
                       hip.alloc(N * M * 4)))
        total += algorithmic_bytes(rb, M, K, N)

    def layer_step(i):
        for kind, M, K, stride, d_w, d_x, d_out in layers:
            hip.linear_d(kind, d_w, d_x, DT_F32, N, K, M, d_out, DT_F32, weight_offset=(i % copies) * stride)

    ms = time_steps_graph(hip, layer_step, max(50, steps // 10), 10, chunk=50)

    # The same seven linears as a layer calls them: q, k, v read one input and gate, up read one input, so the
    # activations are packed once per distinct input (4 packs instead of 7) and the linears take the packed rows.
    groups = [(0, (0, 1, 2)), (3, (3,)), (4, (4, 5)), (6, (6,))]  # (linear whose input is used, linears sharing it)
    packed = {}
    for src, _ in groups:
        kind, M, K = specs[src]
        packed[src] = hip.alloc(hip.packed_activation_bytes(kind, N, K))

    def layer_step_shared(i):
        for src, members in groups:
            kind, M, K = specs[src]
            hip.pack_activations_d(kind, layers[src][5], DT_F32, N, K, packed[src])
            for m in members:
                kind_m, M_m, K_m, stride, d_w, _, d_out = layers[m]
                hip.linear_prepacked_d(kind_m, d_w, packed[src], N, K_m, M_m, d_out,
                                       weight_offset=(i % copies) * stride)

    ms_shared = time_steps_graph(hip, layer_step_shared, max(50, steps // 10), 10, chunk=50)

    # The same again with the linears that share an input as the branches of one section (q | k | v, gate | up): they
    # do not depend on each other, so the tail of one, the launch gap and the start-up of the next overlap.
    def layer_step_branches(i):
        for src, members in groups:
            kind, M, K = specs[src]
            hip.pack_activations_d(kind, layers[src][5], DT_F32, N, K, packed[src])

            def one(m):
                kind_m, M_m, K_m, stride, d_w, _, d_out = layers[m]
                return lambda: hip.linear_prepacked_d(kind_m, d_w, packed[src], N, K_m, M_m, d_out,
                                                      weight_offset=(i % copies) * stride)

            if len(members) > 1:
                hip.branches(*[one(m) for m in members])
            else:
                one(members[0])()

    ms_branches = time_steps_graph(hip, layer_step_branches, max(50, steps // 10), 10, chunk=50)
    ops = sum(2.0 * N * M * K for _, M, K in specs)
    emit({"config": config, "workload": f"7 linears of a Llama-3-8B layer (q,k,o,gate,up Q4_K; v,down Q6_K), N={N}",
          "us": round(ms * 1e3, 2), "GB/s": round(total / ms / 1e6, 1),
          "frac_of_hbm_peak": round(total / ms / 1e6 / HBM_PEAK_GBPS, 4), "tokens_per_s": round(N / ms * 1e3),
          "TOP/s": round(ops / ms / 1e9, 1), "algorithmic_bytes": total,
          "us_shared_inputs": round(ms_shared * 1e3, 2),
          "us_shared_inputs_branches": round(ms_branches * 1e3, 2),
          "branches": "as shared_inputs, with q | k | v and gate | up as branches of one section (separate streams)",
          "shared_inputs": "q/k/v and gate/up take activations packed once per distinct input (4 packs, 7 linears)"})
    for b in packed.values():
        b.free()
    for *_, d_w, d_x, d_out in layers:
        for b in (d_w, d_x, d_out):
            b.free()


def sweep_branches(hip, rng, emit, steps: int, N: int = 16):
    """Independent linears of one layer (q | k | v and gate | up at 16 tokens, activations packed beforehand) four ways:
    one after the other on one stream, as the branches of one section (fork + join per step), both eagerly (HIP events
    around `steps` steps), and as an upper bound every linear on a device object of its own with nothing between them
    (one graph of 200 steps each, launched together, host clock). The weights stay warm (one copy each): the figures
    are for comparing the four, not against the rotating-weight rows of the other configurations."""
    from marmot_amd import DT_F32, HipBackend, capi

    groups = {
        "q | k | v": [(capi.KIND_Q4_K, 4096, 4096), (capi.KIND_Q4_K, 1024, 4096), (capi.KIND_Q6_K, 1024, 4096)],
        "gate | up": [(capi.KIND_Q4_K, 14336, 4096), (capi.KIND_Q4_K, 14336, 4096)],
    }

    def linear_on(backend, kind, M, K):
        bufs = [backend.to_device(random_blocks(rng, kind, M, K)),
                backend.to_device(rng.standard_normal((N, K), dtype=np.float32)),
                backend.alloc(backend.packed_activation_bytes(kind, N, K)), backend.alloc(N * M * 4)]
        backend.pack_activations_d(kind, bufs[1], DT_F32, N, K, bufs[2])
        return (lambda: backend.linear_prepacked_d(kind, bufs[0], bufs[2], N, K, M, bufs[3])), bufs

    for name, specs in groups.items():
        made = [linear_on(hip, *spec) for spec in specs]
        fns = [fn for fn, _ in made]
        row_ms, _ = time_steps(hip, lambda i: [fn() for fn in fns], steps, 50)
        section_ms, _ = time_steps(hip, lambda i: hip.branches(*fns), steps, 50)
        graph_row = time_steps_graph(hip, lambda i: [fn() for fn in fns], steps, 10, chunk=50)
        graph_section = time_steps_graph(hip, lambda i: hip.branches(*fns), steps, 10, chunk=50)
        for _, bufs in made:
            for b in bufs:
                b.free()
        # upper bound: no dependencies at all between the linears
        others = []
        for spec in specs:
            backend = HipBackend(0)
            fn, bufs = linear_on(backend, *spec)
            fn()
            backend.synchronize()
            others.append((backend, backend.graph_capture(lambda fn=fn: [fn() for _ in range(200)]), bufs))

        def together(reps):
            for backend, g, _ in others:
                backend.graph_launch(g)
            for backend, _, _ in others:
                backend.synchronize()
            t0 = time.perf_counter()
            for _ in range(reps):
                for backend, g, _ in others:
                    backend.graph_launch(g)
            for backend, _, _ in others:
                backend.synchronize()
            return (time.perf_counter() - t0) / reps / 200 * 1e3

        together(5)
        free_ms = together(20)
        for backend, g, bufs in others:
            backend.graph_destroy(g)
            for b in bufs:
                b.free()
            backend.close()
        emit({"config": "BRANCH", "workload": f"{name} of a Llama-3-8B layer, N={N}, packed activations, warm weights",
              "us_in_a_row_eager": round(row_ms * 1e3, 2), "us_branch_section_eager": round(section_ms * 1e3, 2),
              "us_in_a_row_graph": round(graph_row * 1e3, 2), "us_branch_section_graph": round(graph_section * 1e3, 2),
              "us_unsynchronized_streams": round(free_ms * 1e3, 2),
              "note": "unsynchronized streams: one device object and one 200-step graph per linear, launched together "
                      "(an upper bound: nothing orders the linears)"})


def sweep_attention(hip, rng, emit, steps: int):
    """Paged attention of a Llama-3-8B layer (32 query heads over 8 key / value heads of 128, block size 16, fp16
    cache, fp32 activations): a decode step of 16 sequences with 4096 positions of history each (one new token per
    sequence), and a prompt of 512 tokens of one sequence. The figure is the cache bytes every (token, kv head) must
    read, once per kv head, over the time of the whole op (cache write + attention)."""
    import ctypes as C

    hq, hkv, d, bs = 32, 8, 128, 16

    def run(name, seqs, fp8=False):
        need = [-(-(h + n) // bs) for h, n in seqs]
        blocks = sum(need)
        table = np.full((len(seqs), max(need)), 0xFFFFFFFF, dtype=np.uint32)
        meta, nxt = [], 0
        for s, (h, n) in enumerate(seqs):
            table[s, :need[s]] = np.arange(nxt, nxt + need[s], dtype=np.uint32)
            nxt += need[s]
            meta += [(s, p, int(table[s, p // bs]) * bs + p % bs, 0) for p in range(h, h + n)]
        meta = np.array(meta, dtype=np.uint32)
        T = len(meta)
        arrays = {
            "token_meta": meta, "block_table": table,
            "q": rng.standard_normal((T, hq, d), dtype=np.float32),
            "k_new": rng.standard_normal((T, hkv, d), dtype=np.float32),
            "v_new": rng.standard_normal((T, hkv, d), dtype=np.float32),
            "kv_k": rng.standard_normal((blocks, 1, hkv, bs, d), dtype=np.float32).astype(np.float16),
            "kv_v": rng.standard_normal((blocks, 1, hkv, bs, d), dtype=np.float32).astype(np.float16),
            "out": np.zeros((T, hq, d), dtype=np.float32),
        }
        if fp8:  # finite e4m3 codes of either sign; scales under which the new rows never raise a block's maximum,
            # the steady state of a decode loop (no re-encoding of the rows already there)
            for n in ("kv_k", "kv_v"):
                arrays[n] = (rng.integers(0, 0x78, arrays[n].shape) | (rng.integers(0, 2, arrays[n].shape) << 7)).astype(np.uint8)
            arrays["k_scale"] = np.full((blocks, 1, hkv), 0.05, dtype=np.float32)
            arrays["v_scale"] = np.full((blocks, 1, hkv), 0.05, dtype=np.float32)
        dev = {k: hip.to_device(v) for k, v in arrays.items()}
        ptr_of = {id(v): dev[k].ptr for k, v in arrays.items()}
        a = arrays
        p = hip.paged_attention_args(lambda x: ptr_of[id(x)], a["token_meta"], a["q"], a["k_new"], a["v_new"], a["kv_k"],
                                     a["kv_v"], a["block_table"], a["out"], 0, float(1.0 / np.sqrt(d)),
                                     kv_k_scale=a.get("k_scale"), kv_v_scale=a.get("v_scale"))

        def step(i):
            rc = hip.lib.marmot_hip_paged_attention(hip.dev, C.byref(p), 0)
            if rc != 0:
                raise RuntimeError(f"marmot_hip_paged_attention -> {rc}")

        ms = time_steps_graph(hip, step, max(20, steps // 20), 5, chunk=20)
        esz = 1 if fp8 else 2
        read = sum(int(pos) + 1 for _, pos, _, _ in meta) * hkv * d * 2 * esz  # K and V rows, once per kv head
        total = read + T * (hq * 2 + hkv * 2) * d * 4 + T * hkv * d * 2 * esz
        flops = 4.0 * sum(int(pos) + 1 for _, pos, _, _ in meta) * hq * d
        emit({"config": "ATTN", "workload": name, "us": round(ms * 1e3, 2), "GB/s": round(total / ms / 1e6, 1),
              "frac_of_hbm_peak": round(total / ms / 1e6 / HBM_PEAK_GBPS, 4), "TFLOP/s": round(flops / ms / 1e9, 2),
              "tokens_per_s": round(T / ms * 1e3), "algorithmic_bytes": total})
        for b in dev.values():
            b.free()

    run("paged attention, decode: 16 sequences x 4096 positions, 32/8 heads of 128, fp16 cache", [(4095, 1)] * 16)
    run("paged attention, decode: 16 sequences x 512 positions", [(511, 1)] * 16)
    run("paged attention, prompt: 512 tokens of one sequence", [(0, 512)])
    run("paged attention, decode: 16 sequences x 4096 positions, FLOAT8_E4M3 cache", [(4095, 1)] * 16, fp8=True)


def sweep_whole_layer(hip, rng, emit, steps: int, T: int = 16, context: int = 4096):
    """One decode step of a whole Llama-3-8B layer for 16 sequences with 4096 positions of history each, every op on
    the device: rms_norm (leaves its rows packed) -> q, k (Q4_K), v (Q6_K) -> rotary embedding of q and k -> paged
    attention (fp16 cache) -> pack -> o (Q4_K) -> add -> rms_norm (packed) -> gate, up (Q4_K) -> swiglu (packed) ->
    down (Q6_K) -> add. Four copies of the 139 MB of weights rotate; the 268 MB cache is one copy."""
    import ctypes as C

    from marmot_amd import DT_F32, capi, row_bytes

    lib, dev, vp, chk = hip.lib, hip.dev, C.c_void_p, capi.check
    H, F, hq, hkv, hd, bs = 4096, 14336, 32, 8, 128, 16
    Q4, Q6 = capi.KIND_Q4_K, capi.KIND_Q6_K
    specs = {"q": (Q4, hq * hd, H), "k": (Q4, hkv * hd, H), "v": (Q6, hkv * hd, H), "o": (Q4, H, hq * hd),
             "g": (Q4, F, H), "u": (Q4, F, H), "d": (Q6, H, F)}
    copies, weights, wbytes = 4, {}, 0
    for name, (kind, M, K) in specs.items():
        stride = (M * row_bytes(kind, K) + 255) & ~255
        blocks = random_blocks(rng, kind, M, K)
        buf = hip.alloc(stride * copies)
        for c in range(copies):
            buf.upload(blocks, offset=c * stride)
        weights[name] = (buf, stride)
        wbytes += M * row_bytes(kind, K)
    f32 = lambda *shape: hip.to_device(rng.standard_normal(shape, dtype=np.float32))
    x, wn1, wn2 = f32(T, H), hip.to_device(np.ones(H, np.float32)), hip.to_device(np.ones(H, np.float32))
    h, q, k, v, att, o, x1, h2, g, u, d, y = (hip.alloc(T * n * 4) for n in
                                              (H, hq * hd, hkv * hd, hkv * hd, hq * hd, H, H, H, F, F, H, H))
    packs = {n: hip.alloc(hip.packed_activation_bytes(Q4, T, K)) for n, K in (("h", H), ("att", hq * hd), ("h2", H), ("a", F))}
    blocks_per_seq = -(-context // bs)
    table = np.arange(T * blocks_per_seq, dtype=np.uint32).reshape(T, blocks_per_seq)
    meta = np.array([[s_, context - 1, int(table[s_, (context - 1) // bs]) * bs + (context - 1) % bs, 0] for s_ in range(T)],
                    dtype=np.uint32)
    cache_shape = (T * blocks_per_seq, 1, hkv, bs, hd)
    arrays = {"token_meta": meta, "block_table": table, "kv_k": np.zeros(cache_shape, np.float16),
              "kv_v": np.zeros(cache_shape, np.float16)}
    arrays["kv_k"][...] = rng.standard_normal(cache_shape, dtype=np.float32)
    arrays["kv_v"][...] = rng.standard_normal(cache_shape, dtype=np.float32)
    devs = {n: hip.to_device(a) for n, a in arrays.items()}
    shaped = {"q": np.empty((T, hq, hd), np.float32), "k_new": np.empty((T, hkv, hd), np.float32),
              "v_new": np.empty((T, hkv, hd), np.float32), "out": np.empty((T, hq, hd), np.float32)}
    ptr_of = {id(arrays[n]): devs[n].ptr for n in arrays}
    ptr_of.update({id(shaped["q"]): q.ptr, id(shaped["k_new"]): k.ptr, id(shaped["v_new"]): v.ptr, id(shaped["out"]): att.ptr})
    pa = hip.paged_attention_args(lambda a: ptr_of[id(a)], meta, shaped["q"], shaped["k_new"], shaped["v_new"],
                                  arrays["kv_k"], arrays["kv_v"], table, shaped["out"], 0, float(1.0 / np.sqrt(hd)))
    freqs, scale, rhd = hip.rope_frequencies(hd, head_dim=hd, theta=500000.0)
    d_f = hip.to_device(freqs)
    pos_q = hip.to_device(np.repeat(meta[:, 1].astype(np.int32), hq))
    pos_k = hip.to_device(np.repeat(meta[:, 1].astype(np.int32), hkv))
    rope_q = capi.Rope(pos_q.ptr, capi.DT_I32, d_f.ptr, scale, rhd, 0, 0, 0)
    rope_k = capi.Rope(pos_k.ptr, capi.DT_I32, d_f.ptr, scale, rhd, 0, 0, 0)

    def linear(name, packed, out, i):
        kind, M, K = specs[name]
        buf, stride = weights[name]
        chk(lib.marmot_hip_matmul_prepacked(dev, kind, vp(buf.ptr + (i % copies) * stride), vp(packed.ptr), T, K, M, None,
                                            DT_F32, vp(out.ptr), DT_F32))

    def step(i):
        chk(lib.marmot_hip_rms_norm_pack(dev, vp(x.ptr), None, vp(wn1.ptr), 0.0, 1e-5, T, H, Q4, vp(h.ptr), vp(packs["h"].ptr)))
        linear("q", packs["h"], q, i)
        linear("k", packs["h"], k, i)
        linear("v", packs["h"], v, i)
        chk(lib.marmot_hip_rope(dev, vp(q.ptr), DT_F32, T * hq, hd, hd, hd, C.byref(rope_q), vp(q.ptr)))
        chk(lib.marmot_hip_rope(dev, vp(k.ptr), DT_F32, T * hkv, hd, hd, hd, C.byref(rope_k), vp(k.ptr)))
        chk(lib.marmot_hip_paged_attention(dev, C.byref(pa), 0))
        chk(lib.marmot_hip_pack_activations(dev, Q4, vp(att.ptr), DT_F32, T, hq * hd, vp(packs["att"].ptr)))
        linear("o", packs["att"], o, i)
        chk(lib.marmot_hip_add(dev, vp(x.ptr), vp(o.ptr), T * H, vp(x1.ptr)))
        chk(lib.marmot_hip_rms_norm_pack(dev, vp(x1.ptr), None, vp(wn2.ptr), 0.0, 1e-5, T, H, Q4, vp(h2.ptr), vp(packs["h2"].ptr)))
        linear("g", packs["h2"], g, i)
        linear("u", packs["h2"], u, i)
        chk(lib.marmot_hip_swiglu_pack(dev, vp(g.ptr), vp(u.ptr), T, F, Q6, vp(packs["a"].ptr)))
        linear("d", packs["a"], d, i)
        chk(lib.marmot_hip_add(dev, vp(x1.ptr), vp(d.ptr), T * H, vp(y.ptr)))

    ms = time_steps_graph(hip, step, max(20, steps // 20), 5, chunk=10)
    cache_read = T * context * hkv * hd * 2 * 2
    emit({"config": "LAYER", "workload": f"whole Llama-3-8B decoder layer, decode step of {T} sequences x {context} positions "
          "(norms, q/k/v/o/gate/up/down linears, rotary embedding, paged attention with fp16 cache, SwiGLU, residual adds)",
          "us": round(ms * 1e3, 2), "GB/s": round((wbytes + cache_read) / ms / 1e6, 1),
          "frac_of_hbm_peak": round((wbytes + cache_read) / ms / 1e6 / HBM_PEAK_GBPS, 4),
          "tokens_per_s_per_layer": round(T / ms * 1e3), "weight_bytes": wbytes, "cache_bytes_read": cache_read,
          "launches_per_step": 16})


def sweep_moe(hip, rng, emit, steps: int):
    """C5: 128 experts, top-8, hidden 2048, expert FFN 768, 64 tokens, all Q4_K; 2 copies of the 340 MB rotate."""
    from marmot_amd import capi, row_bytes

    E, k, H, F, T = 128, 8, 2048, 768, 64
    kind = capi.KIND_Q4_K
    gu_bytes = E * F * row_bytes(kind, H)
    dn_bytes = E * H * row_bytes(kind, F)
    d_g, d_u, d_d = hip.alloc(2 * gu_bytes), hip.alloc(2 * gu_bytes), hip.alloc(2 * dn_bytes)
    for buf, rows, cols, nb in ((d_g, E * F, H, gu_bytes), (d_u, E * F, H, gu_bytes), (d_d, E * H, F, dn_bytes)):
        blocks = random_blocks(rng, kind, rows, cols)
        buf.upload(blocks, offset=0)
        buf.upload(blocks, offset=nb)
    logits = rng.standard_normal((T, E), dtype=np.float32)
    vals, ids = hip.topk(logits, k)
    d_h = hip.to_device(rng.standard_normal((T, H), dtype=np.float32))
    d_ids, d_wts = hip.to_device(ids), hip.to_device(hip.softmax_rows(vals))
    d_out = hip.alloc(T * H * 4)
    active = len(np.unique(ids))

    def moe_step(i):
        c = i % 2
        hip.moe_experts_d(d_h, T, H, F, E, k, kind, kind, d_g, d_u, d_d, d_ids, d_wts, d_out,
                          gate_offset=c * gu_bytes, up_offset=c * gu_bytes, down_offset=c * dn_bytes)

    ms = time_steps_graph(hip, moe_step, max(50, steps // 10), 10, chunk=50)
    nbytes = active * (2 * F * row_bytes(kind, H) + H * row_bytes(kind, F)) + 2 * T * H * 4
    emit({"config": "C5", "workload": f"MoE experts E={E} top-{k} H={H} F={F} T={T} Q4_K ({active} active experts)",
          "us": round(ms * 1e3, 2), "GB/s": round(nbytes / ms / 1e6, 1),
          "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4), "tokens_per_s": round(T / ms * 1e3),
          "algorithmic_bytes": nbytes})


# Marks of the resident-share decode kernel in the timeline build (make -C marmot_amd/csrc TIMELINE=1): slot -> meaning
TIMELINE_LOADER = {0: "start", 2: "first window requested", 3: "barrier passed", 4: "first instruction landed",
                   8: "a quarter landed", 9: "half landed", 10: "three quarters landed", 6: "all requested",
                   7: "all landed"}
TIMELINE_CONSUMER = {0: "start", 1: "barrier passed", 2: "own activations landed", 3: "own activations in registers",
                     4: "own part quantized", 5: "all parts quantized", 6: "task loop starts",
                     7: "first task's bytes there", 8: "first task's products done", 9: "last task's bytes there",
                     10: "last task done", 11: "leaves"}


def timeline_report(shape: str, steps: int, warmup: int):
    """Cycle-counter timeline of the Q4_K decode kernel for one activation row. Needs the timeline build of the
    library (make -C marmot_amd/csrc TIMELINE=1; MARMOT_HIP_LIBRARY=marmot_amd/lib/libmarmot_hip_timeline.so): every
    wavefront keeps up to 12 cycle-counter marks in registers and writes them, with the 100 MHz device clock at its
    first mark and at its exit, into the attached buffer when it leaves. Prints, per mark, the distribution over the
    wavefronts of one launch (microseconds since the workgroup's first wavefront started)."""
    from marmot_amd import DT_F32, HipBackend, capi, row_bytes
    from marmot_amd.capi import check

    M, K = (int(v) for v in shape.split("x"))
    kind = capi.KIND_Q4_K
    hip = HipBackend(0)
    rb = row_bytes(kind, K)
    stride = (M * rb + 255) & ~255
    copies = max(2, -(-2 * MALL_BYTES // stride) + 1)
    rng = np.random.Generator(np.random.PCG64(10))
    blocks = random_blocks(rng, kind, M, K)
    d_w = hip.alloc(stride * copies)
    for c in range(copies):
        d_w.upload(blocks, offset=c * stride)
    d_x = hip.to_device(rng.standard_normal((1, K), dtype=np.float32))
    d_out = hip.alloc(M * 4)
    slots, waves_per_wg = 16, 16
    words = hip.caps()["num_compute_units"] * waves_per_wg * slots
    d_tl = hip.alloc(words * 8)

    def step(i):
        hip.linear_d(kind, d_w, d_x, DT_F32, 1, K, M, d_out, DT_F32, weight_offset=(i % copies) * stride)

    check(hip.lib.marmot_hip_timeline_attach(hip.dev, None, 0))
    ms = time_steps_graph(hip, step, steps, warmup)
    route = hip.last_route()
    print(f"{M}x{K}: {ms * 1e3:.3f} us per launch with the marks switched off (route {route})")
    check(hip.lib.marmot_hip_timeline_attach(hip.dev, ctypes.c_void_p(d_tl.ptr), words * 8))
    ms_on = time_steps_graph(hip, step, steps, warmup)
    print(f"{M}x{K}: {ms_on * 1e3:.3f} us per launch with the marks written")

    def stats(name, a):
        a = np.asarray(a, dtype=np.float64)
        a = a[~np.isnan(a)]
        if a.size:
            print(f"  {name:44s} min {a.min():6.2f} p10 {np.percentile(a, 10):6.2f} med {np.median(a):6.2f} "
                  f"p90 {np.percentile(a, 90):6.2f} max {a.max():6.2f}")

    for rep in range(2):
        hip.lib.marmot_hip_memset(hip.dev, ctypes.c_void_p(d_tl.ptr), 0, words * 8)
        g = hip.graph_capture(lambda: [step(7 + j) for j in range(200)])  # the buffer keeps the last launch
        hip.graph_launch(g)
        hip.synchronize()
        hip.graph_destroy(g)
        t = d_tl.download(np.uint64, (words // slots, slots)).astype(np.int64)
        t = t[t[:, 12] != 0]
        nw = t.shape[0]
        # slots 12 / 14: cycle counter at the first mark / at the flush; 13 / 15: the 100 MHz clock at the same points
        dc = (t[:, 14] - t[:, 12]).astype(np.float64)
        dr = (t[:, 15] - t[:, 13]).astype(np.float64) * 10.0
        rate = np.median(dc[dr > 0] / dr[dr > 0])  # cycle-counter ticks per nanosecond
        print(f" launch {rep}: {nw} wavefronts; cycle counter at {rate * 1e3:.0f} MHz; first start to last exit "
              f"{(t[:, 15].max() - t[:, 13].min()) * 0.01:.2f} us (100 MHz clock)")
        wg = np.arange(nw) // waves_per_wg
        wv = np.arange(nw) % waves_per_wg
        nwg = int(wg.max()) + 1
        base = np.array([t[wg == i, 12].min() for i in range(nwg)])[wg]
        rel = (t - base[:, None]) / rate / 1e3
        rel[t == 0] = np.nan
        dev0 = t[:, 13].min()
        stats("workgroup start after the first one", (np.array([t[wg == i, 13].min() for i in range(nwg)]) - dev0) * 0.01)
        stats("workgroup end after the first start", (np.array([t[wg == i, 15].max() for i in range(nwg)]) - dev0) * 0.01)
        loaders = wv < 4
        for slot, label in TIMELINE_LOADER.items():
            stats("loader: " + label, rel[loaders, slot])
        for slot, label in TIMELINE_CONSUMER.items():
            stats("consumer: " + label, rel[~loaders, slot])
    hip.close()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="time budget of the CPU baseline leg")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg (profiling runs)")
    ap.add_argument("--batch", type=int, default=1, help="activation rows N (1, 4 or 8 are the decode configs)")
    ap.add_argument("--shape", default="4096x14336", help="weight shape MxK (marmot naming)")
    ap.add_argument("--kind", default="q4_k", choices=["q4_k", "q6_k", "q8_0", "q4_0", "q4_1", "q5_0", "q5_1", "q8_1", "q2_k",
                                                       "q3_k", "q5_k"])
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill GEMM leg")
    ap.add_argument("--prefill-tokens", type=int, default=512)
    ap.add_argument("--sweep", action="store_true",
                    help="measure every benchmark configuration (C1..C5, QKV, LOGITS) instead, one JSON line each (documentation runs)")
    ap.add_argument("--configs", default="C1,C2,C3,C4,C5", help="with --sweep: the configurations to run")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                    help="run only a plain device copy of this many MiB (known traffic, for profiler counters)")
    ap.add_argument("--calibrate-read", type=int, default=0, metavar="MIB",
                    help="run only the read-only streaming kernel over this many MiB per launch, rotating over "
                         "copies beyond the Infinity Cache, and print its bandwidth")
    ap.add_argument("--timeline", default="", metavar="MxK",
                    help="print the cycle-counter timeline of the Q4_K decode kernel for this weight shape "
                         "(needs the timeline build of the library)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus must be 1 (no multi-GPU path exists in the hot path)",
              file=sys.stderr)
        sys.exit(2)

    from marmot_amd import DT_F32, HipBackend, row_bytes
    from marmot_amd import capi

    if args.calibrate_copy:
        hip = HipBackend(0)
        n = args.calibrate_copy << 20
        src, dst = hip.alloc(n), hip.alloc(n)
        hip.lib.marmot_hip_memset(hip.dev, src.ptr, 1, n)
        ms, _ = time_steps(hip, lambda i: hip.copy_d(dst, src, n), 20, 3)
        print(json.dumps({"calibration": "plain 16-byte copy kernel", "bytes_read": n, "bytes_written": n,
                          "launches": 23, "ms_per_launch": round(ms, 5),
                          "gbps_read_plus_write": round(2 * n / (ms * 1e-3) / 1e9, 1)}))
        hip.close()
        return

    if args.timeline:
        timeline_report(args.timeline, min(args.steps, 2000), min(args.warmup, 200))
        return

    if args.calibrate_read:
        hip = HipBackend(0)
        print(json.dumps(read_calibration(hip, args.calibrate_read << 20, 400, 40)))
        hip.close()
        return

    if args.sweep:
        hip = HipBackend(0)
        sweep(hip, args.steps, args.warmup, tuple(args.configs.split(",")))
        hip.close()
        return

    kind = getattr(capi, "KIND_" + args.kind.upper())
    M, K = (int(v) for v in args.shape.split("x"))
    N = args.batch
    rb = row_bytes(kind, K)
    wbytes = M * rb
    nbytes = algorithmic_bytes(rb, M, K, N)

    hip = HipBackend(0)
    caps = hip.caps()
    rng = np.random.Generator(np.random.PCG64(10))
    blocks = random_blocks(rng, kind, M, K)
    x = np.random.Generator(np.random.PCG64(20)).standard_normal((N, K), dtype=np.float32)

    # distinct weight copies, 256-byte aligned, together larger than twice the Infinity Cache
    stride = (wbytes + 255) & ~255
    copies = max(2, -(-2 * MALL_BYTES // stride) + 1)
    d_w = hip.alloc(stride * copies)
    for c in range(copies):
        d_w.upload(blocks, offset=c * stride)
    d_x = hip.to_device(x)
    d_out = hip.alloc(N * M * 4)
    d_packed = hip.alloc(hip.packed_activation_bytes(kind, N, K))

    # ---- whole op: activation quantization + matvec, weights rotating
    def step(i):
        hip.linear_d(kind, d_w, d_x, DT_F32, N, K, M, d_out, DT_F32, weight_offset=(i % copies) * stride)

    ms_op_eager, ms_op_host = time_steps(hip, step, args.steps, args.warmup)
    ms_op = time_steps_graph(hip, step, args.steps, args.warmup)
    op_timing = dict(LAST_TIMING)
    route = hip.last_route()
    got = d_out.download(np.float32, (N, M))

    # ---- dominant kernel alone: matvec on pre-packed activations, weights rotating
    hip.pack_activations_d(kind, d_x, DT_F32, N, K, d_packed)

    def kstep(i):
        hip.linear_prepacked_d(kind, d_w, d_packed, N, K, M, d_out, weight_offset=(i % copies) * stride)

    ms_k_eager, _ = time_steps(hip, kstep, args.steps, args.warmup)
    ms_k = time_steps_graph(hip, kstep, args.steps, args.warmup)

    # ---- same kernel with the weights resident in the Infinity Cache (one copy), reported separately
    def kstep_hot(i):
        hip.linear_prepacked_d(kind, d_w, d_packed, N, K, M, d_out, weight_offset=0)

    ms_hot = time_steps_graph(hip, kstep_hot, args.steps, args.warmup)

    value = nbytes / (ms_op * 1e-3) / 1e9
    fused = route.endswith("_fused")  # the whole op is then one kernel: that kernel is the dominant one
    ms_dom, ms_dom_eager = (ms_op, ms_op_eager) if fused else (ms_k, ms_k_eager)
    achieved = nbytes / (ms_dom * 1e-3) / 1e9
    result = {
        "metric": METRIC,
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_op, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {
            "workload": f"{args.kind.upper()} decode matvec, weight {M}x{K} (marmot MxK), N={N} fp32 activations "
                        f"quantized to {'Q8_K' if kind in (9, 11) else 'Q8_0'} on device, fp32 output",
            "weight_copies": copies,
            "weight_bytes": wbytes,
            "algorithmic_bytes_per_step": nbytes,
            "route": route,
            "device": caps["name"] or "AMD Instinct MI355X",
            "weights": "random block bytes with small finite fp16 super-block scales (timing only; parity tests use "
                       "N(0, 0.02) weights through the quantizer)",
            "arch": caps["arch"],
            "compute_units": caps["num_compute_units"],
        },
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "tokens_per_s": round(N / (ms_op * 1e-3), 1),
        "submission": "HIP graph replay of the timed steps (graphs of up to 500 steps); ms_per_step is the median of "
                      "`repeats` timed repeats of exactly `steps` steps each (time-stamp kernels recorded inside the graphs), "
                      "after untimed replays until 50 ms of GPU time have passed",
        "repeats": op_timing["repeats"],
        "ms_per_step_min": round(op_timing["ms_per_step_min"], 6),
        "ms_per_step_max": round(op_timing["ms_per_step_max"], 6),
        "eager_ms_per_step": round(ms_op_eager, 6),
        "eager_ms_per_step_host_clock": round(ms_op_host, 6),
        "roofline": {
            "kernel": route,
            "bound": "hbm",
            "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            # HBM bytes per launch from rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled by a plain copy kernel
            # (profiles/matvec_q4_k_4096x14336_n1.md); only valid for the default workload
            "traffic": (TRAFFIC_FUSED if fused else TRAFFIC_PREPACKED)
            if (args.kind, args.shape, N) == ("q4_k", "4096x14336", 1) else None,
            "avg_launch_us": round(ms_dom * 1e3, 3),
            "avg_launch_us_eager": round(ms_dom_eager * 1e3, 3),
            # the matvec on activations quantized beforehand (the kernel N > 4 uses), and with the weights cache-resident
            "prepacked_kernel_us": round(ms_k * 1e3, 3),
            "prepacked_kernel_gbps": round(nbytes / (ms_k * 1e-3) / 1e9, 2),
            "cache_resident_gbps": round(nbytes / (ms_hot * 1e-3) / 1e9, 2),
        },
    }
    # ---- what a kernel that only reads gets on this box: one dependent launch of the weight size, and a large one
    small = read_calibration(hip, wbytes, max(100, args.steps // 4), max(20, args.steps // 20))
    large = read_calibration(hip, 512 << 20, 20, 3)
    result["roofline"]["measured_read_gbps"] = {
        "same_size_dependent_launch": small["gbps"], "same_size_us": small["us_per_launch"],
        "launch_of_512_MiB": large["gbps"],
        "method": "read-only 16-byte streaming kernel of the library (marmot_hip_read_probe), HIP-graph replay, "
                  "copies rotating beyond the Infinity Cache",
    }
    result["roofline"]["frac_of_measured_read"] = round(achieved / small["gbps"], 4)
    # ---- second half of the metric: Q4_K prefill GEMM, weight 4096 x 4096, fp16 activations, fp32 out
    if (args.kind, args.shape, N) == ("q4_k", "4096x14336", 1) and not args.no_prefill:
        # As many steps as it takes for the clocks to settle under the matrix-core load, whatever --steps says (that
        # flag sizes the headline leg): repeats of 100 steps read 30.9 us, of 1000 steps 29.4 us on the same box.
        result["prefill_gemm"] = prefill_gemm(hip, args.prefill_tokens, max(1000, args.steps // 2),
                                              max(20, args.steps // 20))
        result["prefill_int8"] = prefill_int8(hip, args.prefill_tokens, max(1000, args.steps // 2),
                                              max(20, args.steps // 20))
    if not args.no_cpu:
        cb, err = cpu_baseline(kind, blocks, x, M, K, nbytes, got, args.cpu_seconds)
        result["cpu_baseline"] = cb
        result["parity_max_rel_err_vs_cpu"] = float(f"{err:.3e}")
    else:
        result["cpu_baseline"] = None
    hip.close()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
