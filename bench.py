#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

Headline workload (``config.workload``): BASELINE.json config 2 -- decode-shaped W4A16 GEMMs, the four Llama-3-8B
projection shapes (K,N) x M in {1,4,16}, group 128, symmetric int4, bf16 activations.  One *step* is one pass over
those 12 GEMMs, launched through the public op surface (``vllm_amd._custom_ops.gptq_marlin_gemm`` -> C ABI) and
replayed as a HIP graph, as a serving loop would run them.  Every GEMM of a step reads its own copy of the weights and
two full sets alternate between steps, so ~650 MB of distinct weights cycle through the 256 MB Infinity Cache: the
figure is an HBM figure, not a cache figure.

``value`` = algorithmic bytes of one step / time of one step (GB/s); inputs are resident in HBM before the timed
region.  ``roofline`` prices the dominant kernel (the decode GEMM) against the 8 TB/s HBM peak; ``cpu_baseline`` times
the CPU oracle (torch dequantise + matmul, the reference's CPU-runnable path) on a bounded sample on the host cores.
Extra sections (prefill W4A16, FP8 GEMM and FP8 activation quant, each against its own roofline) are reported under
``extra`` and on stderr; they are measured outside the timed region.

One GPU only: ``--gpus N`` with N > 1 exits with a message.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

LLAMA_SHAPES = [(4096, 6144), (4096, 4096), (4096, 28672), (14336, 4096)]   # (K, N): qkv, o, gate_up, down
DECODE_MS = (1, 4, 16)
HBM_PEAK_GBS = 8000.0
# HBM bytes moved per algorithmic byte over the 12 headline GEMMs, from two hardware-counter runs of
# `bench.py --counter-pass` (FETCH_SIZE, then WRITE_SIZE), each scaled by what the same counter reads for the 256 MiB
# copy in that run (FETCH_SIZE reads 131083.5 for 262144 KiB -> x2.000, WRITE_SIZE reads 262144.0 -> x1.000):
# fetch 351.15 MB + write 2.90 MB = 354.04 MB against 340.30 MB algorithmic.  The excess is the fp32 split-K partials and
# scale rows of the K=14336, M=16 case (1.18x there), activation re-reads by every XCD at M=16, and 3-6 % on the fetch side of the
# small layers (it was 10 % -- a 128-byte line of a scale row spans four 16-column tiles and was fetched by each XCD those
# tiles' workgroups ran on -- before the workgroups of one XCD took neighbouring tiles).
STEPS_PER_GRAPH = 10      # consecutive steps captured into one HIP graph (see headline())
MEASURED_TRAFFIC_PER_ALGORITHMIC_BYTE = 354.04 / 340.30
BF16_PEAK_TFLOPS = 2500.0
FP8_PEAK_TFLOPS = 5000.0
GROUP = 128


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def w4a16_bytes(m, k, n, asym_act=False):
    b = k * n // 2 + (k // GROUP) * n * 2 + m * k * 2 + m * n * 2
    if asym_act:
        b += (k // GROUP) * n // 2 + 4 * k
    return b


def fp8_mm_bytes(m, k, n, bias=True):
    return k * n + 4 * n + m * k + 4 * m + 2 * m * n + (2 * n if bias else 0)


# --------------------------------------------------------------------------------------------- device-side workload

class W4Layer:
    """Synthetic GPTQ layer already in the GEMM's native layout (random bits == uniform int4 codes)."""

    def __init__(self, k, n, dev, gen, asym=False, act_order=False):
        from vllm_amd.layers.quantization.utils.marlin_utils import marlin_make_workspace_new
        from vllm_amd.scalar_type import scalar_types
        self.k, self.n = k, n
        self.w = torch.randint(-2 ** 31, 2 ** 31 - 1, (k // 16, 2 * n), dtype=torch.int32, device=dev, generator=gen)
        self.s = (torch.randn(k // GROUP, n, device=dev, generator=gen).abs() * 0.01 + 1e-3).to(torch.float16).to(torch.bfloat16)
        self.empty = torch.empty(0, dtype=torch.int32, device=dev)
        self.zp = self.empty
        self.wtype = scalar_types.uint4b8
        if asym:
            self.zp = torch.randint(-2 ** 31, 2 ** 31 - 1, (k // GROUP, n // 8), dtype=torch.int32, device=dev, generator=gen)
            self.wtype = scalar_types.uint4
        self.g_idx = self.perm = self.empty
        if act_order:
            self.perm = torch.randperm(k, device=dev, generator=gen).to(torch.int32)
            self.g_idx = (torch.arange(k, device=dev) // GROUP).to(torch.int32)
        self.ws = marlin_make_workspace_new(dev)

    def __call__(self, a):
        import vllm_amd._custom_ops as ops
        return ops.gptq_marlin_gemm(a, None, self.w, None, self.s, None, self.zp, self.g_idx, self.perm, self.ws,
                                    self.wtype, a.shape[0], self.n, self.k, is_k_full=True, use_fp32_reduce=True)


def time_graph(fn, iters, warmup, inner=1):
    """Capture ``fn`` (a sequence of launches) into a HIP graph, replay; returns seconds per replay."""
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        fn()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    # warm up for at least ~30 ms of GPU time: the shader clock needs milliseconds to ramp up
    t_end = time.perf_counter() + 0.03
    n = 0
    while n < warmup or time.perf_counter() < t_end:
        g.replay()
        n += 1
        if n % 8 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    best = None
    for _ in range(3):                      # median of three timed bursts
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) * 1e-3 / iters / inner
        best = [t] if best is None else best + [t]
    return sorted(best)[1]


def headline(dev, steps, warmup):
    gen = torch.Generator(device=dev).manual_seed(0)
    sets = []
    for _ in range(2):          # two full weight sets alternate between steps
        layers = [(W4Layer(k, n, dev, gen), m) for (k, n) in LLAMA_SHAPES for m in DECODE_MS]
        sets.append(layers)
    acts = {(k, m): torch.randn(m, k, device=dev, generator=gen).to(torch.bfloat16) for (k, _) in LLAMA_SHAPES for m in DECODE_MS}
    step_bytes = sum(w4a16_bytes(m, k, n) for (k, n) in LLAMA_SHAPES for m in DECODE_MS)
    weight_bytes = sum(l.w.numel() * 4 for layers in sets for l, _ in layers)
    log(f"[headline] 12 GEMMs/step, {step_bytes / 1e6:.1f} MB algorithmic per step, {weight_bytes / 1e6:.0f} MB of distinct weights cycling")

    def run_set(i):
        for layer, m in sets[i]:
            layer(acts[(layer.k, m)])

    # Steps are replayed from HIP graphs of up to STEPS_PER_GRAPH consecutive steps (the two weight sets alternating inside
    # the graph as they do between steps): a decode step of a model is one graph of hundreds of kernels, so the gap
    # between two graph launches (several microseconds) belongs to the harness, not to a 12-GEMM step.
    run_set(0)
    run_set(1)
    torch.cuda.synchronize()
    cache = {}

    def graph_of(n_steps, first):
        key = (n_steps, first & 1)
        if key not in cache:
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                for i in range(n_steps):
                    run_set((first + i) & 1)
            cache[key] = g
        return cache[key]

    def plan(n_steps):
        out, done = [], 0
        while done < n_steps:
            n = min(STEPS_PER_GRAPH, n_steps - done)
            out.append(graph_of(n, done))
            done += n
        return out

    warm, timed = plan(warmup), plan(steps)
    for g in warm:
        g.replay()
    torch.cuda.synchronize()
    # timed region: exactly `steps` steps, events on the stream the kernels run on, synchronised on both sides
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for g in timed:
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    sec = e0.elapsed_time(e1) * 1e-3 / steps
    return sec, step_bytes, sets, acts


def per_shape_decode(dev, sets, acts):
    """Each decode GEMM on its own: graph of its launches over both weight copies plus enough extra copies to stay
    cold would need more memory than is useful; instead alternate the two copies interleaved with the other layers'
    launches removed -- i.e. warm-ish for small layers.  Reported as 'cache-resident unless noted'."""
    rows = []
    gen = torch.Generator(device=dev).manual_seed(1)
    for (k, n) in LLAMA_SHAPES:
        copies = max(2, int(600e6 // (k * n // 2)))
        layers = [W4Layer(k, n, dev, gen) for _ in range(copies)]
        for m in DECODE_MS:
            a = acts[(k, m)]

            def fn():
                for l in layers:
                    l(a)
            t = time_graph(fn, iters=10, warmup=3, inner=copies)
            b = w4a16_bytes(m, k, n)
            rows.append(dict(kind="w4a16_decode", K=k, N=n, M=m, us=t * 1e6, GBps=b / t / 1e9, hbm_frac=b / t / 1e9 / HBM_PEAK_GBS,
                             TFLOPs=2 * m * n * k / t / 1e12, cold=True))
            log(f"[decode  cold] K={k:5d} N={n:5d} M={m:2d}: {t * 1e6:7.2f} us  {b / t / 1e9:7.0f} GB/s ({100 * b / t / 1e9 / HBM_PEAK_GBS:4.1f}% of 8 TB/s)")
        del layers
    return rows


def stream_ceiling_section(dev):
    """What a kernel that only READS a layer's bytes achieves on this machine, launch to launch in the same kind of HIP
    graph as the decode GEMMs and on buffers that have left the caches (600 MB of copies cycling): launch gap +
    first-byte latency + streaming.  `vaq_stream_read_probe` (16-byte loads, every load of a wavefront in flight at
    once), best of a few wavefront counts and depths per size.  The sum over the 12 headline GEMMs is the practical
    ceiling the headline is also priced against."""
    import ctypes
    from vllm_amd.build import BENCH_PROBE_PATH
    if not BENCH_PROBE_PATH.exists():
        raise RuntimeError(f"{BENCH_PROBE_PATH.name} is not built")
    lib = ctypes.CDLL(str(BENCH_PROBE_PATH))
    lib.vaq_stream_read_probe.restype = ctypes.c_int
    lib.vaq_stream_read_probe.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    rows = []
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    pool = torch.empty(640 << 20, dtype=torch.uint8, device=dev).random_()
    stream = lambda: ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)      # noqa: E731
    for (k, n) in LLAMA_SHAPES:
        nbytes = k * n // 2 + (k // GROUP) * n * 2                   # what every GEMM on this layer must read
        copies = max(2, pool.numel() // nbytes)
        best = None
        for waves in (1024, 2048, 4096):
            for depth in (4, 8):
                if nbytes // 1024 // waves < depth:
                    continue

                def fn():
                    for c in range(copies):
                        rc = lib.vaq_stream_read_probe(ctypes.c_void_p(pool.data_ptr() + c * (nbytes & ~1023)), nbytes, waves,
                                                       depth, ctypes.c_void_p(sink.data_ptr()), stream())
                        if rc != 0:
                            raise RuntimeError(f"vaq_stream_read_probe returned {rc}")
                t = time_graph(fn, iters=5, warmup=2, inner=copies)
                read = (nbytes // 1024 // waves) * waves * 1024
                t_full = t * nbytes / read                                  # (the probe reads whole KiB per wavefront)
                if best is None or t_full < best[0]:
                    best = (t_full, waves, depth)
        rows.append(dict(kind="stream_read_ceiling", K=k, N=n, bytes=nbytes, us=best[0] * 1e6, GBps=nbytes / best[0] / 1e9,
                         waves=best[1], depth=best[2]))
        log(f"[read ceiling] {nbytes / 1e6:6.2f} MB (K={k} N={n}): {best[0] * 1e6:6.2f} us launch to launch = {nbytes / best[0] / 1e9:5.0f} GB/s "
            f"({best[1]} wavefronts, {best[2]} loads in flight)")
    # for scale: what the same kernel reaches when one launch reads the whole pool (more than twice the memory-side cache)
    big = pool.numel() & ~((1 << 23) - 1)

    def fn_big():
        rc = lib.vaq_stream_read_probe(ctypes.c_void_p(pool.data_ptr()), big, 8192, 8, ctypes.c_void_p(sink.data_ptr()), stream())
        if rc != 0:
            raise RuntimeError(f"vaq_stream_read_probe returned {rc}")
    t_big = time_graph(fn_big, iters=5, warmup=2, inner=1)
    log(f"[read ceiling] {big / 1e6:6.1f} MB in one launch: {t_big * 1e6:6.1f} us = {big / t_big / 1e9:5.0f} GB/s (8192 wavefronts, 8 loads in flight): "
        "what the layers' sizes leave unreached")
    return rows


def mix_probe(dev, iters=3000):
    """The matrix core under the instruction mixes of candidate GEMM main loops (`vaq_mfma_mix_probe` of the bench-only
    probe library: MFMAs of either shape with LDS fragment reads and VALU work between them, operands that vary).  Not a
    measurement of the product: it prices design alternatives (weights dequantised into LDS or in registers, one or two
    wavefronts per SIMD, 32x32 or 16x16 MFMAs) and gives the ceiling a real main loop can be read against.  Each
    configuration runs twice; the second launch is timed by its own 100 MHz counter and by events."""
    import ctypes
    from vllm_amd.build import BENCH_PROBE_PATH
    lib = ctypes.CDLL(str(BENCH_PROBE_PATH))
    lib.vaq_mfma_mix_probe_name.restype = ctypes.c_char_p
    lib.vaq_mfma_mix_probe_flops.restype = ctypes.c_double
    lib.vaq_mfma_mix_probe.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    ticks = torch.zeros(2048, dtype=torch.int64, device=dev)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    rows = []
    for i in range(lib.vaq_mfma_mix_probe_count()):
        name = lib.vaq_mfma_mix_probe_name(i).decode()
        flops = lib.vaq_mfma_mix_probe_flops(i, iters)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for rep in range(2):
            ticks.zero_()
            e0.record()
            rc = lib.vaq_mfma_mix_probe(i, iters, ctypes.c_void_p(ticks.data_ptr()), ctypes.c_void_p(sink.data_ptr()), stream)
            e1.record()
            if rc != 0:
                raise RuntimeError(f"vaq_mfma_mix_probe({i}) returned {rc}")
            torch.cuda.synchronize()
        # (the mean of the wavefronts' own loop times reads lower than the kernel's duration when two share a SIMD:
        # the older wavefront is served first and finishes early; the kernel's duration is what counts)
        t = ticks[ticks > 0].double()
        loop_us = float(t.mean()) / 100.0
        ev_us = e0.elapsed_time(e1) * 1e3
        rows.append(dict(config=name, event_us=ev_us, PFLOPs=flops / ev_us / 1e9, mean_wavefront_loop_us=loop_us))
        log(f"[mix probe] {flops / ev_us / 1e9:5.2f} PFLOP/s  {name}")
    return rows


def weight_walk_probe(dev):
    """Cold read rate of a GEMM tile kernel's weight access pattern, without the GEMM (`vaq_weight_walk_probe` of the
    bench-only probe library): workgroups that own 64 .. 256 rows of a 4096 x 28672-byte weight matrix (the FP8 gate_up
    layer) and take 64 .. 512 bytes of each row per step, against long contiguous runs.  Copies of the matrix cycle
    through 700 MB, so every launch reads from HBM; launch to launch in a HIP graph like the GEMMs."""
    import ctypes
    from vllm_amd.build import BENCH_PROBE_PATH
    lib = ctypes.CDLL(str(BENCH_PROBE_PATH))
    lib.vaq_weight_walk_probe_name.restype = ctypes.c_char_p
    lib.vaq_weight_walk_probe.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    rows_total, rowbytes, copies = 28672, 4096, 6
    pool = torch.empty(copies * rows_total * rowbytes, dtype=torch.uint8, device=dev).random_()
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    out = []
    for i in range(lib.vaq_weight_walk_probe_count()):
        name = lib.vaq_weight_walk_probe_name(i).decode()

        def fn():
            st = torch.cuda.current_stream(dev).cuda_stream
            for c in range(copies):
                rc = lib.vaq_weight_walk_probe(i, pool.data_ptr() + c * rows_total * rowbytes, rows_total, rowbytes,
                                               sink.data_ptr(), st)
                if rc != 0:
                    raise RuntimeError(f"vaq_weight_walk_probe({i}) returned {rc}")
        t = time_graph(fn, iters=5, warmup=2, inner=copies)
        out.append(dict(config=name, us=t * 1e6, GBps=rows_total * rowbytes / t / 1e9))
        log(f"[weight walk] {t * 1e6:6.1f} us = {rows_total * rowbytes / t / 1e9:5.0f} GB/s  {name}")
    # the GEMM beside it: the same bytes as FP8 weights at M = 256, cold
    import vllm_amd._custom_ops as ops
    gen = torch.Generator(device=dev).manual_seed(5)
    w = [pool[c * rows_total * rowbytes:(c + 1) * rows_total * rowbytes].view(torch.float8_e4m3fn).view(rows_total, rowbytes).t()
         for c in range(copies)]
    for m in (16, 256):
        a = torch.randn(m, rowbytes, device=dev, generator=gen).to(torch.float8_e4m3fn)
        sa = torch.rand(m, 1, device=dev, generator=gen) + 0.5
        sb = torch.rand(rows_total, 1, device=dev, generator=gen) + 0.5
        t = time_graph(lambda: [ops.cutlass_scaled_mm(a, wc, sa, sb, torch.bfloat16) for wc in w], iters=5, warmup=2, inner=copies)
        out.append(dict(config=f"FP8 GEMM M={m}", us=t * 1e6, GBps=rows_total * rowbytes / t / 1e9))
        log(f"[weight walk] {t * 1e6:6.1f} us = {rows_total * rowbytes / t / 1e9:5.0f} GB/s  the FP8 GEMM on the same bytes at M = {m}")
    return out


def prefill_section(dev):
    """BASELINE.json config 3: asymmetric uint4 + act_order, both readings of its act_order wording.  `rows`: g_idx from a
    random permutation of the K rows (the reference's generator): activations are reordered on every call.  `groups`:
    g_idx permutes whole groups: the linear method folds it into the scale / zero-point rows at load time, so the GEMM
    runs without a permutation (same kernel as no act_order)."""
    rows = []
    gen = torch.Generator(device=dev).manual_seed(2)
    for (k, n) in LLAMA_SHAPES:
        for variant in ("rows", "groups"):
            layer = W4Layer(k, n, dev, gen, asym=True, act_order=(variant == "rows"))
            for m in (512, 2048, 4096):
                a = torch.randn(m, k, device=dev, generator=gen).to(torch.bfloat16)
                inner = 4 if m <= 512 else 1
                t = time_graph(lambda: [layer(a) for _ in range(inner)], iters=5, warmup=2, inner=inner)
                fl = 2.0 * m * n * k
                rows.append(dict(kind=f"w4a16_prefill_asym_actorder_{variant}", K=k, N=n, M=m, us=t * 1e6, TFLOPs=fl / t / 1e12,
                                 mfma_frac=fl / t / 1e12 / BF16_PEAK_TFLOPS, GBps=w4a16_bytes(m, k, n, True) / t / 1e9))
                log(f"[prefill {variant:6s}] K={k:5d} N={n:5d} M={m:4d}: {t * 1e6:8.1f} us  {fl / t / 1e12:7.1f} TFLOP/s ({100 * fl / t / 1e12 / BF16_PEAK_TFLOPS:4.1f}% of 2.5 PF)")
            del layer
    return rows


def fused_norm_quant_section(dev):
    """RMSNorm + per-token FP8 quant in one pass (the step in front of the FP8 GEMM) against its HBM roofline, and the
    unfused pair (torch rms_norm, then scaled_fp8_quant) beside it."""
    import torch.nn.functional as F
    import vllm_amd._custom_ops as ops
    rows = []
    gen = torch.Generator(device=dev).manual_seed(6)
    for k in (4096, 14336):
        w = (1.0 + 0.1 * torch.randn(k, device=dev, generator=gen)).to(torch.bfloat16)
        for m in (16, 256, 4096):
            x = torch.randn(m, k, device=dev, generator=gen).to(torch.bfloat16)
            t = time_graph(lambda: [ops.rms_norm_dynamic_per_token_quant(x, w, 1e-5, torch.float8_e4m3fn) for _ in range(20)],
                           iters=5, warmup=2, inner=20)
            tu = time_graph(lambda: [ops.scaled_fp8_quant(F.rms_norm(x, (k,), w, 1e-5), use_per_token_if_dynamic=True) for _ in range(20)],
                            iters=5, warmup=2, inner=20)
            b = 3 * m * k + 4 * m + 2 * k
            rows.append(dict(kind="rms_norm_dynamic_per_token_fp8_quant", hidden=k, M=m, us=t * 1e6, GBps=b / t / 1e9,
                             hbm_frac=b / t / 1e9 / HBM_PEAK_GBS, unfused_us=tu * 1e6, cold=False))
            log(f"[norm+quant  ] hidden={k:5d} M={m:4d}: {t * 1e6:6.1f} us {b / t / 1e9:6.0f} GB/s ({100 * b / t / 1e9 / HBM_PEAK_GBS:4.1f}% of 8 TB/s) | "
                f"unfused rms_norm + quant {tu * 1e6:6.1f} us")
    # static-scale variants at the prefill size: norm (+ residual) + quant, and silu(gate) * up + quant (d = 14336)
    one = torch.ones(1, device=dev, dtype=torch.float32)
    m, k = 4096, 4096
    w = (1.0 + 0.1 * torch.randn(k, device=dev, generator=gen)).to(torch.bfloat16)
    x = torch.randn(m, k, device=dev, generator=gen).to(torch.bfloat16)
    res = torch.randn(m, k, device=dev, generator=gen).to(torch.bfloat16)
    out = torch.empty(m, k, device=dev, dtype=torch.float8_e4m3fn)
    for kind, fn, b in (
            ("rms_norm_static_fp8_quant", lambda: ops.rms_norm_static_fp8_quant(out, x, w, one, 1e-6), 3 * m * k + 2 * k),
            ("fused_add_rms_norm_static_fp8_quant",
             lambda: ops.fused_add_rms_norm_static_fp8_quant(out, x, res, w, one, 1e-6), 7 * m * k + 2 * k)):
        t = time_graph(lambda: [fn() for _ in range(20)], iters=5, warmup=2, inner=20)
        rows.append(dict(kind=kind, hidden=k, M=m, us=t * 1e6, GBps=b / t / 1e9, hbm_frac=b / t / 1e9 / HBM_PEAK_GBS, cold=False))
        log(f"[norm+quant  ] {kind} hidden={k} M={m}: {t * 1e6:6.1f} us {b / t / 1e9:6.0f} GB/s ({100 * b / t / 1e9 / HBM_PEAK_GBS:4.1f}% of 8 TB/s)")
    d = 14336
    gu = torch.randn(m, 2 * d, device=dev, generator=gen).to(torch.bfloat16)
    out2 = torch.empty(m, d, device=dev, dtype=torch.float8_e4m3fn)
    t = time_graph(lambda: [ops.silu_and_mul_quant(out2, gu, one) for _ in range(10)], iters=5, warmup=2, inner=10)
    tu = time_graph(lambda: [ops.scaled_fp8_quant(F.silu(gu[:, :d]) * gu[:, d:], one) for _ in range(10)], iters=5, warmup=2, inner=10)
    b = 5 * m * d
    rows.append(dict(kind="silu_and_mul_quant", d=d, M=m, us=t * 1e6, GBps=b / t / 1e9, hbm_frac=b / t / 1e9 / HBM_PEAK_GBS,
                     unfused_us=tu * 1e6, cold=False))
    log(f"[silu+quant  ] d={d} M={m}: {t * 1e6:6.1f} us {b / t / 1e9:6.0f} GB/s ({100 * b / t / 1e9 / HBM_PEAK_GBS:4.1f}% of 8 TB/s) | "
        f"unfused silu*mul + quant {tu * 1e6:6.1f} us")
    return rows


def variants_section(dev):
    """The other weight formats of the W4A16 GEMM -- groups of 64 / 32 rows, channelwise scales, 8-bit codes
    (uint8b128), FP8 e4m3 weights with 16-bit activations -- on gate_up_proj (4096 x 28672) at a decode size (cold weights, several copies cycling) and at
    M = 4096.  Bytes count weights, scales and zero points of the format."""
    from vllm_amd.scalar_type import scalar_types
    rows = []
    gen = torch.Generator(device=dev).manual_seed(7)
    k, n = 4096, 28672
    for name, gs, bits in (("g128", 128, 4), ("g64", 64, 4), ("g32", 32, 4), ("channelwise", -1, 4), ("8bit_g128", 128, 8),
                           ("fp8_weights_channelwise", -1, 8)):
        grp = 1 if gs == -1 else k // gs
        copies = 6
        layers = []
        for _ in range(copies):
            l = W4Layer(k, n, dev, gen)
            if bits == 8:
                l.w = torch.randint(-2 ** 31, 2 ** 31 - 1, (k // 16, 4 * n), dtype=torch.int32, device=dev, generator=gen)
                l.wtype = scalar_types.uint8b128
                if name.startswith("fp8"):
                    # e4m3 bytes in the byte-native order: any byte but the two NaN codes (0x7f, 0xff -> clear bit 0)
                    l.w &= ~0x01010101
                    l.wtype = scalar_types.float8_e4m3fn
            l.s = (torch.randn(grp, n, device=dev, generator=gen).abs() * 0.01 + 1e-3).to(torch.bfloat16)
            layers.append(l)
        wbytes = k * n * bits // 8 + grp * n * 2
        for m in (1, 16, 4096):
            a = torch.randn(m, k, device=dev, generator=gen).to(torch.bfloat16)
            use = layers if m <= 16 else layers[:2]

            def fn():
                for l in use:
                    l(a)
            t = time_graph(fn, iters=5, warmup=2, inner=len(use))
            b = wbytes + 2 * m * (k + n)
            fl = 2.0 * m * n * k
            rows.append(dict(kind="w4a16_variant", variant=name, K=k, N=n, M=m, us=t * 1e6, GBps=b / t / 1e9,
                             hbm_frac=b / t / 1e9 / HBM_PEAK_GBS, TFLOPs=fl / t / 1e12, cold=m <= 16))
            log(f"[variant {name:11s}] K={k} N={n} M={m:4d}: {t * 1e6:8.1f} us  {b / t / 1e9:6.0f} GB/s ({100 * b / t / 1e9 / HBM_PEAK_GBS:4.1f}% of 8 TB/s)  "
                f"{fl / t / 1e12:7.1f} TFLOP/s")
        del layers
    return rows


def host_overhead_section(dev):
    """Host time per eager call of the ops (Python checks + ctypes + workspace query + launch), M = 1 on 4096 x 4096: what a
    caller pays per GEMM outside a HIP graph.  The queue is kept short enough that the host, not the device, is timed."""
    import vllm_amd._custom_ops as ops
    gen = torch.Generator(device=dev).manual_seed(9)
    k = n = 4096
    layer = W4Layer(k, n, dev, gen)
    a = torch.randn(1, k, device=dev, generator=gen).to(torch.bfloat16)
    w = (torch.randn(n, k, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
    wq, wsc = ops.scaled_fp8_quant(w, use_per_token_if_dynamic=True)
    aq, sa = ops.scaled_fp8_quant(a, use_per_token_if_dynamic=True)
    calls = (("gptq_marlin_gemm", lambda: layer(a)),
             ("cutlass_scaled_mm", lambda: ops.cutlass_scaled_mm(aq, wq.t(), sa, wsc, torch.bfloat16)),
             ("scaled_fp8_quant", lambda: ops.scaled_fp8_quant(a, use_per_token_if_dynamic=True)))
    rows = []
    for name, fn in calls:
        for _ in range(50):
            fn()
        torch.cuda.synchronize()
        n_calls = 1000
        t0 = time.perf_counter()
        for _ in range(n_calls):
            fn()
        t = (time.perf_counter() - t0) / n_calls
        torch.cuda.synchronize()
        rows.append(dict(kind="eager_host_time_per_call", op=name, us=t * 1e6))
        log(f"[host overhead] {name:18s}: {t * 1e6:6.1f} us of host time per eager call")
    return rows


def vendor_ceiling_section(dev):
    """Practical ceilings on the same box and shapes: the vendor GEMM library through torch (bf16 `matmul`, row-wise
    scaled FP8 `_scaled_mm`) at M = 4096.  Context for the MFMA fractions above, not part of the product path."""
    rows = []
    gen = torch.Generator(device=dev).manual_seed(4)
    m = 4096
    for (k, n) in LLAMA_SHAPES:
        a = torch.randn(m, k, device=dev, generator=gen).to(torch.bfloat16)
        w = (torch.randn(n, k, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
        fl = 2.0 * m * n * k
        t = time_graph(lambda: [torch.matmul(a, w.t()) for _ in range(2)], iters=5, warmup=2, inner=2)
        rows.append(dict(kind="vendor_bf16_matmul", K=k, N=n, M=m, us=t * 1e6, TFLOPs=fl / t / 1e12))
        log(f"[vendor bf16 ] K={k:5d} N={n:5d} M={m:4d}: {t * 1e6:8.1f} us  {fl / t / 1e12:7.1f} TFLOP/s")
        try:
            aq = a.to(torch.float8_e4m3fn)
            wq = w.to(torch.float8_e4m3fn)
            sa = torch.ones(m, 1, device=dev, dtype=torch.float32)
            sb = torch.ones(1, n, device=dev, dtype=torch.float32)
            t = time_graph(lambda: [torch._scaled_mm(aq, wq.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16) for _ in range(2)],
                           iters=5, warmup=2, inner=2)
            rows.append(dict(kind="vendor_fp8_scaled_mm_rowwise", K=k, N=n, M=m, us=t * 1e6, TFLOPs=fl / t / 1e12))
            log(f"[vendor fp8  ] K={k:5d} N={n:5d} M={m:4d}: {t * 1e6:8.1f} us  {fl / t / 1e12:7.1f} TFLOP/s")
        except Exception as e:   # not every torch build exposes row-wise FP8 scaling
            log(f"[vendor fp8  ] unavailable: {str(e)[:80]}")
        del a, w
    return rows


def vendor_small_m_section(dev):
    """The same two vendor GEMMs beside this library's at M = 16 / 64 / 128 / 256 / 1024 with cold weights (distinct copies cycle
    through the graph, as in the decode section): where the weight bytes and the launch matter more than the matrix
    core.  The W4A16 GEMM stands beside the vendor's bf16 GEMM, which reads four times its weight bytes."""
    import vllm_amd._custom_ops as ops
    rows = []
    gen = torch.Generator(device=dev).manual_seed(5)
    for (k, n) in LLAMA_SHAPES:
        n8 = max(2, int(600e6 // (k * n)))
        w8 = [(torch.randn(n, k, device=dev, generator=gen) * 0.05).to(torch.float8_e4m3fn) for _ in range(n8)]
        n16 = max(2, n8 // 2)
        w16 = [(torch.randn(n, k, device=dev, generator=gen) * 0.05).to(torch.bfloat16) for _ in range(n16)]
        layers = [W4Layer(k, n, dev, gen, asym=True) for _ in range(max(2, int(600e6 // (k * n // 2))))]
        sb = torch.rand(n, 1, device=dev, generator=gen) + 0.5
        for m in (16, 64, 128, 256, 1024):
            a8 = torch.randn(m, k, device=dev, generator=gen).to(torch.float8_e4m3fn)
            a16 = torch.randn(m, k, device=dev, generator=gen).to(torch.bfloat16)
            sa = torch.rand(m, 1, device=dev, generator=gen) + 0.5
            t = {}
            t["fp8"] = time_graph(lambda: [ops.cutlass_scaled_mm(a8, w.t(), sa, sb, torch.bfloat16) for w in w8], iters=5, warmup=2, inner=n8)
            try:
                t["vendor_fp8"] = time_graph(lambda: [torch._scaled_mm(a8, w.t(), scale_a=sa, scale_b=sb.t(), out_dtype=torch.bfloat16)
                                                      for w in w8], iters=5, warmup=2, inner=n8)
            except Exception:   # not every torch build exposes row-wise FP8 scaling
                t["vendor_fp8"] = float("nan")
            t["w4a16"] = time_graph(lambda: [l(a16) for l in layers], iters=5, warmup=2, inner=len(layers))
            t["vendor_bf16"] = time_graph(lambda: [torch.matmul(a16, w.t()) for w in w16], iters=5, warmup=2, inner=n16)
            rows.append(dict(kind="vendor_small_m", K=k, N=n, M=m, cold=True, **{f"{name}_us": v * 1e6 for name, v in t.items()}))
            log(f"[vendor small M] K={k:5d} N={n:5d} M={m:4d}: FP8 {t['fp8'] * 1e6:6.1f} us (vendor {t['vendor_fp8'] * 1e6:6.1f}) | "
                f"W4A16 {t['w4a16'] * 1e6:6.1f} us (vendor bf16 {t['vendor_bf16'] * 1e6:6.1f})")
        del w8, w16, layers
    return rows


def operand_toggle_section(dev):
    """The M = 4096 GEMMs on 4096 x 4096 with random operands and with operands that do not toggle (all activations 1.0,
    all weight codes / bytes equal): the same instruction stream on the same addresses, so the difference is what the
    chip's power management takes when the data paths switch -- the reason these kernels are read against a power-
    limited matrix-core ceiling rather than the nominal one.  The vendor GEMMs of the same shape ride along."""
    import vllm_amd._custom_ops as ops
    rows = []
    gen = torch.Generator(device=dev).manual_seed(7)
    m, k, n = 4096, 4096, 4096
    fl = 2.0 * m * n * k
    for const in (False, True):
        layer = W4Layer(k, n, dev, gen, asym=True)
        a = torch.randn(m, k, device=dev, generator=gen).to(torch.bfloat16)
        w16 = (torch.randn(n, k, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
        if const:
            a.fill_(1.0)
            w16.fill_(0.02)
            layer.w.fill_(0x11111111)
            layer.s.fill_(0.0078125)
            layer.zp.fill_(0)
        wq, ws = ops.scaled_fp8_quant(w16, use_per_token_if_dynamic=True)
        aq, sa = ops.scaled_fp8_quant(a, use_per_token_if_dynamic=True)
        sb1 = torch.ones(1, n, device=dev, dtype=torch.float32)
        sa1 = torch.ones(m, 1, device=dev, dtype=torch.float32)
        cases = (("w4a16", lambda: layer(a)), ("fp8", lambda: ops.cutlass_scaled_mm(aq, wq.t(), sa, ws, torch.bfloat16, None)),
                 ("vendor_bf16", lambda: torch.matmul(a, w16.t())),
                 ("vendor_fp8", lambda: torch._scaled_mm(aq, wq.t(), scale_a=sa1, scale_b=sb1, out_dtype=torch.bfloat16)))
        for name, fn in cases:
            try:
                t = time_graph(lambda: [fn() for _ in range(2)], iters=8, warmup=3, inner=2)
            except Exception as e:
                log(f"[operand toggle] {name}: unavailable ({str(e)[:60]})")
                continue
            rows.append(dict(kind=name, operands="constant" if const else "random", K=k, N=n, M=m, us=t * 1e6, TFLOPs=fl / t / 1e12))
            log(f"[operand toggle] {name:11s} {'constant' if const else 'random  '} operands: {t * 1e6:7.1f} us  {fl / t / 1e12:7.1f} TFLOP/s")
    # The other face of the same limit: one workgroup per 256 x 256 tile, K unsplit, on a quarter, half and all of the
    # compute units (M = 1024 / 2048 / 4096).  Every workgroup does the same work; what changes is how many run at once.
    from vllm_amd import _tuning
    layer = W4Layer(k, n, dev, gen, asym=True)
    for mm in (1024, 2048, 4096):
        a = torch.randn(mm, k, device=dev, generator=gen).to(torch.bfloat16)

        def whole_tiles():
            with _tuning.override(prefill_tile=21, prefill_split=1):
                layer(a)
        t = time_graph(lambda: [whole_tiles() for _ in range(2)], iters=8, warmup=3, inner=2)
        rows.append(dict(kind="w4a16_whole_tiles", workgroups=(mm // 256) * (n // 256), K=k, N=n, M=mm, us=t * 1e6))
        log(f"[operand toggle] w4a16, one workgroup per 256 x 256 tile, K unsplit: {(mm // 256) * (n // 256):3d} workgroups {t * 1e6:7.1f} us")
    return rows


def decode_step_section(dev):
    """BASELINE.json config 5: one decode step of a random-init Llama-3-8B-architecture model, batch 32, context 1024.  The
    32 x 4 linear layers are `QKVParallelLinear` / `RowParallelLinear` / `MergedColumnParallelLinear` modules carrying
    `GPTQMarlinLinearMethod` (random int4 codes and scales written into the checkpoint-format parameters, then
    `process_weights_after_loading`), called through `layer(x)` -> `quant_method.apply`: M = 32, distinct weights per
    layer (3.6 GB).  Norms, rotary-free attention over a bf16 KV cache, SiLU-mul, embedding and the bf16 lm_head are plain
    torch ops standing in for the rest of the model.  Reports the step time, tokens/s, and the time share of the
    quantized GEMMs per projection type: each type's 32 layers replayed as their own HIP graph (cold weights), the way
    the reference's layerwise profiler (vllm/profiler/layerwise_profile.py:365) attributes kernel time to modules."""
    import torch.nn.functional as F
    from vllm_amd.layers.linear import MergedColumnParallelLinear, QKVParallelLinear, RowParallelLinear
    from vllm_amd.layers.quantization import get_quantization_config
    gen = torch.Generator(device=dev).manual_seed(5)
    B, CTX, H, NQ, NKV, HD, FF, V, L = 32, 1024, 4096, 32, 8, 128, 14336, 128256, 32
    cfg = get_quantization_config("gptq_marlin").from_config(dict(bits=4, group_size=GROUP, desc_act=False, sym=True))

    def quantized(layer):
        layer = layer.to(dev)
        layer.qweight.data.random_(-2 ** 31, 2 ** 31 - 1, generator=gen)       # uniform int4 codes
        layer.scales.data.copy_((torch.randn(layer.scales.shape, device=dev, generator=gen).abs() * 0.01 + 1e-3)
                                .to(torch.float16).to(torch.bfloat16))
        layer.g_idx.data.copy_(torch.arange(layer.input_size, device=dev, dtype=torch.int32) // GROUP)
        layer.process_weights_after_loading()
        return layer

    kw = dict(quant_config=cfg, params_dtype=torch.bfloat16, return_bias=False)
    layers = []
    for _ in range(L):
        layers.append(dict(qkv=quantized(QKVParallelLinear(H, HD, NQ, NKV, **kw)), o=quantized(RowParallelLinear(H, H, **kw)),
                           gate_up=quantized(MergedColumnParallelLinear(H, [FF, FF], **kw)),
                           down=quantized(RowParallelLinear(FF, H, **kw)),
                           kc=torch.randn(B, NKV, CTX, HD, device=dev, generator=gen).to(torch.bfloat16),
                           vc=torch.randn(B, NKV, CTX, HD, device=dev, generator=gen).to(torch.bfloat16),
                           n1=torch.ones(H, device=dev, dtype=torch.bfloat16), n2=torch.ones(H, device=dev, dtype=torch.bfloat16)))
    emb = (torch.randn(V, H, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
    lm_head = (torch.randn(V, H, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
    ids = torch.randint(0, V, (B,), device=dev, generator=gen)

    def step():
        x = emb[ids]
        for ly in layers:
            qkv = ly["qkv"](F.rms_norm(x, (H,), ly["n1"], 1e-5))
            q = qkv[:, :NQ * HD].view(B, NQ, 1, HD)
            att = F.scaled_dot_product_attention(q, ly["kc"], ly["vc"], enable_gqa=True).reshape(B, H)
            x = x + ly["o"](att)
            gu = ly["gate_up"](F.rms_norm(x, (H,), ly["n2"], 1e-5))
            x = x + ly["down"](F.silu(gu[:, :FF]) * gu[:, FF:])
        return torch.matmul(x, lm_head.t())

    t_full = time_graph(step, iters=5, warmup=2)
    x_h = torch.randn(B, H, device=dev, generator=gen).to(torch.bfloat16)
    x_f = torch.randn(B, FF, device=dev, generator=gen).to(torch.bfloat16)
    shapes = dict(qkv=(H, (NQ + 2 * NKV) * HD), o=(H, H), gate_up=(H, 2 * FF), down=(FF, H))
    per_type = {}
    for name, (k, n) in shapes.items():
        xin = x_f if k == FF else x_h
        t = time_graph(lambda: [ly[name](xin) for ly in layers], iters=5, warmup=2)
        b = L * w4a16_bytes(B, k, n)
        per_type[name] = dict(K=k, N=n, us_per_layer=t * 1e6 / L, us_per_step=t * 1e6, share_of_step=t / t_full,
                              GBps=b / t / 1e9, hbm_frac=b / t / 1e9 / HBM_PEAK_GBS)
        log(f"[decode step ] {name:8s} {k:5d}x{n:5d} M={B}: {t * 1e6 / L:6.2f} us per layer, {100 * t / t_full:4.1f}% of the step, "
            f"{b / t / 1e9:5.0f} GB/s ({100 * b / t / 1e9 / HBM_PEAK_GBS:4.1f}% of 8 TB/s)")
    t_lin = sum(v["us_per_step"] for v in per_type.values()) * 1e-6
    gemm_bytes = L * sum(w4a16_bytes(B, k, n) for (k, n) in LLAMA_SHAPES)
    row = dict(kind="llama3_8b_decode_step", batch=B, context=CTX, layers=L, surface="GPTQMarlinLinearMethod.apply",
               step_us=t_full * 1e6, linear_us=t_lin * 1e6, linear_share=t_lin / t_full, tokens_per_s=B / t_full,
               tokens_per_s_linear_only=B / t_lin, linear_GBps=gemm_bytes / t_lin / 1e9,
               linear_hbm_frac=gemm_bytes / t_lin / 1e9 / HBM_PEAK_GBS, per_projection=per_type)
    log(f"[decode step ] batch {B} ctx {CTX}: {t_full * 1e6:.0f} us/step = {B / t_full:.0f} tok/s; the 128 W4A16 GEMMs (M=32) take "
        f"{t_lin * 1e6:.0f} us = {100 * t_lin / t_full:.0f}% of the step, {gemm_bytes / t_lin / 1e9:.0f} GB/s "
        f"({100 * gemm_bytes / t_lin / 1e9 / HBM_PEAK_GBS:.1f}% of 8 TB/s)")
    return [row]


def fp8_section(dev):
    import vllm_amd._custom_ops as ops
    rows = []
    gen = torch.Generator(device=dev).manual_seed(3)
    for (k, n) in LLAMA_SHAPES:
        w = (torch.randn(n, k, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
        wq, ws = ops.scaled_fp8_quant(w, use_per_token_if_dynamic=True)
        del w
        bias = (torch.randn(n, device=dev, generator=gen) * 0.01).to(torch.bfloat16)
        wt = wq.t()
        # memory-bound sizes (M <= 256) read cold weights: ~600 MB of distinct copies cycle through the graph, as in the
        # decode section; the compute-bound M = 4096 repeats one copy
        copies = [wq.clone().t() for _ in range(max(2, int(600e6 // (k * n))))]
        for m in (1, 16, 256, 4096):
            a = torch.randn(m, k, device=dev, generator=gen).to(torch.bfloat16)
            aq, sa = ops.scaled_fp8_quant(a, use_per_token_if_dynamic=True)
            cold = m <= 256
            inner = len(copies) if cold else 2
            if cold:
                t = time_graph(lambda: [ops.cutlass_scaled_mm(aq, wc, sa, ws, torch.bfloat16, bias) for wc in copies],
                               iters=5, warmup=2, inner=inner)
            else:
                t = time_graph(lambda: [ops.cutlass_scaled_mm(aq, wt, sa, ws, torch.bfloat16, bias) for _ in range(inner)],
                               iters=5, warmup=2, inner=inner)
            tq = time_graph(lambda: [ops.scaled_fp8_quant(a, use_per_token_if_dynamic=True) for _ in range(20)],
                            iters=5, warmup=2, inner=20)
            fl = 2.0 * m * n * k
            b = fp8_mm_bytes(m, k, n)
            qb = 3 * m * k + 4 * m
            rows.append(dict(kind="fp8_scaled_mm", K=k, N=n, M=m, us=t * 1e6, TFLOPs=fl / t / 1e12, mfma_frac=fl / t / 1e12 / FP8_PEAK_TFLOPS,
                             GBps=b / t / 1e9, hbm_frac=b / t / 1e9 / HBM_PEAK_GBS, quant_us=tq * 1e6, quant_GBps=qb / tq / 1e9,
                             cold=cold))
            log(f"[fp8 mm  {'cold' if cold else 'warm'}] K={k:5d} N={n:5d} M={m:4d}: {t * 1e6:8.1f} us  {fl / t / 1e12:7.1f} TFLOP/s ({100 * fl / t / 1e12 / FP8_PEAK_TFLOPS:4.1f}% of 5 PF)  "
                f"{b / t / 1e9:6.0f} GB/s | quant {tq * 1e6:6.1f} us {qb / tq / 1e9:6.0f} GB/s")
        del wq, wt, copies
    return rows


def medium_m_section(dev):
    """The sizes between decode and prefill (M = 64 .. 1024: large decode batches, chunked prefill), cold weights (~600 MB of
    distinct copies cycling): W4A16 (symmetric, groups of 128) and FP8 W8A8 per shape and M."""
    import vllm_amd._custom_ops as ops
    rows = []
    gen = torch.Generator(device=dev).manual_seed(5)
    for (k, n) in LLAMA_SHAPES:
        layers = [W4Layer(k, n, dev, gen) for _ in range(max(2, int(600e6 // (k * n // 2))))]
        wq, ws = ops.scaled_fp8_quant((torch.randn(n, k, device=dev, generator=gen) * 0.02).to(torch.bfloat16),
                                      use_per_token_if_dynamic=True)
        copies = [wq.clone().t() for _ in range(max(2, int(600e6 // (k * n))))]
        for m in (64, 128, 256, 512, 1024):
            a = torch.randn(m, k, device=dev, generator=gen).to(torch.bfloat16)
            aq, sa = ops.scaled_fp8_quant(a, use_per_token_if_dynamic=True)
            t4 = time_graph(lambda: [l(a) for l in layers], iters=5, warmup=2, inner=len(layers))
            t8 = time_graph(lambda: [ops.cutlass_scaled_mm(aq, wc, sa, ws, torch.bfloat16, None) for wc in copies],
                            iters=5, warmup=2, inner=len(copies))
            fl = 2.0 * m * n * k
            rows.append(dict(kind="medium_m", K=k, N=n, M=m, w4a16_us=t4 * 1e6, w4a16_TFLOPs=fl / t4 / 1e12,
                             fp8_us=t8 * 1e6, fp8_TFLOPs=fl / t8 / 1e12, cold=True))
            log(f"[medium M    ] K={k:5d} N={n:5d} M={m:4d}: W4A16 {t4 * 1e6:7.1f} us {fl / t4 / 1e12:6.0f} TFLOP/s | "
                f"FP8 {t8 * 1e6:7.1f} us {fl / t8 / 1e12:6.0f} TFLOP/s")
        del layers, copies, wq
        torch.cuda.empty_cache()
    return rows


def roofline_mfma(extra):
    """The compute-bound kernels against the dense MFMA peaks, from the M = 4096 rows of the prefill and FP8 sections
    (HIP-graph timings of this run): per kernel the FLOPs of one launch, its average duration, the fraction of peak and,
    where the vendor section ran, the vendor library's plain GEMM of the same shape and precision beside it."""
    vendor = {(r["kind"], r["K"], r["N"]): r["us"] for r in extra.get("vendor_ceiling", []) if r.get("M") == 4096}
    out = []
    for r in extra.get("prefill", []):
        if r["M"] == 4096 and r["kind"].endswith("groups"):
            # whole 256 x 256 tiles run on the register-dequantising kernel; a count that ends in a round of workgroups at
            # most half full runs on the 8-wavefront kernel, the tiles of that round in K parts
            tiles, cus = -(-r["M"] // 256) * -(-r["N"] // 256), torch.cuda.get_device_properties(0).multi_processor_count
            name = "vaq::w4a16_prefill2_kernel" if 0 < tiles % cus <= cus // 2 and tiles > cus else "vaq::w4a16_prefill3_kernel"
            row = dict(kernel=name, K=r["K"], N=r["N"], M=r["M"], flops_per_launch=2.0 * r["M"] * r["N"] * r["K"],
                       avg_ns=round(r["us"] * 1e3), peak_TFLOPs=BF16_PEAK_TFLOPS, frac=round(r["mfma_frac"], 4))
            v = vendor.get(("vendor_bf16_matmul", r["K"], r["N"]))
            if v:
                row["vendor_bf16_gemm_ns"] = round(v * 1e3)
            out.append(row)
    for r in extra.get("fp8", []):
        if r["M"] == 4096:
            row = dict(kernel="vaq::fp8_mm_tile3_kernel", K=r["K"], N=r["N"], M=r["M"], flops_per_launch=2.0 * r["M"] * r["N"] * r["K"],
                       avg_ns=round(r["us"] * 1e3), peak_TFLOPs=FP8_PEAK_TFLOPS, frac=round(r["mfma_frac"], 4))
            v = vendor.get(("vendor_fp8_scaled_mm_rowwise", r["K"], r["N"]))
            if v:
                row["vendor_fp8_gemm_ns"] = round(v * 1e3)
            out.append(row)
    return out or None


def mfma_pass(dev):
    """Workload for a matrix-core counter run (`rocprofv3 --pmc`): the vendor library's plain bf16 GEMM at 4096^3 (the
    calibration: a kernel whose FLOPs are known) followed by the W4A16 and FP8 GEMMs at M = 4096 on the four Llama-3-8B
    shapes, eagerly, three times; the last repetition's dispatches are the ones to read."""
    import vllm_amd._custom_ops as ops
    gen = torch.Generator(device=dev).manual_seed(0)
    m = 4096
    a_cal = torch.randn(m, 4096, device=dev, generator=gen).to(torch.bfloat16)
    w_cal = torch.randn(4096, 4096, device=dev, generator=gen).to(torch.bfloat16)
    w4 = [W4Layer(k, n, dev, gen, asym=True) for (k, n) in LLAMA_SHAPES]
    acts = {k: torch.randn(m, k, device=dev, generator=gen).to(torch.bfloat16) for (k, _) in LLAMA_SHAPES}
    f8 = []
    for (k, n) in LLAMA_SHAPES:
        wq, ws = ops.scaled_fp8_quant((torch.randn(n, k, device=dev, generator=gen) * 0.02).to(torch.bfloat16),
                                      use_per_token_if_dynamic=True)
        aq, sa = ops.scaled_fp8_quant(acts[k], use_per_token_if_dynamic=True)
        f8.append((aq, wq.t(), sa, ws))
    torch.cuda.synchronize()
    for _ in range(3):
        torch.matmul(a_cal, w_cal.t())
        for layer in w4:
            layer(acts[layer.k])
        for aq, wt, sa, ws in f8:
            ops.cutlass_scaled_mm(aq, wt, sa, ws, torch.bfloat16, None)
    torch.cuda.synchronize()
    log(f"[mfma pass] calibration GEMM: {2.0 * m * 4096 * 4096:.0f} FLOP; GEMMs: " +
        ", ".join(f"{k}x{n}: {2.0 * m * n * k:.0f}" for (k, n) in LLAMA_SHAPES))


def counter_pass(dev):
    """Workload for a hardware-counter run: a plain 256 MiB device-to-device copy (the calibration kernel: it reads and
    writes exactly 262144 KiB) followed by one eager pass over the 12 headline GEMMs, three times; the last repetition's
    dispatches are the ones to read."""
    gen = torch.Generator(device=dev).manual_seed(0)
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(generator=gen)
    dst = torch.empty_like(src)
    layers = [(W4Layer(k, n, dev, gen), m) for (k, n) in LLAMA_SHAPES for m in DECODE_MS]
    acts = {(k, m): torch.randn(m, k, device=dev, generator=gen).to(torch.bfloat16) for (k, _) in LLAMA_SHAPES for m in DECODE_MS}
    torch.cuda.synchronize()
    for _ in range(3):
        dst.copy_(src)
        for layer, m in layers:
            layer(acts[(layer.k, m)])
    torch.cuda.synchronize()
    for layer, m in layers:
        log(f"[counter pass] K={layer.k} N={layer.n} M={m}: algorithmic bytes {w4a16_bytes(m, layer.k, layer.n)}")


# --------------------------------------------------------------------------------------------- CPU baseline

def cpu_baseline(budget_s: float = 15.0):
    """The reference's CPU-runnable path, restated by the oracle: unpack int4 -> (q - 8).to(bf16) * s -> torch.matmul,
    dequantisation included in every call (the reference path dequantises per call).  Bounded sample of the headline
    workload: whole steps (the 12 GEMMs) are repeated until about `budget_s` seconds of CPU work have been timed.
    Two smaller side figures ride along in the sample text: the same GEMMs with weights dequantised beforehand (matmul
    only), and the FP8 path (per-token quant + fp32 scaled matmul, the reference's `baseline_scaled_mm`) on one layer."""
    from oracle import fp8 as of
    from oracle import w4a16 as o
    threads = torch.get_num_threads()
    rng = np.random.default_rng(0)
    layers = []
    for (k, n) in LLAMA_SHAPES:
        qweight = rng.integers(-2 ** 31, 2 ** 31 - 1, size=(k // 8, n), dtype=np.int64).astype(np.int32)
        scales = (torch.randn(k // GROUP, n).abs() * 0.01 + 1e-3).to(torch.bfloat16)
        layers.append((k, n, qweight, scales))
    total_b, total_t, steps_done = 0, 0.0, 0
    while total_t < budget_s and steps_done < 50:
        for (k, n, qweight, scales) in layers:
            for m in DECODE_MS:
                a = torch.randn(m, k).to(torch.bfloat16)
                t0 = time.perf_counter()
                w = o.dequantize(o.unpack_rows(qweight, 4), scales, 8, GROUP)
                out = o.gemm_ref_like_reference(a, w)
                total_t += time.perf_counter() - t0
                total_b += w4a16_bytes(m, k, n)
                assert out.shape == (m, n)
        steps_done += 1
    log(f"[cpu baseline] {steps_done} step(s) of 12 GEMMs in {total_t:.1f} s on {threads} threads: {total_b / total_t / 1e9:.3f} GB/s")
    # matmul only (weights dequantised once, outside the timed region): one step
    pre_t, pre_b = 0.0, 0
    for (k, n, qweight, scales) in layers:
        w = o.dequantize(o.unpack_rows(qweight, 4), scales, 8, GROUP)
        for m in DECODE_MS:
            a = torch.randn(m, k).to(torch.bfloat16)
            t0 = time.perf_counter()
            o.gemm_ref_like_reference(a, w)
            pre_t += time.perf_counter() - t0
            pre_b += w4a16_bytes(m, k, n)
        del w
    log(f"[cpu baseline] matmul only, weights dequantised beforehand: {pre_b / pre_t / 1e9:.3f} GB/s (one step, {pre_t:.2f} s)")
    # FP8 path on the 4096 x 4096 layer, M = 16
    k, n, m = 4096, 4096, 16
    wq, ws = of.make_fp8_weight(n, k)
    a = torch.randn(m, k).to(torch.bfloat16)
    t0 = time.perf_counter()
    reps = 3
    for _ in range(reps):
        aq, sa = of.ref_dynamic_per_token_quant(a)
        of.scaled_mm_ref(aq, wq.t(), sa, ws, torch.bfloat16, None, order="baseline")
    f8_t = (time.perf_counter() - t0) / reps
    log(f"[cpu baseline] FP8 quant + scaled matmul, M={m} K={k} N={n}: {f8_t * 1e3:.1f} ms = {fp8_mm_bytes(m, k, n, False) / f8_t / 1e9:.3f} GB/s")
    return dict(value=round(total_b / total_t / 1e9, 4), unit="GB/s", cores=threads, kind="port",
                sample=f"{steps_done} full step(s) of the headline workload (12 GEMMs each) through the oracle: unpack + "
                       f"dequantise (bf16) + torch.matmul per call, {total_t:.1f} s of CPU time; side figures: matmul only "
                       f"with pre-dequantised weights {pre_b / pre_t / 1e9:.3f} GB/s (one step); FP8 per-token quant + "
                       f"scaled matmul at M={m}, {k}x{n}: {fp8_mm_bytes(m, k, n, False) / f8_t / 1e9:.3f} GB/s")


# --------------------------------------------------------------------------------------------- output

MAX_LINE_BYTES = 4096


def final_line(record: dict) -> str:
    """The one JSON line for stdout: the headline record without the per-section tables, at most MAX_LINE_BYTES long so
    that a reader who keeps only the tail of stdout still gets all of it.  Over the limit, the free-text fields are
    shortened first and the compact matrix-core rows dropped last; the headline, `roofline` and `cpu_baseline` stay."""
    rec = {k: v for k, v in record.items() if k != "extra"}
    line = json.dumps(rec, separators=(",", ":"))
    if len(line) > MAX_LINE_BYTES and isinstance(rec.get("cpu_baseline"), dict):
        rec["cpu_baseline"] = dict(rec["cpu_baseline"], sample=str(rec["cpu_baseline"].get("sample", ""))[:200])
        line = json.dumps(rec, separators=(",", ":"))
    if len(line) > MAX_LINE_BYTES:
        rec.pop("roofline_mfma", None)
        line = json.dumps(rec, separators=(",", ":"))
    assert len(line) <= MAX_LINE_BYTES and "\n" not in line
    return line


def write_extra(extra: dict, path: str | None = None) -> None:
    """The per-section tables (per-shape decode, prefill, FP8, vendor library, ...) go to a side file, never to stdout."""
    path = path or os.path.join(os.path.dirname(os.path.abspath(__file__)), "gpurun_out", "bench_extra.json")
    try:
        os.makedirs(os.path.dirname(path), exist_ok=True)
        with open(path, "w") as f:
            json.dump(extra, f, indent=1)
        log(f"[extra] per-section tables written to {path}")
    except OSError as e:
        log(f"[extra] not written ({e})")


# --------------------------------------------------------------------------------------------- main

def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-extra", action="store_true", help="skip the prefill / FP8 sections")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--mfma-pass", action="store_true",
                    help="for `rocprofv3 --pmc`: three eager passes of [vendor bf16 GEMM 4096^3, W4A16 and FP8 GEMMs at M = 4096], no timing")
    ap.add_argument("--sections", default="", help="comma-separated subset of the extra sections to run (default: all)")
    ap.add_argument("--weight-walk-probe", action="store_true",
                    help="run the weight access pattern probe (bench-only library) and print its table; no product timing")
    ap.add_argument("--mix-probe", action="store_true",
                    help="run the matrix-core instruction-mix probe (bench-only library) and print its table; no product timing")
    ap.add_argument("--counter-pass", action="store_true",
                    help="for `rocprofv3 --pmc`: three eager passes of [256 MiB device copy, the 12 headline GEMMs], no timing")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures ONE GPU (the quantized-linear path has no cross-GPU step); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from vllm_amd import _lib
    _lib.load()      # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.weight_walk_probe:
        print(json.dumps(weight_walk_probe(dev), indent=1))
        return
    if args.mix_probe:
        print(json.dumps(mix_probe(dev), indent=1))
        return
    if args.counter_pass:
        counter_pass(dev)
        return
    if args.mfma_pass:
        mfma_pass(dev)
        return
    sec, step_bytes, sets, acts = headline(dev, args.steps, args.warmup)
    value = step_bytes / sec / 1e9
    launches = len(LLAMA_SHAPES) * len(DECODE_MS)
    log(f"[headline] {sec * 1e6:.1f} us/step, {value:.0f} GB/s = {100 * value / HBM_PEAK_GBS:.1f}% of HBM peak")
    extra = {}
    try:
        extra["decode_per_shape"] = per_shape_decode(dev, sets, acts)
    except Exception as e:   # extras never invalidate the headline
        log(f"[decode per shape] failed: {e}")
    del sets
    torch.cuda.empty_cache()
    practical = None
    try:
        extra["stream_read_ceiling"] = stream_ceiling_section(dev)
        t_floor = len(DECODE_MS) * sum(r["us"] for r in extra["stream_read_ceiling"]) * 1e-6
        practical = step_bytes / t_floor / 1e9
        log(f"[read ceiling] 12 reads of the headline layers: {t_floor * 1e6:.1f} us -> practical ceiling {practical:.0f} GB/s; "
            f"the headline is at {100 * value / practical:.1f}% of it")
    except Exception as e:
        log(f"[read ceiling] failed: {e}")
    torch.cuda.empty_cache()
    if not args.no_extra:
        for name, fn in (("prefill", prefill_section), ("fp8", fp8_section), ("fused_norm_quant", fused_norm_quant_section),
                         ("variants", variants_section),
                         ("vendor_ceiling", vendor_ceiling_section),
                         ("vendor_small_m", vendor_small_m_section),
                         ("operand_toggle", operand_toggle_section),
                         ("host_overhead", host_overhead_section),
                         ("medium_m", medium_m_section),
                         ("decode_step", decode_step_section)):
            if args.sections and name not in args.sections.split(","):
                continue
            try:
                extra[name] = fn(dev)
            except Exception as e:
                log(f"[{name}] failed: {e}")
            torch.cuda.empty_cache()
    cpu = None if args.no_cpu else cpu_baseline()

    out = {
        "metric": "W4A16 decode GEMM effective HBM bandwidth (Llama-3-8B shapes, M in {1,4,16})",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "BASELINE.json configs[1]: decode W4A16 GEMMs, (K,N) in {(4096,6144),(4096,4096),(4096,28672),"
                               "(14336,4096)} x M in {1,4,16}, group 128, symmetric int4, bf16 act, fp32 acc; one step = "
                               "12 GEMMs in a HIP graph, weights cold (650 MB cycling)",
                   "launches_per_step": launches},
        "roofline": {"bound": "hbm", "kernel": "vaq::w4a16_decode2_kernel", "achieved": round(value, 2), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(value / HBM_PEAK_GBS, 4),
                     "traffic": int(MEASURED_TRAFFIC_PER_ALGORITHMIC_BYTE * step_bytes / launches),
                     "avg_launch_us": round(sec * 1e6 / launches, 3),
                     "algorithmic_bytes_per_launch": step_bytes // launches,
                     # what a read-only kernel reaches on the same layers in the same kind of graph (cold buffers)
                     "practical_peak": None if practical is None else round(practical, 1),
                     "practical_frac": None if practical is None else round(value / practical, 4)},
        "roofline_mfma": roofline_mfma(extra),
        "cpu_baseline": cpu,
    }
    write_extra(extra)
    print(final_line(out))


if __name__ == "__main__":
    main()
