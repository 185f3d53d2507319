#!/usr/bin/env python3
"""Decode throughput of the int8 (w8a32) Qwen2-1.5B-shaped decoder on one
MI355X, next to the CPU oracle timed on the same host.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
    python bench.py --workload gemv|mlp|prefill|llama8b|kvdiscard|w4a16|model_abi|sampler|quantize   (the other configurations)

A step is one greedy decode step (one token) at batch 1 with the KV cache
already holding 1024 positions; weights, KV cache and activations are resident
in HBM before the timed region; each step's argmax feeds the next step on the
device.  Prints one JSON line.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

# The CPU baseline runs OpenMP loops: pin its threads to neighbouring cores like
# the reference's own runs do (docs/Runtime.md:192 leaves the thread count to
# OMP_NUM_THREADS).  Must be in the environment before any OpenMP runtime loads.
# Only when the baseline will run: the binding also pins the process's first
# thread, and every helper thread a profiler starts inherits that.
OMP_BINDING = {"OMP_PROC_BIND": "close", "OMP_PLACES": "cores"}
if "--no-cpu-baseline" not in sys.argv:
    for _k, _v in OMP_BINDING.items():
        os.environ.setdefault(_k, _v)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth
CONTEXT = 1024
GATE_UP_KERNEL = "gemv_w8a32_digits_kernel<1, 2, 1, 3, false>"
TRAFFIC_PROFILE = "profiles/decode_kernels_hbm_traffic.md"


def gate_up_traffic(collecting: bool = False):
    """HBM bytes per launch of the dominant kernel as the counter summary under
    profiles/ records them (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a
    copy of known size): a counter reading, not something this script can
    measure live.  A summary that was taken for another kernel is refused --
    except in the run that collects the counters for a new one (`collecting`,
    the --calibrate-copy form), which reports no figure instead."""
    import re

    path = ROOT / TRAFFIC_PROFILE
    if not path.exists():
        return None, f"{TRAFFIC_PROFILE} not found"
    m = re.search(r"gate\|up GEMV \(`([^`]+)`\) per launch:.*?=\s*([0-9,]+) B against",
                  path.read_text(), re.S)
    if not m:
        raise SystemExit(f"bench.py: no per-launch traffic line in {TRAFFIC_PROFILE}")
    if m.group(1) != GATE_UP_KERNEL:
        why = (f"{TRAFFIC_PROFILE} holds the counters of `{m.group(1)}`, but the dominant "
               f"kernel is `{GATE_UP_KERNEL}`: take the counters again")
        if not collecting:
            raise SystemExit("bench.py: " + why)
        return None, why
    return int(m.group(2).replace(",", "")), TRAFFIC_PROFILE


TRACE_PROFILE = "profiles/decode_step_qwen2_1p5b_ctx1024_kernel_trace.md"


def gate_up_rocprof_us():
    """Average duration of the dominant kernel in the timed replay of the loop
    below, as rocprofv3's kernel trace of this same command recorded it (the
    summary under profiles/): the second clock on `roofline.avg_launch_us`, so
    that the fraction can be recomputed from the line alone.  None when the
    summary is missing or was taken for another kernel."""
    import re

    path = ROOT / TRACE_PROFILE
    if not path.exists():
        return None, f"{TRACE_PROFILE} not found"
    text = path.read_text()
    m = re.search(r"## Dominant kernel: `([^`]+)`", text)
    t = re.search(r"timed replay of the roofline loop.*?average ([0-9.]+) us", text, re.S)
    if not m or not t:
        return None, f"no dominant-kernel figures in {TRACE_PROFILE}"
    if m.group(1) != GATE_UP_KERNEL:
        return None, f"{TRACE_PROFILE} was taken for `{m.group(1)}`"
    return float(t.group(1)), TRACE_PROFILE


def gate_up_bytes(hidden: int, inter: int) -> int:
    """Algorithmic bytes of one fused RMSNorm + gate|up GEMV + SiLU*mul launch:
    two int8 matrices, their scales, the activation row, the norm weight and
    the output row."""
    return 2 * hidden * inter + 2 * 4 * inter + 4 * hidden + 4 * hidden + 4 * inter


def decode_step_bytes(shape, ctx: int) -> int:
    """Algorithmic bytes of one decode step at context `ctx` (rows 0..ctx read)."""
    H, I, V, L = shape.hidden, shape.inter, shape.vocab, shape.layers
    QN, KVN = shape.heads * shape.head_dim, shape.kv_heads * shape.head_dim
    w = L * (H * (QN + 2 * KVN) + QN * H + 3 * H * I) + H * V
    scales = 4 * (L * (QN + 2 * KVN + H + 2 * I + H) + V)
    kv = L * 2 * KVN * 4 * (ctx + 1)
    norms = 4 * H * (2 * L + 1)
    return w + scales + kv + norms + 4 * H + 4 * V


def time_gate_up(bh, shape, sess_stream, layers, iters, use_graph=True):
    """Average duration of the dominant kernel (fused gate|up GEMV), launched
    back to back over `layers` distinct weight sets (more than the 256 MB
    last-level cache holds) from a replayed hipGraph, as the decode step
    launches it, timed with HIP events on the launch stream."""
    import torch
    from buddy_mlir_amd import check, ops, synthetic

    H, I = shape.hidden, shape.inter
    sets = []
    for i in range(layers):
        qg, sg = synthetic.quantized_linear(H, I, 9000 + 2 * i)
        qu, su = synthetic.quantized_linear(H, I, 9001 + 2 * i)
        sets.append((ops.pack_w8(qg), sg, ops.pack_w8(qu), su))
        del qg, qu
    x = torch.randn((1, H), device="cuda")
    w = torch.ones(H, device="cuda")
    h = torch.empty((1, I), device="cuda")
    descs = []
    for pg, sg, pu, su in sets:
        d = ops.LinearDesc()
        d.A, d.lda, d.W0, d.scale0, d.W1, d.scale1 = (x.data_ptr(), H, pg.data_ptr(),
                                                     sg.data_ptr(), pu.data_ptr(),
                                                     su.data_ptr())
        d.bias, d.norm_w, d.norm_eps = None, w.data_ptr(), shape.rms_eps
        d.C, d.ldc, d.M, d.K, d.N, d.epilogue = h.data_ptr(), I, 1, H, I, 2
        descs.append(d)
    torch.cuda.synchronize()
    stream = torch.cuda.ExternalStream(sess_stream)
    for d in descs:
        check(bh.buddy_hip_linear_w8a32(ctypes.byref(d), sess_stream))
    stream.synchronize()

    def enqueue():
        for i in range(iters):
            bh.buddy_hip_linear_w8a32(ctypes.byref(descs[i % layers]), sess_stream)

    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    if not use_graph:  # plain stream launches (what a per-dispatch counter run needs)
        e0.record(stream)
        enqueue()
        e1.record(stream)
        e1.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / iters
    # the decode step launches this kernel from a replayed hipGraph: time it the
    # same way, `iters` launches per replay
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        enqueue()
    with torch.cuda.stream(stream):
        graph.replay()
        stream.synchronize()
        e0.record(stream)
        graph.replay()
        e1.record(stream)
    e1.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / iters


def cpu_baseline(shape, host, first_token, budget_s=12.0, max_steps=4096):
    """The CPU oracle (OpenMP restatement of the reference's kernels) on the
    same weights: whole decode steps at context 1024.. until ~budget_s is used
    (positions cycle inside the cache's spare room, so context stays ~1024)."""
    import oracle_lib

    oracle = oracle_lib.load()
    om = oracle_lib.model_from_host(oracle, shape, host)
    kv = host["kv"]
    tok = first_token
    tok, _ = om.decode_step(tok, CONTEXT, kv)  # warm-up (page-in, thread start)
    spare = max(1, shape.max_len - CONTEXT - 2)
    t0 = time.perf_counter()
    n = 0
    while n < max_steps:
        tok, _ = om.decode_step(tok, CONTEXT + 1 + n % spare, kv)
        n += 1
        if time.perf_counter() - t0 > budget_s:
            break
    dt = time.perf_counter() - t0
    return {"value": n / dt, "unit": "tokens/s", "cores": oracle.num_threads(),
            "kind": "port",
            "sample": f"{n} decode steps at context {CONTEXT}, same weights, "
                      f"{dt:.1f} s of CPU time",
            "omp": {k: os.environ.get(k) for k in OMP_BINDING}}


# ---------------------------------------------------------------------------
# The other measured configurations (one JSON line each, same field names).
# ---------------------------------------------------------------------------
MFMA_I8_PEAK_TOPS = 5000.0   # dense int8, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16


def _time_launches(fn, iters, warm=8):
    """Average seconds per call of fn(i), launched back to back on torch's
    current stream and timed with HIP events on that stream."""
    import torch

    for i in range(warm):
        fn(i)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for i in range(iters):
        fn(i)
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / iters


def _time_launches_graph(make_fn, iters, warm=8):
    """The same for launches short enough for the host to fall behind a plain
    stream: `iters` calls of fn(i) are recorded into a hipGraph once and the
    replay is timed.  make_fn(stream_handle) returns fn."""
    import torch

    stream = torch.cuda.Stream()
    fn = make_fn(stream.cuda_stream)
    torch.cuda.synchronize()
    for i in range(warm):
        fn(i)
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        for i in range(iters):
            fn(i)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with torch.cuda.stream(stream):
        graph.replay()
        stream.synchronize()
        e0.record(stream)
        graph.replay()
        e1.record(stream)
    e1.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / iters


def _random_packed(K, N, copies):
    """`copies` wave-tile buffers of random int8 (timing only: any bytes do)."""
    import torch

    import buddy_mlir_amd as bma

    nbytes = bma.lib().buddy_hip_w8_packed_bytes(K, N)
    return [torch.randint(-127, 128, (nbytes,), dtype=torch.int8, device="cuda")
            for _ in range(copies)]


def _linear_fn(bh, sets, x, out, K, N, M, dual, norm_w, epilogue):
    """Returns fn(i) that launches one fused linear on weight set i % len(sets)."""
    import torch

    from buddy_mlir_amd import ops

    scale = torch.full((N,), 1e-3, device="cuda")
    descs = []
    for w in sets:
        d = ops.LinearDesc()
        d.A, d.lda = x.data_ptr(), K
        d.W0, d.scale0 = w[0].data_ptr(), scale.data_ptr()
        if dual:
            d.W1, d.scale1 = w[1].data_ptr(), scale.data_ptr()
        d.bias, d.norm_w, d.norm_eps = None, (norm_w.data_ptr() if norm_w is not None else None), 1e-6
        d.C, d.ldc, d.M, d.K, d.N, d.epilogue = out.data_ptr(), N, M, K, N, epilogue
        descs.append(d)
    stream = torch.cuda.current_stream().cuda_stream
    keep = (scale, descs)

    def fn(i, keep=keep):
        rc = bh.buddy_hip_linear_w8a32(ctypes.byref(descs[i % len(descs)]), stream)
        if rc:
            raise RuntimeError("linear_w8a32 failed")
    return fn


def _linear_bytes(K, N, M, dual, norm):
    return (2 if dual else 1) * (K * N + 4 * N) + 4 * M * (K + N) + (4 * K if norm else 0)


def cpu_baseline_gemv(K, N, budget_s=6.0, copies=8):
    """The CPU oracle's int8 GEMV on this shape, weights rotated over `copies`
    matrices (110 MB: beyond the host's last-level cache), ~budget_s each for the
    reference's plain row-major layout (stride-N inner loop,
    DequantMatMulVectorizationDecode.cpp:259-283) and for the same loop over the
    reference's packed-panel order applied to int8, so that the GPU is not
    compared with the slower layout only."""
    import numpy as np

    import oracle_lib

    oracle = oracle_lib.load()
    rng = np.random.default_rng(1)
    x = rng.standard_normal(K).astype(np.float32)
    scale = np.full(N, 1e-3, np.float32)
    plain = [rng.integers(-127, 128, (K, N), dtype=np.int8) for _ in range(copies)]
    panels = [np.ascontiguousarray(w.reshape(K, N // 32, 32).transpose(1, 0, 2)) for w in plain]
    by = K * N + 4 * N + 4 * (K + N)
    out = {}
    for name, fn in (("plain_row_major", lambda i: oracle.dequant_gemv(x, plain[i], scale)),
                     ("packed_panels", lambda i: oracle.dequant_gemv_panels(x, panels[i], scale, K, N))):
        fn(0)
        t0 = time.perf_counter()
        n = 0
        while time.perf_counter() - t0 < budget_s:
            fn(n % copies)
            n += 1
        dt = (time.perf_counter() - t0) / n
        out[name] = {"us": dt * 1e6, "gbps": by / dt / 1e9, "calls": n}
    return {"value": out["plain_row_major"]["gbps"], "unit": "GB/s",
            "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{out['plain_row_major']['calls']} + {out['packed_panels']['calls']} "
                      f"GEMVs {K} -> {N} over {copies} rotating matrices, {budget_s:.0f} s each",
            "plain_row_major": out["plain_row_major"], "packed_panels": out["packed_panels"],
            "omp": {k: os.environ.get(k) for k in OMP_BINDING}}


def bench_gemv(bh, args):
    """configs[0]: one int8 GEMV 1536 -> 8960 at M = 1, weights rotated over 48
    copies (HBM-cold, 660 MB) and over one copy (cache-warm)."""
    import torch

    K, N = 1536, 8960
    x = torch.randn((1, K), device="cuda")
    y = torch.empty((1, N), device="cuda")
    by = _linear_bytes(K, N, 1, False, False)
    res = {}
    for name, copies in (("hbm_cold", 48), ("cache_warm", 1)):
        sets = [(w,) for w in _random_packed(K, N, copies)]
        fn = _linear_fn(bh, sets, x, y, K, N, 1, False, None, 0)
        t = _time_launches(fn, 960)
        res[name] = {"us": t * 1e6, "gbps": by / t / 1e9, "frac": by / t / 1e9 / HBM_PEAK_GBPS}
        del sets
    # the same shape through the other GEMV kernels of the path, weights rotated
    # over HBM-cold copies: int8 activations with exact int32 sums (w8a8), and the
    # f32 GEMV in row-major and in the reference's packed-panel layout
    packed = _random_packed(K, N, 24)
    wscale = torch.full((N,), 1e-3, device="cuda")
    ws_bytes = bh.buddy_hip_w8a8_workspace_bytes(1, K)
    ws = torch.empty((ws_bytes,), dtype=torch.int8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream

    def make_w8a8(stream):
        def w8a8(i):
            if bh.buddy_hip_w8a8_matmul(x.data_ptr(), packed[i % 24].data_ptr(),
                                        wscale.data_ptr(), y.data_ptr(), None, 1, K, N,
                                        ws.data_ptr(), ws_bytes, stream):
                raise RuntimeError("w8a8_matmul failed")
        return w8a8
    # (two short launches per call: recorded into a graph so that the host's
    # launch rate does not enter)
    t8 = _time_launches_graph(make_w8a8, 240)
    by8 = K * N + 4 * N + 4 * (K + N)
    res["w8a8_int32_sums"] = {"us": t8 * 1e6, "gbps": by8 / t8 / 1e9,
                              "frac": by8 / t8 / 1e9 / HBM_PEAK_GBPS,
                              "note": "two launches: activation quantisation, then the GEMV"}
    del packed
    Bf = [torch.randn((K, N), device="cuda") for _ in range(12)]  # 660 MB of f32
    byf = 4 * K * N + 4 * (K + N)

    def f32_plain(i):
        if bh.buddy_hip_gemv_f32(x.data_ptr(), Bf[i % 12].data_ptr(), None, y.data_ptr(), K, N,
                                 0, stream):
            raise RuntimeError("gemv_f32 failed")
    tf = _time_launches(f32_plain, 240)
    res["f32_row_major"] = {"us": tf * 1e6, "gbps": byf / tf / 1e9,
                            "frac": byf / tf / 1e9 / HBM_PEAK_GBPS}
    Pf = [torch.empty_like(b) for b in Bf]
    for b_, p_ in zip(Bf, Pf):
        if bh.buddy_hip_pack_panels_f32(b_.data_ptr(), K, N, 32, p_.data_ptr(), stream):
            raise RuntimeError("pack_panels_f32 failed")
    del Bf

    def f32_panels(i):
        if bh.buddy_hip_gemv_f32_panels(x.data_ptr(), Pf[i % 12].data_ptr(), y.data_ptr(), K, N,
                                        0, stream):
            raise RuntimeError("gemv_f32_panels failed")
    tp = _time_launches(f32_panels, 240)
    res["f32_reference_panels"] = {"us": tp * 1e6, "gbps": byf / tp / 1e9,
                                   "frac": byf / tp / 1e9 / HBM_PEAK_GBPS}
    del Pf
    t = res["hbm_cold"]["us"] * 1e-6
    cpu = None if args.no_cpu_baseline else cpu_baseline_gemv(K, N)
    return {
        **({"cpu_baseline": cpu} if cpu else {}),
        "metric": "int8_gemv_hbm_gbps", "value": res["hbm_cold"]["gbps"], "unit": "GB/s",
        "n_gpus": 1, "steps": 960, "warmup": 8, "ms_per_step": t * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "single int8 weight-only GEMV x[1,1536] . W[1536,8960] "
                               "(BASELINE configs[0]), 48 rotating weight copies"},
        "detail": res,
        "roofline": {"kernel": "gemv_w8a32_digits_kernel<1, 0, 0, 3, false>", "bound": "hbm",
                     "achieved": res["hbm_cold"]["gbps"], "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": res["hbm_cold"]["frac"],
                     "algorithmic_bytes_per_launch": by, "avg_launch_us": t * 1e6,
                     "traffic": None},
    }


def bench_mlp(bh, args):
    """configs[1]: h = SiLU(x G) * (x U), y = h D at M in {1, 4, 16} (--mlp-rows): one call of
    buddy_hip_mlp_block_w8a32 (two launches: fused gate|up, then down), 12
    rotating weight sets (496 MB)."""
    import torch

    H, I = 1536, 8960
    gu = _random_packed(H, I, 24)
    dn = _random_packed(I, H, 12)
    res = {}
    rows = [int(v) for v in args.mlp_rows.split(",")]
    if any(M < 1 or M > 16 for M in rows) or 1 not in rows:
        raise SystemExit("--mlp-rows: row counts from 1 to 16, 1 among them")
    for M in rows:
        x = torch.randn((M, H), device="cuda")
        h = torch.empty((M, I), device="cuda")
        y = torch.zeros((M, H), device="cuda")
        f1 = _linear_fn(bh, [(gu[2 * i], gu[2 * i + 1]) for i in range(12)], x, h, H, I, M, True, None, 2)
        f2 = _linear_fn(bh, [(w,) for w in dn], h, y, I, H, M, False, None, 0)

        def two_calls(i):
            f1(i)
            f2(i)
        # the block as one call (buddy_hip_mlp_block_w8a32)
        from buddy_mlir_amd import ops
        sc_i = torch.full((I,), 1e-3, device="cuda")
        sc_h = torch.full((H,), 1e-3, device="cuda")
        stream = torch.cuda.current_stream().cuda_stream
        descs = [ops.mlp_block_desc(x, gu[2 * i], sc_i, gu[2 * i + 1], sc_i, dn[i], sc_h, y, H, I)
                 for i in range(12)]

        def block(i):
            if bh.buddy_hip_mlp_block_w8a32(ctypes.byref(descs[i % 12][0]), stream):
                raise RuntimeError("mlp_block_w8a32 failed")
        t = _time_launches(block, 480)
        # three int8 matrices, their scales, M rows in and M rows out
        by = 3 * H * I + 4 * (2 * I + H) + 4 * M * 2 * H
        res[f"M={M}"] = {"us": t * 1e6, "gbps": by / t / 1e9,
                         "frac": by / t / 1e9 / HBM_PEAK_GBPS,
                         # the same two matmuls as two buddy_hip_linear_w8a32 calls (f32
                         # rows between them), and each of those on its own
                         "two_linear_calls_us": _time_launches(two_calls, 480) * 1e6,
                         "gate_up_us": _time_launches(f1, 240) * 1e6,
                         "down_us": _time_launches(f2, 240) * 1e6}
    t = res["M=1"]["us"] * 1e-6
    return {
        "metric": "int8_mlp_hbm_gbps", "value": res["M=1"]["gbps"], "unit": "GB/s",
        "n_gpus": 1, "steps": 480, "warmup": 8, "ms_per_step": t * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "int8 MLP block 1536 -> 8960 -> 1536 at M in {1,4,16} "
                               "(BASELINE configs[1]); value is M=1"},
        "detail": res,
        "roofline": {"kernel": "gate|up + down GEMV pair", "bound": "hbm",
                     "achieved": res["M=1"]["gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": res["M=1"]["frac"], "traffic": None},
    }


def bench_prefill(bh, args):
    """configs[3]: a 512-token prompt through all 28 layers (causal GQA
    attention included).  The matmuls multiply the int8 weights as they are on
    the int8 matrix cores, the f32 activations carried as three int8 digit
    planes (23 bits below each row's maximum); the two bf16 modes (one term =
    the configuration's wording, three terms = every f32 bit) are timed beside
    it."""
    import numpy as np
    import torch

    from buddy_mlir_amd import synthetic
    from buddy_mlir_amd.session import Shape

    M = 512
    shape = Shape(max_len=M + 64)
    sess, _ = synthetic.build_session(shape, context=0)
    toks = synthetic.first_tokens(shape, M)
    H, I, L = shape.hidden, shape.inter, shape.layers
    QN, KVN = shape.heads * shape.head_dim, shape.kv_heads * shape.head_dim
    gemm_flop = 2 * M * L * (H * (QN + 2 * KVN) + QN * H + 3 * H * I)
    attn_flop = L * shape.heads * M * M * shape.head_dim * 2 * 2 // 2
    res = {}
    n = max(1, min(args.steps, 20))
    for name, precision, peak in (("i8_3digit", "digits", MFMA_I8_PEAK_TOPS),
                                  ("i8_2digit", "digits2", MFMA_I8_PEAK_TOPS),
                                  ("bf16_1term", "bf16", MFMA_BF16_PEAK_TFLOPS),
                                  ("bf16_3term_exact", "exact", MFMA_BF16_PEAK_TFLOPS)):
        for _ in range(max(1, args.warmup)):
            sess.prefill(toks, 0, want_logits=False, precision=precision)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            sess.prefill(toks, 0, want_logits=False, precision=precision)
        torch.cuda.synchronize()
        t = (time.perf_counter() - t0) / n
        res[name] = {"ms": t * 1e3, "tokens_per_s": M / t,
                     "gemm_tflops": gemm_flop / t / 1e12,
                     "mfma_frac": gemm_flop / t / 1e12 / peak}
    sess.close()
    # the w8a8 matmul (int8 activations, exact int32 sums) at 512 rows of the two
    # MLP shapes: quantisation (two launches) + one int8 plane through the same
    # matrix-core kernel
    for K, N in ((H, I), (I, H)):
        x = torch.randn((M, K), device="cuda")
        packed = _random_packed(K, N, 4)
        wscale = torch.full((N,), 1e-3, device="cuda")
        y = torch.empty((M, N), device="cuda")
        nb = bh.buddy_hip_w8a8_workspace_bytes(M, K)
        ws = torch.empty((nb,), dtype=torch.int8, device="cuda")
        stream = torch.cuda.current_stream().cuda_stream

        def w8a8(i):
            if bh.buddy_hip_w8a8_matmul(x.data_ptr(), packed[i % 4].data_ptr(), wscale.data_ptr(),
                                        y.data_ptr(), None, M, K, N, ws.data_ptr(), nb, stream):
                raise RuntimeError("w8a8_matmul failed")
        t8 = _time_launches(w8a8, 80)
        res[f"w8a8_512x{K}x{N}"] = {"us": t8 * 1e6, "tops": 2 * M * K * N / t8 / 1e12,
                                    "mfma_frac": 2 * M * K * N / t8 / 1e12 / MFMA_I8_PEAK_TOPS}
    t = res["i8_3digit"]["ms"] * 1e-3
    return {
        "metric": "prefill_tokens_per_s", "value": M / t, "unit": "tokens/s",
        "n_gpus": 1, "steps": n, "warmup": max(1, args.warmup), "ms_per_step": t * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "prefill of 512 tokens, Qwen2-1.5B shape, 28 layers "
                               "(BASELINE configs[3]); value is the int8 digit-plane mode; "
                               "time includes attention, norms and the last-row lm_head"},
        "detail": res, "gemm_flop": gemm_flop, "attention_flop": attn_flop,
        # algorithmic flops 2 M K N (each digit plane is not counted again)
        # over the time of the whole pass, against the dense int8 peak
        "roofline": {"kernel": "gemm_w8_i8_wide_kernel<3, 4, 5> (gate, up), <3, 4, 4> (down), "
                               "gemm_w8_i8_kernel<3> (q|k|v, o)",
                     "bound": "mfma", "achieved": res["i8_3digit"]["gemm_tflops"],
                     "peak": MFMA_I8_PEAK_TOPS, "unit": "TFLOP/s",
                     "frac": res["i8_3digit"]["mfma_frac"], "traffic": None},
    }


def bench_kvdiscard(bh, args):
    """KV-cache overflow at the Qwen2-1.5B shape: 56 cache tensors
    [2, 1088, 128] f32 full to the last row, keep 4 tokens, discard 256, move
    and re-rotate the other 828 rows, clear the rest."""
    import numpy as np
    import torch

    from buddy_mlir_amd import synthetic

    heads, L, D, n = 2, 1088, 128, 56
    keep, discard, count = 4, 256, 1088
    tensors = [torch.randn((heads, L, D), device="cuda") for _ in range(n)]
    ptrs = (ctypes.c_void_p * n)(*[t.data_ptr() for t in tensors])
    f = np.ascontiguousarray(synthetic.inv_freq(D).cpu().numpy(), np.float32)
    stream = torch.cuda.current_stream().cuda_stream

    def fn(i):
        rc = bh.buddy_hip_kv_discard(ptrs, n, heads, L, D, keep, discard, count,
                                     f.ctypes.data, stream)
        if rc:
            raise RuntimeError("kv_discard failed")
    t = _time_launches(fn, 50, warm=3)
    tail = count - keep - discard
    by = n * heads * D * 4 * (2 * tail + (L - keep - tail))  # read + write tail, clear rest
    # the same on the host: the reference's own discardKVCache + adjustKeyCacheRope
    # (KVCacheManager.h compiled as oracle/_ref) where that build exists, else the
    # restatement
    cpu = None
    if not args.no_cpu_baseline:
        import time

        sys.path.insert(0, str(ROOT / "tests"))
        import oracle_lib

        host = [x.cpu().numpy() for x in tensors]
        ref = oracle_lib.load_reference_runtime()
        reps = 5
        t0 = time.perf_counter()
        for _ in range(reps):
            if ref is not None:
                ref.kv_discard(host, keep, discard, count)
                ref.kv_adjust_rope(host, keep, discard, count, f)
            else:
                o = oracle_lib.load()
                for j in range(n):
                    _, host[j] = o.kv_discard(host[j], keep, discard, count)
                    if j % 2 == 0:
                        host[j] = o.kv_adjust_rope(host[j], keep, discard, count, f)
        t_cpu = (time.perf_counter() - t0) / reps
        cpu = {"value": by / t_cpu / 1e9, "unit": "GB/s", "cores": 1,
               "kind": "reference" if ref is not None else "port",
               "sample": f"{reps} calls on 56 host tensors [2,1088,128], {t_cpu * 1e3:.2f} ms each"}
    out = {
        "metric": "kv_discard_hbm_gbps", "value": by / t / 1e9, "unit": "GB/s",
        "n_gpus": 1, "steps": 50, "warmup": 3, "ms_per_step": t * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "KV-cache discard + key re-rotation, 56 tensors [2,1088,128], "
                               "keep 4 / discard 256 / count 1088"},
        "roofline": {"kernel": "kv_discard_kernel", "bound": "hbm",
                     "achieved": by / t / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": by / t / 1e9 / HBM_PEAK_GBPS,
                     "algorithmic_bytes_per_launch": by, "avg_launch_us": t * 1e6,
                     "traffic": None},
    }
    if cpu:
        out["cpu_baseline"] = cpu
    return out


def bench_quantize(bh, args):
    """The import-time pair: per-output-channel int8 quantisation of an f32
    matrix (amax pass + quantise pass) and the repacking of the int8 matrix into
    wave tiles, at the gate/up shape.  CPU figure: the restated quantiser."""
    import time

    import torch

    from buddy_mlir_amd import ops

    K, N = 1536, 8960
    ws = [torch.randn((K, N), device="cuda") * 0.02 for _ in range(8)]
    qs = [ops.quantize_w8(w)[0] for w in ws]
    # outputs allocated once: the loop times the kernels, not the allocator
    q_out = torch.empty((K, N), dtype=torch.int8, device="cuda")
    s_out = torch.empty((N,), dtype=torch.float32, device="cuda")
    p_out = torch.empty_like(ops.pack_w8(qs[0]))
    stream = torch.cuda.current_stream().cuda_stream

    def quantize(i):
        if bh.buddy_hip_quantize_w8(ws[i % 8].data_ptr(), K, N, q_out.data_ptr(),
                                    s_out.data_ptr(), stream):
            raise RuntimeError("quantize_w8 failed")

    def pack(i):
        if bh.buddy_hip_pack_w8(qs[i % 8].data_ptr(), K, N, p_out.data_ptr(), stream):
            raise RuntimeError("pack_w8 failed")

    tq = _time_launches(quantize, 40, warm=3)
    tp = _time_launches(pack, 40, warm=3)
    by_q, by_p = 9 * K * N, 2 * K * N  # f32 read twice + int8 write; int8 read + write
    out = {
        "metric": "quantize_hbm_gbps", "value": by_q / tq / 1e9, "unit": "GB/s",
        "n_gpus": 1, "steps": 40, "warmup": 3, "ms_per_step": tq * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32->int8",
        "data": "synthetic",
        "config": {"workload": "per-channel int8 quantisation of f32 W[1536,8960], and its "
                               "wave-tile packing"},
        "detail": {"quantize": {"us": tq * 1e6, "gbps": by_q / tq / 1e9,
                                "frac": by_q / tq / 1e9 / HBM_PEAK_GBPS},
                   "pack": {"us": tp * 1e6, "gbps": by_p / tp / 1e9,
                            "frac": by_p / tp / 1e9 / HBM_PEAK_GBPS}},
        "roofline": {"kernel": "colwise_absmax + finalize_scale + quantize", "bound": "hbm",
                     "achieved": by_q / tq / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": by_q / tq / 1e9 / HBM_PEAK_GBPS,
                     "algorithmic_bytes_per_launch": by_q, "avg_launch_us": tq * 1e6,
                     "traffic": None},
    }
    if not args.no_cpu_baseline:
        sys.path.insert(0, str(ROOT / "tests"))
        import oracle_lib

        o = oracle_lib.load()
        wh = ws[0].cpu().numpy()
        t0 = time.perf_counter()
        reps = 5
        for _ in range(reps):
            o.quantize_w8(wh)
        t_cpu = (time.perf_counter() - t0) / reps
        out["cpu_baseline"] = {"value": by_q / t_cpu / 1e9, "unit": "GB/s",
                               "cores": o.num_threads(), "kind": "port",
                               "sample": f"{reps} calls of the restated quantiser on the same "
                                         f"matrix, {t_cpu * 1e3:.1f} ms each"}
    return out


def bench_sampler(bh, args):
    """One sampled token from device logits of the Qwen2 vocabulary: penalty,
    temperature and top-40 on the device, the rest on the host.  The CPU figure
    is the restated reference sampler on logits copied back first, which is what
    a host sampler behind device logits costs."""
    import time

    import numpy as np
    import torch

    from buddy_mlir_amd.session import Sampler

    sys.path.insert(0, str(ROOT / "tests"))
    import oracle_lib

    vocab = 151936
    cfg = dict(temperature=0.8, top_k=40, top_p=0.95, min_p=0.05, repeat_penalty=1.1,
               repeat_last_n=64)
    logits = [torch.randn(vocab, device="cuda") * 3 for _ in range(8)]
    recent = list(np.random.default_rng(0).integers(0, vocab, 64))
    sampler = Sampler(seed=1, **cfg)
    iters = 200
    for i in range(8):
        sampler.sample(logits[i % 8], recent)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(iters):
        sampler.sample(logits[i % 8], recent)
    t = (time.perf_counter() - t0) / iters
    ref = oracle_lib.load_reference_runtime()  # the reference's own Sampler.h, where built
    if ref is not None:
        cpu, kind = ref.sampler(seed=1, **cfg), "reference"
    else:
        cpu, kind = oracle_lib.OracleSampler(oracle_lib.load(), seed=1, **cfg), "port"
    host = torch.empty(vocab, pin_memory=True)
    n_cpu = 40
    t0 = time.perf_counter()
    for i in range(n_cpu):
        host.copy_(logits[i % 8])
        cpu.sample(host.numpy(), recent)
    t_cpu = (time.perf_counter() - t0) / n_cpu
    by = vocab * 4
    return {
        "metric": "sampled_tokens_per_sec", "value": 1.0 / t, "unit": "samples/s",
        "n_gpus": 1, "steps": iters, "warmup": 8, "ms_per_step": t * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "sampler, vocabulary 151936, temperature 0.8 / top-K 40 / "
                               "top-P 0.95 / min-P 0.05 / penalty 1.1 over 64 ids; each call "
                               "synchronous (three launches, 328 B written to pinned host memory, host finish)"},
        "roofline": {"kernel": "sampler_keys_kernel + sampler_candidates_kernel + sampler_pick_kernel",
                     "bound": "hbm", "achieved": by / t / 1e9, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": by / t / 1e9 / HBM_PEAK_GBPS,
                     "algorithmic_bytes_per_launch": by, "avg_launch_us": t * 1e6,
                     "traffic": None,
                     "note": "latency-bound: 608 KB of logits, three short launches and a host "
                             "round trip; the call's wall time is used, not a kernel's"},
        "cpu_baseline": {"value": 1.0 / t_cpu, "unit": "samples/s", "cores": 1, "kind": kind,
                         "sample": f"{n_cpu} calls of the "
                                   + ("reference's own sampler (Sampler.h compiled as oracle/_ref)"
                                      if kind == "reference" else "restated reference sampler")
                                   + ", each after copying the 151936 logits to pinned host memory"},
    }


def bench_w4a16(bh, args):
    """The int4 weight-only decode GEMV at 1536 -> 8960, 8960 -> 1536 and (a
    Llama-3-8B gate matrix) 4096 -> 14336 over 24 weight copies, both kernels: the one that keeps the reference's order of f16
    operations (bit-exact, the default) and the opt-in streaming one (exact
    products, one rounding to f16).  `value` is the streaming kernel."""
    import torch

    res = {}
    for K, N in ((1536, 8960), (8960, 1536), (4096, 14336)):
        copies = 24
        packs = [torch.randint(-128, 128, (K, N // 2), dtype=torch.int8, device="cuda")
                 for _ in range(copies)]
        nt = bh.buddy_hip_w4_tiles_bytes(K, N)
        tiles = [torch.empty(nt, dtype=torch.int8, device="cuda") for _ in range(copies)]
        for p, t in zip(packs, tiles):
            if bh.buddy_hip_pack_w4_tiles(p.data_ptr(), K, N, t.data_ptr(), None):
                raise RuntimeError("pack_w4_tiles failed")
        torch.cuda.synchronize()
        a = torch.randn(K, device="cuda").half()
        sc = torch.full((N,), 0.01, device="cuda").half()
        c = torch.zeros(N, device="cuda").half()

        def chain(stream):
            def fn(i):
                if bh.buddy_hip_gemv_w4a16(a.data_ptr(), packs[i % copies].data_ptr(),
                                           sc.data_ptr(), c.data_ptr(), K, N, stream):
                    raise RuntimeError("gemv_w4a16 failed")
            return fn

        def fast(stream):
            def fn(i):
                if bh.buddy_hip_gemv_w4a16_fast(a.data_ptr(), tiles[i % copies].data_ptr(),
                                                sc.data_ptr(), c.data_ptr(), K, N, stream):
                    raise RuntimeError("gemv_w4a16_fast failed")
            return fn
        by = K * N // 2 + 2 * K + 2 * N + 4 * N
        for name, make in (("f16_chain", chain), ("fast", fast)):
            c.zero_()
            t = _time_launches_graph(make, 240)  # replayed hipGraph, as a decode step launches
            res[f"{K}->{N} {name}"] = {"us": t * 1e6, "gbps": by / t / 1e9,
                                       "frac": by / t / 1e9 / HBM_PEAK_GBPS, "bytes": by}
    r = res["1536->8960 fast"]
    return {
        "metric": "int4_gemv_hbm_gbps", "value": r["gbps"], "unit": "GB/s", "n_gpus": 1,
        "steps": 240, "warmup": 8, "ms_per_step": r["us"] * 1e-3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": "W4A16 decode GEMV 1536 -> 8960, the opt-in streaming kernel "
                               "(int4 weights widened to int8 in registers, f16 activations "
                               "as four int8 digit planes, exact int32 sums, f16 result); "
                               "detail also times the default kernel that keeps the "
                               "reference's f16 order, and 8960 -> 1536"},
        "detail": res,
        "roofline": {"kernel": "w4a16_fast_kernel", "bound": "hbm", "achieved": r["gbps"],
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": r["frac"],
                     "algorithmic_bytes_per_launch": r["bytes"], "avg_launch_us": r["us"],
                     "traffic": None},
    }


def bench_llama8b(bh, args):
    """configs[4]: the decode GEMVs of a Llama-3-8B-shaped step, 32 layers of
    distinct weights (q|k|v, o, gate|up fused, down) plus lm_head: 7.5 GB of int8
    streamed once per sweep, at M = 1 and M = 8."""
    import torch

    H, I, V, L = 4096, 14336, 128256, 32
    QKV = 4096 + 2 * 1024
    mats = []  # (name, K, N, dual, count)
    layers = []
    for _ in range(L):
        layers.append({
            "qkv": _random_packed(H, QKV, 1), "o": _random_packed(H, H, 1),
            "gu": _random_packed(H, I, 2), "down": _random_packed(I, H, 1)})
    lm = _random_packed(H, V, 1)
    res = {}
    for M in (1, 8):
        x = torch.randn((M, H), device="cuda")
        hbuf = torch.empty((M, I), device="cuda")
        qkv = torch.empty((M, QKV), device="cuda")
        y = torch.zeros((M, H), device="cuda")
        logits = torch.empty((M, V), device="cuda")
        nw = torch.ones(H, device="cuda") if M == 1 else None  # fused norm at M = 1
        f_qkv = _linear_fn(bh, [(l["qkv"][0],) for l in layers], x, qkv, H, QKV, M, False, nw, 0)
        f_o = _linear_fn(bh, [(l["o"][0],) for l in layers], x, y, H, H, M, False, None, 1)
        f_gu = _linear_fn(bh, [tuple(l["gu"]) for l in layers], x, hbuf, H, I, M, True, nw, 2)
        f_dn = _linear_fn(bh, [(l["down"][0],) for l in layers], hbuf, y, I, H, M, False, None, 1)
        f_lm = _linear_fn(bh, [(lm[0],)], x, logits, H, V, M, False, nw, 0)

        def sweep(_):
            for i in range(L):
                f_qkv(i)
                f_o(i)
                f_gu(i)
                f_dn(i)
            f_lm(0)
        t = _time_launches(sweep, 10, warm=2)
        by = (L * (_linear_bytes(H, QKV, M, False, M == 1) + _linear_bytes(H, H, M, False, False)
                   + _linear_bytes(H, I, M, True, M == 1) + _linear_bytes(I, H, M, False, False))
              + _linear_bytes(H, V, M, False, M == 1))
        per = {}
        for nm, f, k, n, dual in (("qkv", f_qkv, H, QKV, False), ("o", f_o, H, H, False),
                                  ("gate|up", f_gu, H, I, True), ("down", f_dn, I, H, False),
                                  ("lm_head", f_lm, H, V, False)):
            tt = _time_launches(f, 128)
            b = _linear_bytes(k, n, M, dual, False)
            per[nm] = {"us": tt * 1e6, "gbps": b / tt / 1e9, "frac": b / tt / 1e9 / HBM_PEAK_GBPS}
        res[f"M={M}"] = {"sweep_ms": t * 1e3, "bytes": by, "gbps": by / t / 1e9,
                         "frac": by / t / 1e9 / HBM_PEAK_GBPS, "per_matrix": per}
    r1 = res["M=1"]
    return {
        "metric": "int8_gemv_sweep_hbm_gbps", "value": r1["gbps"], "unit": "GB/s",
        "n_gpus": 1, "steps": 10, "warmup": 2, "ms_per_step": r1["sweep_ms"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "Llama-3-8B-shaped decode GEMV sweep, 32 layers + lm_head, "
                               "161 dependent launches (BASELINE configs[4]); value is M=1"},
        "detail": res,
        "roofline": {"kernel": "gemv_w8a32_digits_kernel, gemv_w8a32_bcast_kernel for lm_head (all shapes of the sweep)",
                     "bound": "hbm", "achieved": r1["gbps"], "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": r1["frac"], "traffic": None},
    }


def bench_model_abi(bh, args):
    """The reference's own decode entry point, `_mlir_ciface_forward_decode`
    with its 88 memref arguments (two weight blobs, token, position, 56 KV
    tensors), called token after token the way buddy-cli's runtime does: host
    buffers in, malloc'd logits out, argmax on the host.  The library keeps
    weights and KV caches resident on the device between calls."""
    import numpy as np

    import buddy_mlir_amd as bma
    import test_gpu_model_abi as T
    from buddy_mlir_amd.session import Shape

    L = 1024
    shape = Shape(max_len=L)
    f32, i8, _ = T.make_blobs(bh, shape, seed=2)
    mf = bma.MemRef(f32.ctypes.data, [f32.size])
    mi = bma.MemRef(i8.ctypes.data, [i8.size], ctype=ctypes.c_int8)
    kv = [np.random.default_rng(j).standard_normal((2, L, 128)).astype(np.float32)
          for j in range(2 * shape.layers)]
    kvm = [bma.MemRef(a.ctypes.data, [1, 2, L, 128]) for a in kv]
    posbuf, tokbuf = np.zeros(1, np.int64), np.zeros((1, 1), np.int64)
    dummies = [np.zeros(1, np.int64) for _ in range(shape.layers - 1)]
    mpos = bma.MemRef(posbuf.ctypes.data, [1], ctype=ctypes.c_longlong)
    mtok = bma.MemRef(tokbuf.ctypes.data, [1, 1], ctype=ctypes.c_longlong)
    mdum = [bma.MemRef(d.ctypes.data, [1], ctype=ctypes.c_longlong) for d in dummies]
    free = ctypes.CDLL(None).free
    free.argtypes = [ctypes.c_void_p]

    def step(pos, tok):
        tokbuf[0, 0], posbuf[0] = tok, pos
        for d in dummies:
            d[0] = pos
        res = T.DecodeResult()
        a = [ctypes.byref(res), ctypes.byref(mf), ctypes.byref(mi), ctypes.byref(mtok),
             ctypes.byref(mpos), ctypes.byref(kvm[0]), ctypes.byref(kvm[1])]
        for i in range(shape.layers - 1):
            a += [ctypes.byref(mdum[i]), ctypes.byref(kvm[2 + 2 * i]), ctypes.byref(kvm[3 + 2 * i])]
        bh._mlir_ciface_forward_decode(*a)
        if not res.logits.aligned:
            raise RuntimeError(bh.buddy_hip_last_error())
        lg = np.ctypeslib.as_array(res.logits.aligned, shape=(shape.vocab,))
        nxt = int(lg.argmax())
        free(ctypes.cast(res.logits.allocated, ctypes.c_void_p))
        return nxt

    tok = 5
    for w in range(max(1, args.warmup)):  # the first call uploads and packs the blobs
        tok = step(900 + w, tok)
    n = max(1, min(args.steps, L - 901 - args.warmup))
    t0 = time.perf_counter()
    for s_ in range(n):
        tok = step(900 + max(1, args.warmup) + s_, tok)
    t = (time.perf_counter() - t0) / n
    bh.buddy_hip_forward_reset()
    return {
        "metric": "decode_tokens_per_s", "value": 1.0 / t, "unit": "tokens/s",
        "n_gpus": 1, "steps": n, "warmup": max(1, args.warmup), "ms_per_step": t * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "_mlir_ciface_forward_decode (the reference's 88-argument decode "
                               "entry point), Qwen2-1.5B shape, context ~900, host buffers in and "
                               "out, host argmax; PCIe-inclusive"},
        "roofline": {"kernel": "whole call", "bound": "hbm",
                     "achieved": decode_step_bytes(shape, 900) / t / 1e9, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": decode_step_bytes(shape, 900) / t / 1e9 / HBM_PEAK_GBPS,
                     "traffic": None},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--workload", default="decode",
                    choices=["decode", "gemv", "mlp", "prefill", "llama8b", "kvdiscard", "w4a16",
                             "model_abi", "sampler", "quantize"],
                    help="decode (default): the full decode step the headline metric "
                         "is quoted on; the others measure the remaining configurations")
    ap.add_argument("--mlp-rows", default="1,4,16",
                    help="--workload mlp: the row counts to time (1..16, comma separated)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a 256 MiB device-to-device copy (a kernel of "
                         "known traffic) for scaling hardware counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU's decode throughput; --gpus above 1 is "
              "not supported in this build (nothing here uses a second GPU).",
              file=sys.stderr)
        sys.exit(2)

    import torch

    import buddy_mlir_amd as bma
    from buddy_mlir_amd import synthetic
    from buddy_mlir_amd.session import Shape

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    bh = bma.lib()
    if args.workload != "decode":
        fn = {"gemv": bench_gemv, "mlp": bench_mlp, "prefill": bench_prefill,
              "llama8b": bench_llama8b, "kvdiscard": bench_kvdiscard, "w4a16": bench_w4a16,
              "model_abi": bench_model_abi, "sampler": bench_sampler,
              "quantize": bench_quantize}[args.workload]
        print(json.dumps(fn(bh, args)))
        return
    K, W = args.steps, args.warmup
    max_len = (CONTEXT + W + K + 63) // 64 * 64
    shape = Shape(max_len=max_len)
    want_cpu = not args.no_cpu_baseline
    sess, host = synthetic.build_session(shape, context=CONTEXT, keep_host=want_cpu)
    sess.use_graph(not args.no_graph)
    first = int(synthetic.first_tokens(shape, 1)[0])

    stream = torch.cuda.ExternalStream(sess.stream)
    sess.set_state(first, CONTEXT)
    sess.enqueue_steps(W)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    stream.synchronize()
    t0 = time.perf_counter()
    e0.record(stream)
    sess.enqueue_steps(K)
    e1.record(stream)
    e1.synchronize()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    dev_s = e0.elapsed_time(e1) * 1e-3
    step_s = max(dev_s, wall) / K  # the slower of the two clocks

    # dominant kernel, measured live on its launch stream
    gu_s = time_gate_up(bh, shape, sess.stream, layers=16, iters=160, use_graph=not args.no_graph)
    gu_b = gate_up_bytes(shape.hidden, shape.inter)
    achieved = gu_b / gu_s / 1e9
    step_b = decode_step_bytes(shape, CONTEXT + W + K // 2)
    traffic, traffic_source = gate_up_traffic(collecting=args.calibrate_copy)
    prof_us, prof_source = gate_up_rocprof_us()

    out = {
        "metric": "decode_tokens_per_s",
        "value": 1.0 / step_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": step_s * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {
            "arithmetic": "per-layer GEMVs: int8 weights x f32 activations cut into four int8 "
                          "digit planes (31-bit fixed point per wavefront's run) on the int8 "
                          "matrix cores, exact int32 sums; attention, norms, lm_head and every "
                          "kernel boundary: f32",
            "workload": "Qwen2-1.5B-shaped int8 weight-only (w8a32) decoder, one "
                        "greedy decode step, batch 1, KV cache prefilled to 1024 "
                        "positions (BASELINE configs[2])",
            "layers": shape.layers, "hidden": shape.hidden, "heads": shape.heads,
            "kv_heads": shape.kv_heads, "inter": shape.inter, "vocab": shape.vocab,
            "context": CONTEXT, "hip_graph": not args.no_graph,
        },
        "decode_step_algorithmic_bytes": step_b,
        "decode_step_hbm_gbps": step_b / step_s / 1e9,
        "decode_step_hbm_frac": step_b / step_s / 1e9 / HBM_PEAK_GBPS,
        "roofline": {
            "kernel": GATE_UP_KERNEL + " (RMSNorm + gate|up int8 GEMV "
                      "+ SiLU*mul, 1536 -> 2 x 8960)",
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "algorithmic_bytes_per_launch": gu_b,
            "avg_launch_us": gu_s * 1e6,
            "traffic": traffic,
            "traffic_source": traffic_source,
            # the same launches under rocprofv3 --kernel-trace (durations under the
            # profiler come out a few per cent longer than HIP events without it)
            "rocprof_avg_launch_us": prof_us,
            "frac_rocprof": (gu_b / (prof_us * 1e-6) / 1e9 / HBM_PEAK_GBPS) if prof_us else None,
            "rocprof_source": prof_source,
        },
    }
    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
    if want_cpu:
        out["cpu_baseline"] = cpu_baseline(shape, host, first)
    sess.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
