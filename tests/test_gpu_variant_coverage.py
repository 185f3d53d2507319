"""Every compiled variant of the kernels that issue their global loads by hand,
and of the one-to-four-row GEMV with its many slot counts, meets the oracle.

The first (the int8 and bf16 matrix-core kernels of the small-batch GEMV and of
the prefill matmul, and the prefill attention) wait for their loads by
counting; a mistake in one template variant shows only in that variant.  The
library lists every variant it was built with (buddy_hip_variant_report); this
test drives one parity case through each plan that selects one, and fails when
a variant is left that none of its cases launched -- so a variant added to the
source without a case here fails the suite."""
import ctypes

import numpy as np
import pytest
import torch

import buddy_mlir_amd as bma
import oracle_lib
from buddy_mlir_amd import ops, synthetic
from buddy_mlir_amd.session import Shape
from parity import check_close
from test_gpu_prefill import (SCALE, SILU_PAIR_SHAPES, bf16_round, fixed_point_round, run_attn,
                              silu_pair_case)

pytestmark = pytest.mark.gpu


def report(bh):
    n = bh.buddy_hip_variant_report(None, 0)
    buf = ctypes.create_string_buffer(n)
    bh.buddy_hip_variant_report(buf, n)
    out = {}
    for line in buf.value.decode().splitlines():
        name, hits = line.split("\t")
        out[name] = int(hits)
    return out


def launched(bh, family):
    return {k for k, v in report(bh).items() if k.startswith(family + "<") and v > 0}


def compiled(bh, family):
    return {k for k in report(bh) if k.startswith(family + "<")}


# ---- small-batch GEMV: <epilogue, channel groups per wavefront, fused norm> ----
# N picks the channel groups per wavefront (see launch_gemv_i8 / launch_gemv_mfma)
def gemv_case(bh, oracle, M, K, N, epilogue, norm, seed):
    dual = epilogue == 2
    q0, s0 = synthetic.quantized_linear(K, N, seed)
    q1, s1 = synthetic.quantized_linear(K, N, seed + 1) if dual else (None, None)
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn((M, K), generator=g, device="cuda")
    w = torch.rand((K,), generator=g, device="cuda") + 0.5
    c0 = torch.randn((M, N), generator=g, device="cuda")
    c = c0.clone()
    kw = dict(A=x, lda=K, W0=ops.pack_w8(q0), scale0=s0, C=c, ldc=N, M=M, K=K, N=N,
              epilogue=epilogue)
    if dual:
        kw.update(W1=ops.pack_w8(q1), scale1=s1)
    if norm:
        kw.update(norm_w=w, norm_eps=1e-6)
    torch.cuda.synchronize()
    ops.linear_w8a32(stream=None, **kw)
    torch.cuda.synchronize()
    xh = x.cpu().numpy()
    if norm:
        xh = np.stack([oracle.rmsnorm(r, w.cpu().numpy(), eps=np.float32(1e-6)) for r in xh])
    y0 = np.stack([oracle.dequant_gemv(r, q0.cpu().numpy(), s0.cpu().numpy()) for r in xh])
    if dual:
        y1 = np.stack([oracle.dequant_gemv(r, q1.cpu().numpy(), s1.cpu().numpy()) for r in xh])
        want = np.stack([oracle.silu_mul(a, b) for a, b in zip(y0, y1)])
    elif epilogue == 1:
        want = c0.cpu().numpy() + y0
    else:
        want = y0
    got = c.cpu().numpy()
    for m in range(M):
        check_close(got[m], want[m])


GEMV_I8_N = [2560, 8192, 32768]       # 1, 2, 4 channel groups per wavefront
GEMV_BF16_N = [320, 8192, 131072]     # 2, 4, 8


def test_every_int8_batch_gemv_variant(bh, oracle):
    bh.buddy_hip_variant_reset()
    # up to 8 rows take the variants that convert two tiles at a time (K = 192:
    # a pair and a last tile without a partner; K = 320 ends inside a pair's
    # second tile), more rows the one-tile variants
    # (more than 8 rows of a matrix of up to 128 channel groups go to two
    # workgroups of up to 8 rows on the two-tile variants: the last case)
    for i, N in enumerate(GEMV_I8_N):
        for epilogue in (0, 1, 2):
            for norm in (False, True):
                gemv_case(bh, oracle, 9 + 3 * i, 192, N, epilogue, norm, 100 + i)
                if i < 2:
                    gemv_case(bh, oracle, 5 + 3 * i, 192 + 108 * i, (320, 8192)[i], epilogue,
                              norm, 150 + i)
                if i == 0:
                    gemv_case(bh, oracle, 13, 192, 320, epilogue, norm, 170)
    fam = "gemv_w8a32_i8_kernel"
    assert launched(bh, fam) == compiled(bh, fam), compiled(bh, fam) - launched(bh, fam)


def test_every_bf16_batch_gemv_variant(bh, oracle):
    bh.buddy_hip_variant_reset()
    assert bh.buddy_hip_set_gemv_batch_kernel(1) == 0
    try:
        for i, N in enumerate(GEMV_BF16_N):
            for epilogue in (0, 1, 2):
                for norm in (False, True):
                    gemv_case(bh, oracle, 6 + 5 * i, 128, N, epilogue, norm, 200 + i)
    finally:
        assert bh.buddy_hip_set_gemv_batch_kernel(0) == 0
    fam = "gemv_w8a32_mfma_kernel"
    assert launched(bh, fam) == compiled(bh, fam), compiled(bh, fam) - launched(bh, fam)


# ---- GEMV of up to four rows over digit planes on the matrix cores: <rows, epilogue, input,
# tile slots per wavefront, channel group split over two workgroups> ---------------
# With more than 128 channel groups a wavefront gets ceil(K / 64 / 16) tiles (16
# k-slices) once K >= 4096, and K = 128, 192 give runs of 2 and 3; with 4 channel
# groups and K >= 4096 the groups are split and the tiles go in pairs.  The rows
# end inside a tile (K % 64 != 0) wherever that keeps the run's length; K stays a
# multiple of 4 so that batches of rows keep 16-byte aligned rows (one row with
# K % 4 != 0 is covered by the shapes of test_gpu_gemv.py).
ROW_K = {2: 124, 3: 188, **{t: 1024 * t - 8 for t in range(4, 17)}}
ROW_SINGLE = {1: [2, 3, 4, 5, 6, 7, 8, 9, 10, 12, 14, 16], 2: [2, 3, 4, 6, 8, 10, 12],
              3: [2, 3, 4, 6, 8]}
ROW_DUAL = {1: [2, 3, 4, 5, 6, 7, 8, 9], 2: [2, 3, 4, 6, 8], 3: [2, 3, 4, 6]}
ROW_SPLIT = [4, 6, 8, 10]
FOLD_HEADS = {2: (12, 2), 3: (24, 4), 4: (32, 4)}  # o_proj of heads x 128 inputs: 2, 3, 4 tiles


def test_every_row_gemv_variant(bh, oracle):
    bh.buddy_hip_variant_reset()
    for rows in (1, 2, 3):  # three rows run the kernel compiled for four
        for t in ROW_SINGLE[rows]:
            for epilogue in (0, 1):
                for norm in (False, True):
                    gemv_case(bh, oracle, rows, ROW_K[t], 2064, epilogue, norm, 300 + t)
        for t in ROW_DUAL[rows]:
            for norm in (False, True):
                gemv_case(bh, oracle, rows, ROW_K[t], 2064, 2, norm, 330 + t)
        for t in ROW_SPLIT:
            for epilogue in (0, 1):
                for norm in (False, True):
                    gemv_case(bh, oracle, rows, ROW_K[t] - 1024 * (t == 10), 64, epilogue, norm,
                              360 + t)
    # input folded from the attention partials: the o_proj of a decode step
    for tiles, (heads, kv_heads) in FOLD_HEADS.items():
        shape = Shape(layers=1, hidden=256, heads=heads, kv_heads=kv_heads, head_dim=128, inter=512,
                      vocab=1024, max_len=128, rms_eps=1e-6)
        sess, host = synthetic.build_session(shape, context=70, keep_host=True, ln_jitter=0.1)
        om = oracle_lib.model_from_host(oracle, shape, host)
        kv = [a.copy() for a in host["kv"]]
        tok = 3
        for step in range(3):
            nxt, logits = sess.decode(tok, 70 + step)
            tok, ologits = om.decode_step(tok, 70 + step, kv)
            check_close(logits, ologits)
            assert nxt == tok
        sess.close()
    fam = "gemv_w8a32_digits_kernel"
    assert launched(bh, fam) == compiled(bh, fam), compiled(bh, fam) - launched(bh, fam)


def test_row_gemv_random_shapes(bh, oracle):
    """120 seeded random shapes, row counts and fused forms through whatever
    kernel the launch's cut picks (ragged K and N, rows whose length is not a
    multiple of four, narrow long matrices that are split over two workgroups)."""
    rng = np.random.default_rng(2024)
    for case in range(120):
        K = int(rng.choice([rng.integers(1, 300), rng.integers(300, 12000)]))
        N = int(rng.choice([rng.integers(1, 200), rng.integers(200, 3000)]))
        M = int(rng.integers(1, 5))
        epilogue = int(rng.integers(0, 3))
        norm = bool(rng.integers(0, 2))
        gemv_case(bh, oracle, M, K, N, epilogue, norm, 1000 + case)


# ---- prefill matmul: the tile shape comes out of the launch's cost model -------
GEMM_I8_SHAPES = [(144, 256, 16384), (300, 256, 10240), (200, 192, 16384), (512, 192, 8960),
                  (17, 64, 64)]
# with two planes every unsplit tile costs the loop's floor per chunk, so the
# widest tile wins there; the other tile shapes are reached with K split over
# workgroups
GEMM_I8_SPLIT_K_SHAPES = [(17, 1536, 256), (100, 4096, 8192), (100, 4096, 12288)]
# one plane (w8a8): the same, the K slices leaving int32 sums
W8A8_SPLIT_K_SHAPES = [(17, 1536, 256), (100, 4096, 12288), (300, 4096, 5120)]
GEMM_BF16_SHAPES = [(512, 64, 8960), (300, 64, 10240), (17, 64, 64)]


def gemm_case(oracle, M, K, N, mode):
    q, s = synthetic.quantized_linear(K, N, M + K + N)
    g = torch.Generator(device="cuda").manual_seed(M)
    x = torch.randn((M, K), generator=g, device="cuda")
    y = ops.gemm_w8a32(x, ops.pack_w8(q), s, K, N, exact=mode == "exact",
                       digits={"digits": 3, "digits2": 2}.get(mode, False))
    torch.cuda.synchronize()
    xh = x.cpu().numpy()
    a_in = bf16_round(xh) if mode == "bf16" else xh
    if mode == "digits2":
        a_in, _ = fixed_point_round(xh, digits=2)
    want = oracle.blis_gemm_w8a32(a_in, q.cpu().numpy(), s.cpu().numpy())
    got = y.cpu().numpy()
    for m in range(M):
        check_close(got[m], want[m])


def w8a8_case(bh, oracle, M, K, N):
    q, s = synthetic.quantized_linear(K, N, M + K + N)
    g = torch.Generator(device="cuda").manual_seed(M)
    x = torch.randn((M, K), generator=g, device="cuda")
    C = torch.empty((M, N), device="cuda")
    acc = torch.empty((M, N), dtype=torch.int32, device="cuda")
    nb = bh.buddy_hip_w8a8_workspace_bytes(M, K)
    ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
    packed = ops.pack_w8(q)
    torch.cuda.synchronize()
    assert bh.buddy_hip_w8a8_matmul(x.data_ptr(), packed.data_ptr(), s.data_ptr(), C.data_ptr(),
                                    acc.data_ptr(), M, K, N, ws.data_ptr(), nb, None) == 0
    torch.cuda.synchronize()
    wC, wacc = oracle.w8a8_matmul(x.cpu().numpy(), q.cpu().numpy(), s.cpu().numpy())
    np.testing.assert_array_equal(acc.cpu().numpy(), wacc)
    np.testing.assert_array_equal(C.cpu().numpy(), wC)


def test_every_int8_prefill_matmul_variant(bh, oracle):
    bh.buddy_hip_variant_reset()
    for M, K, N in GEMM_I8_SHAPES:
        gemm_case(oracle, M, K, N, "digits")
        gemm_case(oracle, M, K, N, "digits2")  # the two-plane variants
        w8a8_case(bh, oracle, M, K, N)  # the one-plane variants of the same tile shapes
    for M, K, N in GEMM_I8_SPLIT_K_SHAPES:
        gemm_case(oracle, M, K, N, "digits")
        gemm_case(oracle, M, K, N, "digits2")
    for M, K, N in W8A8_SPLIT_K_SHAPES:
        w8a8_case(bh, oracle, M, K, N)
    for M, K, N in SILU_PAIR_SHAPES[1:5]:  # the paired variants
        silu_pair_case(oracle, M, K, N)
        silu_pair_case(oracle, M, K, N, digits=2)
    for fam in ("gemm_w8_i8_wide_kernel", "gemm_w8_i8_kernel"):
        assert launched(bh, fam) == compiled(bh, fam), compiled(bh, fam) - launched(bh, fam)


def test_every_bf16_prefill_matmul_variant(bh, oracle):
    bh.buddy_hip_variant_reset()
    for M, K, N in GEMM_BF16_SHAPES:
        for mode in ("bf16", "exact"):
            gemm_case(oracle, M, K, N, mode)
    for fam in ("gemm_w8_bf16_wide_kernel", "gemm_w8_bf16_kernel"):
        assert launched(bh, fam) == compiled(bh, fam), compiled(bh, fam) - launched(bh, fam)


def test_prefill_attention_and_no_unlisted_family(bh, oracle):
    bh.buddy_hip_variant_reset()
    heads, kv_heads, L, D = 4, 2, 40, 128
    g = torch.Generator(device="cuda").manual_seed(3)
    q = torch.randn((heads, L, D), generator=g, device="cuda")
    k = torch.randn((kv_heads, L, D), generator=g, device="cuda")
    v = torch.randn((kv_heads, L, D), generator=g, device="cuda")
    got = run_attn(bh, q, k, v, None, heads, kv_heads, L, L)
    rep = heads // kv_heads
    kk = np.repeat(k.cpu().numpy(), rep, axis=0)
    vv = np.repeat(v.cpu().numpy(), rep, axis=0)
    mask = np.triu(np.full((L, L), -np.inf, np.float32), 1)
    want = oracle.prefill_flash_attention(q.cpu().numpy(), kk, vv, mask, SCALE)
    check_close(got, want)
    # more workgroups than compute units: four wavefronts per workgroup
    heads, kv_heads, L = 32, 8, 272
    q = torch.randn((heads, L, D), generator=g, device="cuda")
    k = torch.randn((kv_heads, L, D), generator=g, device="cuda")
    v = torch.randn((kv_heads, L, D), generator=g, device="cuda")
    got = run_attn(bh, q, k, v, None, heads, kv_heads, L, L)
    rep = heads // kv_heads
    mask = np.triu(np.full((L, L), -np.inf, np.float32), 1)
    want = oracle.prefill_flash_attention(q.cpu().numpy(), np.repeat(k.cpu().numpy(), rep, axis=0),
                                          np.repeat(v.cpu().numpy(), rep, axis=0), mask, SCALE)
    check_close(got, want)
    assert launched(bh, "attn_prefill_kernel") == compiled(bh, "attn_prefill_kernel")
    # every family the library lists is one of those this file drives
    known = ("gemv_w8a32_i8_kernel", "gemv_w8a32_mfma_kernel", "gemm_w8_i8_wide_kernel",
             "gemm_w8_i8_kernel", "gemm_w8_bf16_wide_kernel", "gemm_w8_bf16_kernel",
             "attn_prefill_kernel", "gemv_w8a32_digits_kernel")
    assert {name.split("<")[0] for name in report(bh)} == set(known)
