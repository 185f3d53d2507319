"""GPU parity: quantizer, wave-tile packing and the int8 dequant GEMV against
the CPU oracle, through the C ABI.  Bit-exact for int8 tensors and pack/unpack;
fp32 outputs within 1e-3 relative (see tests/parity.py; observed differences
are ~1e-6, from the different summation order)."""
import ctypes
import os

import numpy as np
import pytest
import torch

import buddy_mlir_amd as bma
from buddy_mlir_amd import ops

pytestmark = pytest.mark.gpu

from parity import check_close


def make_weight(K, N, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.randn((K, N), generator=g, device="cuda") * 0.02


@pytest.mark.parametrize("K,N", [(64, 16), (1536, 8960), (8960, 1536), (100, 70), (1, 1),
                                 (131, 68), (3, 4), (70000, 8)])
def test_quantizer_bit_exact(oracle, K, N):
    W = make_weight(K, N, K * 7 + N)
    if K > 3 and N > 2:
        W[:, 1] = 0.0  # an all-zero channel
    q, s = ops.quantize_w8(W)
    rq, rs = oracle.quantize_w8(W.cpu().numpy())
    np.testing.assert_array_equal(q.cpu().numpy(), rq)
    np.testing.assert_array_equal(s.cpu().numpy(), rs)


@pytest.mark.parametrize("K,N", [(64, 16), (128, 64), (1536, 256), (100, 70), (1, 1), (65, 17)])
def test_pack_roundtrip_and_layout(K, N):
    g = torch.Generator(device="cuda").manual_seed(K + N)
    q = torch.randint(-128, 128, (K, N), generator=g, device="cuda", dtype=torch.int8)
    p = ops.pack_w8(q)
    assert p.numel() == ((K + 63) // 64 * 64) * ((N + 15) // 16 * 16)
    np.testing.assert_array_equal(ops.unpack_w8(p, K, N).cpu().numpy(), q.cpu().numpy())
    # closed form of the layout, checked on the host
    qh, ph = q.cpu().numpy(), p.cpu().numpy()
    chunks = (K + 63) // 64
    rng = np.random.default_rng(0)
    for _ in range(200):
        k, n = int(rng.integers(K)), int(rng.integers(N))
        lane = ((k % 64) // 16) * 16 + n % 16
        off = (((n // 16) * chunks + k // 64) * 64 + lane) * 16 + k % 16
        assert ph[off] == qh[k, n]
    # padding is zero
    assert int(np.abs(ph.astype(np.int32)).sum()) == int(np.abs(qh.astype(np.int32)).sum())


@pytest.mark.parametrize("tn", [8, 4])
@pytest.mark.parametrize("K,N", [(256, 8), (8960, 1536), (1536, 1536), (300, 50), (1, 1)])
def test_narrow_tile_layouts(oracle, K, N, tn):
    g = torch.Generator(device="cuda").manual_seed(K + N + tn)
    q = torch.randint(-128, 128, (K, N), generator=g, device="cuda", dtype=torch.int8)
    p = ops.pack_w8_tiles(q, tn)
    tk = 1024 // tn
    assert p.numel() == ((K + tk - 1) // tk * tk) * ((N + tn - 1) // tn * tn)
    np.testing.assert_array_equal(ops.unpack_w8_tiles(p, K, N, tn).cpu().numpy(),
                                  q.cpu().numpy())
    qh, ph = q.cpu().numpy(), p.cpu().numpy()
    chunks = (K + tk - 1) // tk
    rng = np.random.default_rng(1)
    for _ in range(100):
        k, n = int(rng.integers(K)), int(rng.integers(N))
        lane = ((k % tk) // 16) * tn + n % tn
        off = (((n // tn) * chunks + k // tk) * 64 + lane) * 16 + k % 16
        assert ph[off] == qh[k, n]
    # GEMV over the narrow tiles, plain and accumulating
    s = torch.rand(N, generator=g, device="cuda") * 1e-3 + 1e-4
    x = torch.randn((1, K), generator=g, device="cuda")
    c0 = torch.randn((1, N), generator=g, device="cuda")
    y = torch.empty((1, N), device="cuda")
    c = c0.clone()
    torch.cuda.synchronize()
    ops.linear_w8a32(A=x, lda=K, W0=p, scale0=s, C=y, ldc=N, M=1, K=K, N=N, epilogue=0, tile_n=tn)
    ops.linear_w8a32(A=x, lda=K, W0=p, scale0=s, C=c, ldc=N, M=1, K=K, N=N, epilogue=1, tile_n=tn)
    torch.cuda.synchronize()
    xh, sh = x.cpu().numpy()[0], s.cpu().numpy()
    check_close(y.cpu().numpy()[0], oracle.dequant_gemv(xh, qh, sh))
    check_close(c.cpu().numpy()[0], oracle.dequant_gemv(xh, qh, sh, c0.cpu().numpy()[0]))


# (102, 70): K % 4 != 0 keeps every batch size on the f32 FMA kernel; (100, 70)
# and (1100, 40) end a row inside a 16-k run of the matrix-core kernel
SHAPES = [(1536, 8960), (8960, 1536), (1536, 1536), (1536, 256), (64, 16), (100, 70),
          (102, 70), (1100, 40), (1536, 151936), (4096, 4096), (1, 1), (3, 17), (5, 33)]


@pytest.mark.parametrize("K,N", SHAPES)
@pytest.mark.parametrize("M", [1, 2, 4, 5, 8, 13, 16])
def test_gemv_matches_oracle(oracle, K, N, M):
    W = make_weight(K, N, K + 3 * N)
    q, s = ops.quantize_w8(W)
    packed = ops.pack_w8(q)
    g = torch.Generator(device="cuda").manual_seed(M)
    x = torch.randn((M, K), generator=g, device="cuda")
    y = ops.gemv_w8a32(x, packed, s, K, N)
    torch.cuda.synchronize()
    qh, sh, xh = q.cpu().numpy(), s.cpu().numpy(), x.cpu().numpy()
    want = np.stack([oracle.dequant_gemv(xh[m], qh, sh) for m in range(M)])
    check_close(y.cpu().numpy(), want)


# The decode GEMV set of a Llama-3-8B-shaped step: q_proj, kv_proj, gate/up, down
# and lm_head, each alone at one row and at eight.
LLAMA3_8B = [(4096, 4096), (4096, 1024), (4096, 14336), (14336, 4096), (4096, 128256)]


@pytest.mark.parametrize("K,N", LLAMA3_8B)
@pytest.mark.parametrize("M", [1, 8])
def test_llama3_8b_gemv_set_matches_oracle(oracle, K, N, M):
    q, s = ops.quantize_w8(make_weight(K, N, K + 5 * N))
    packed = ops.pack_w8(q)
    g = torch.Generator(device="cuda").manual_seed(10 + M)
    x = torch.randn((M, K), generator=g, device="cuda")
    y = ops.gemv_w8a32(x, packed, s, K, N)
    torch.cuda.synchronize()
    qh, sh, xh = q.cpu().numpy(), s.cpu().numpy(), x.cpu().numpy()
    want = np.stack([oracle.dequant_gemv(xh[m], qh, sh) for m in range(M)])
    check_close(y.cpu().numpy(), want)


@pytest.mark.parametrize("M", [1, 8])
def test_llama3_8b_fused_launches_match_oracle(oracle, M):
    """The launches a Llama-3-8B-shaped decode step makes: RMSNorm + q|k|v as one
    matrix (4096 -> 6144), o_proj accumulating into the residual row, RMSNorm +
    gate|up + SiLU*mul (4096 -> 2 x 14336), down accumulating (14336 -> 4096),
    RMSNorm + lm_head (4096 -> 128256)."""
    H, I, QKV, V = 4096, 14336, 4096 + 2 * 1024, 128256
    eps = np.float32(1e-5)
    g = torch.Generator(device="cuda").manual_seed(40 + M)
    x = torch.randn((M, H), generator=g, device="cuda") * 2
    w = 1 + 0.1 * torch.randn(H, generator=g, device="cuda")
    xh, wh = x.cpu().numpy(), w.cpu().numpy()
    xn = np.stack([oracle.rmsnorm(xh[m], wh, eps, np.float32(1.0) / np.float32(H))
                   for m in range(M)])

    def launch(**kw):
        torch.cuda.synchronize()
        ops.linear_w8a32(**kw)
        torch.cuda.synchronize()

    # RMSNorm + q|k|v
    q, s = ops.quantize_w8(make_weight(H, QKV, 1))
    out = torch.empty((M, QKV), device="cuda")
    launch(A=x, lda=H, W0=ops.pack_w8(q), scale0=s, norm_w=w, norm_eps=float(eps), C=out,
           ldc=QKV, M=M, K=H, N=QKV, epilogue=0)
    qh, sh = q.cpu().numpy(), s.cpu().numpy()
    check_close(out.cpu().numpy(), np.stack([oracle.dequant_gemv(xn[m], qh, sh) for m in range(M)]))
    # o_proj, C += ...
    q, s = ops.quantize_w8(make_weight(H, H, 2))
    c0 = torch.randn((M, H), generator=g, device="cuda")
    c = c0.clone()
    launch(A=x, lda=H, W0=ops.pack_w8(q), scale0=s, C=c, ldc=H, M=M, K=H, N=H, epilogue=1)
    qh, sh, c0h = q.cpu().numpy(), s.cpu().numpy(), c0.cpu().numpy()
    check_close(c.cpu().numpy(),
                np.stack([oracle.dequant_gemv(xh[m], qh, sh, c0h[m]) for m in range(M)]))
    # RMSNorm + gate|up + SiLU*mul
    qg, sg = ops.quantize_w8(make_weight(H, I, 3))
    qu, su = ops.quantize_w8(make_weight(H, I, 4))
    h = torch.empty((M, I), device="cuda")
    launch(A=x, lda=H, W0=ops.pack_w8(qg), scale0=sg, W1=ops.pack_w8(qu), scale1=su, norm_w=w,
           norm_eps=float(eps), C=h, ldc=I, M=M, K=H, N=I, epilogue=2)
    qgh, sgh, quh, suh = (t.cpu().numpy() for t in (qg, sg, qu, su))
    hh = np.stack([oracle.silu_mul(oracle.dequant_gemv(xn[m], qgh, sgh),
                                   oracle.dequant_gemv(xn[m], quh, suh)) for m in range(M)])
    check_close(h.cpu().numpy(), hh)
    del qg, qu
    # down, C += ...
    q, s = ops.quantize_w8(make_weight(I, H, 5))
    c = c0.clone()
    hin = torch.from_numpy(hh).cuda()
    launch(A=hin, lda=I, W0=ops.pack_w8(q), scale0=s, C=c, ldc=H, M=M, K=I, N=H, epilogue=1)
    qh, sh = q.cpu().numpy(), s.cpu().numpy()
    check_close(c.cpu().numpy(),
                np.stack([oracle.dequant_gemv(hh[m], qh, sh, c0h[m]) for m in range(M)]))
    # RMSNorm + lm_head
    q, s = ops.quantize_w8(make_weight(H, V, 6))
    out = torch.empty((M, V), device="cuda")
    launch(A=x, lda=H, W0=ops.pack_w8(q), scale0=s, norm_w=w, norm_eps=float(eps), C=out,
           ldc=V, M=M, K=H, N=V, epilogue=0)
    qh, sh = q.cpu().numpy(), s.cpu().numpy()
    check_close(out.cpu().numpy(), np.stack([oracle.dequant_gemv(xn[m], qh, sh) for m in range(M)]))


@pytest.mark.parametrize("M", [1, 3])
def test_norm_weight_alignment_and_ragged_k(bh, oracle, M):
    """RMSNorm fused into the GEMV with K not a multiple of 4: the kernels read
    the norm weight in 16-byte pieces, so one that is not 16-byte aligned (a
    piece could run past its end) is refused; an aligned one gives the oracle's
    result whatever lies behind its last value."""
    K, N = 1001, 272
    eps = np.float32(1e-6)
    g = torch.Generator(device="cuda").manual_seed(70 + M)
    x = torch.randn((M, K), generator=g, device="cuda")
    wbuf = 1 + 0.1 * torch.randn(K + 1, generator=g, device="cuda")
    q, s = ops.quantize_w8(make_weight(K, N, 7))
    out = torch.empty((M, N), device="cuda")
    assert wbuf[1:].data_ptr() % 16 == 4
    with pytest.raises(bma.BuddyHipError, match="16-byte aligned"):
        ops.linear_w8a32(A=x, lda=K, W0=ops.pack_w8(q), scale0=s, norm_w=wbuf[1:],
                         norm_eps=float(eps), C=out, ldc=N, M=M, K=K, N=N, epilogue=0)
    # the weight's last 16-byte piece reaches past its K values, and what lies
    # there (NaNs here) must not reach the result
    wpad = torch.full((K + 7,), float("nan"), device="cuda")
    wpad[:K] = wbuf[:K]
    w = wpad[:K]
    assert w.data_ptr() % 16 == 0
    ops.linear_w8a32(A=x, lda=K, W0=ops.pack_w8(q), scale0=s, norm_w=w, norm_eps=float(eps),
                     C=out, ldc=N, M=M, K=K, N=N, epilogue=0)
    torch.cuda.synchronize()
    xh, wh, qh, sh = x.cpu().numpy(), w.cpu().numpy(), q.cpu().numpy(), s.cpu().numpy()
    xn = [oracle.rmsnorm(xh[m], wh, eps, np.float32(1.0) / np.float32(K)) for m in range(M)]
    check_close(out.cpu().numpy(), np.stack([oracle.dequant_gemv(xn[m], qh, sh) for m in range(M)]))


@pytest.fixture
def bf16_batch_kernel(bh):
    """Batches of 5..16 rows through the bf16 matrix-core kernel (every f32 bit of
    the activations) instead of the default int8 matrix-core kernel."""
    assert bh.buddy_hip_set_gemv_batch_kernel(1) == 0
    yield
    assert bh.buddy_hip_set_gemv_batch_kernel(0) == 0


@pytest.mark.parametrize("K,N", [(1536, 8960), (8960, 1536), (100, 70), (1100, 40)])
@pytest.mark.parametrize("M", [5, 16])
def test_gemv_bf16_batch_kernel_matches_oracle(oracle, bf16_batch_kernel, K, N, M):
    q, s = ops.quantize_w8(make_weight(K, N, K + N))
    packed = ops.pack_w8(q)
    g = torch.Generator(device="cuda").manual_seed(M)
    x = torch.randn((M, K), generator=g, device="cuda")
    y = ops.gemv_w8a32(x, packed, s, K, N)
    torch.cuda.synchronize()
    qh, sh, xh = q.cpu().numpy(), s.cpu().numpy(), x.cpu().numpy()
    want = np.stack([oracle.dequant_gemv(xh[m], qh, sh) for m in range(M)])
    check_close(y.cpu().numpy(), want)


def test_row_kernel_fixed_point_keeps_f32_accuracy():
    """One row goes through the int8 matrix cores: every wavefront turns its
    own run of the row (here 1536 / 8 = 192 values) into 31-bit fixed point with
    a step of its own.  Rows of any magnitude, a loud run next to quiet ones and
    a zero row each agree with a float64 sum to f32 accuracy; inside a run, a
    value keeps all its bits down to 2^-7 of the run's largest and is rounded
    to 2^-31 of that largest below, which the comparison allows for through the
    run's largest value."""
    K, N = 1536, 4096
    q, s = ops.quantize_w8(make_weight(K, N, 79))
    packed = ops.pack_w8(q)
    qh, sh = q.cpu().numpy().astype(np.float64), s.cpu().numpy().astype(np.float64)
    rng = np.random.default_rng(7)
    base = rng.standard_normal(K).astype(np.float32)
    rows = {"plain": base, "huge": base * np.float32(1e20), "tiny": base * np.float32(1e-20),
            "zero": np.zeros(K, np.float32)}
    loud = base.copy()
    loud[192:384] *= np.float32(1e6)          # one wavefront's run, 10^6 louder
    rows["loud run"] = loud
    for name, xh in rows.items():
        y = ops.gemv_w8a32(torch.from_numpy(xh[None]).cuda(), packed, s, K, N).cpu().numpy()[0]
        want = (xh.astype(np.float64) @ qh) * sh
        if name == "zero":
            assert not y.any()
            continue
        check_close(y, want)
    # the quiet runs are not drowned by the loud one: without it the rest still
    # agrees to f32 accuracy
    quiet = loud.copy()
    quiet[192:384] = 0.0
    y = ops.gemv_w8a32(torch.from_numpy(quiet[None]).cuda(), packed, s, K, N).cpu().numpy()[0]
    check_close(y, (quiet.astype(np.float64) @ qh) * sh)
    # an outlier inside a run costs that run's other values resolution below
    # 2^-31 of the outlier and nothing more: the error stays below 2^-30 of the
    # outlier times sum |w| (plus the rounding of the f32 results)
    out = base.copy()
    out[200] = np.float32(3e4)
    y = ops.gemv_w8a32(torch.from_numpy(out[None]).cuda(), packed, s, K, N).cpu().numpy()[0]
    want = (out.astype(np.float64) @ qh) * sh
    bound = 2.0 ** -30 * 3e4 * np.abs(qh[192:384]).sum(0) * sh + 1e-6 * np.abs(want).max()
    assert (np.abs(y - want) <= bound).all()


def test_row_kernel_steps_are_per_row():
    """Four rows in one launch, 40 orders of magnitude apart and one of them
    zero: every row has its own fixed-point step, so each keeps f32 accuracy;
    a NaN in one row leaves the others alone."""
    K, N = 1536, 4096
    q, s = ops.quantize_w8(make_weight(K, N, 81))
    packed = ops.pack_w8(q)
    qh, sh = q.cpu().numpy().astype(np.float64), s.cpu().numpy().astype(np.float64)
    rng = np.random.default_rng(9)
    xh = rng.standard_normal((4, K)).astype(np.float32)
    xh[1] *= np.float32(1e20)
    xh[2] *= np.float32(1e-20)
    xh[3] = 0.0
    y = ops.gemv_w8a32(torch.from_numpy(xh).cuda(), packed, s, K, N).cpu().numpy()
    want = (xh.astype(np.float64) @ qh) * sh
    for m in range(3):
        check_close(y[m], want[m])
    assert not y[3].any()
    xh[1, 5] = np.nan
    y = ops.gemv_w8a32(torch.from_numpy(xh).cuda(), packed, s, K, N).cpu().numpy()
    assert np.isnan(y[1]).all()
    check_close(y[0], want[0])
    check_close(y[2], want[2])
    assert not y[3].any()


@pytest.mark.parametrize("M", [1, 3, 4])
@pytest.mark.parametrize("shift", [0, 1])
def test_row_kernel_strided_and_unaligned_rows(oracle, M, shift):
    """Rows with a stride beyond their length and an output with a stride of its
    own; with `shift` the first row starts 4 bytes off a 16-byte boundary, which
    sends the launch to the f32 kernel (the matrix-core kernel reads 16-byte
    pieces of the rows)."""
    K, N, lda, ldc = 1536, 272, 1536 + 12, 272 + 5
    q, s = ops.quantize_w8(make_weight(K, N, 82))
    packed = ops.pack_w8(q)
    g = torch.Generator(device="cuda").manual_seed(83 + M)
    buf = torch.randn((M * lda + 4,), generator=g, device="cuda")
    out = torch.full((M * ldc,), 7.0, device="cuda")
    a = buf[shift:]
    torch.cuda.synchronize()
    ops.linear_w8a32(A=a.data_ptr(), lda=lda, W0=packed, scale0=s, C=out, ldc=ldc, M=M, K=K, N=N,
                     epilogue=0)
    torch.cuda.synchronize()
    ah = a.cpu().numpy()
    oh = out.cpu().numpy()
    qh, sh = q.cpu().numpy(), s.cpu().numpy()
    for m in range(M):
        check_close(oh[m * ldc:m * ldc + N], oracle.dequant_gemv(ah[m * lda:m * lda + K], qh, sh))
        if m + 1 < M:  # the gap between output rows is left alone
            assert (oh[m * ldc + N:(m + 1) * ldc] == 7.0).all()


def test_row_kernel_shows_non_finite_activations():
    """A NaN or an infinity in the row gives NaN results (the f32 product would
    give NaN or infinity there, and with BUDDY_HIP_GEMV_ROW=f32 does)."""
    K, N = 1536, 256
    q, s = ops.quantize_w8(make_weight(K, N, 80))
    packed = ops.pack_w8(q)
    rng = np.random.default_rng(8)
    for bad in (np.nan, np.inf, -np.inf):
        xh = rng.standard_normal((1, K)).astype(np.float32)
        xh[0, 777] = bad
        y = ops.gemv_w8a32(torch.from_numpy(xh).cuda(), packed, s, K, N).cpu().numpy()
        if os.environ.get("BUDDY_HIP_GEMV_ROW") == "f32":
            assert not np.isfinite(y).any()
        else:
            assert np.isnan(y).all()


def test_int8_batch_kernel_scales_every_64_activations_on_their_own(oracle):
    """The int8 matrix-core kernel turns the activations into fixed point 64 at a
    time, each row and each run of 64 with a step of its own: rows 40 orders of
    magnitude apart, and runs of one row 12 orders apart, must each keep f32
    accuracy (compared row by row, and against a float64 sum)."""
    K, N, M = 1536, 256, 8
    q, s = ops.quantize_w8(make_weight(K, N, 77))
    packed = ops.pack_w8(q)
    rng = np.random.default_rng(5)
    xh = rng.standard_normal((M, K)).astype(np.float32)
    xh[1] *= 1e20
    xh[2] *= 1e-20
    xh[3, 64:128] *= 1e6      # one loud run of 64 in a quiet row
    xh[4, :] *= 1e-6
    xh[4, 640:704] *= 1e12
    xh[5, 130] = 3e4          # a single outlier inside a run
    xh[6] = 0.0               # a zero row stays zero
    x = torch.from_numpy(xh).cuda()
    y = ops.gemv_w8a32(x, packed, s, K, N).cpu().numpy()
    qh, sh = q.cpu().numpy(), s.cpu().numpy()
    want = (xh.astype(np.float64) @ qh.astype(np.float64)) * sh.astype(np.float64)
    for m in range(M):
        check_close(y[m], want[m])
    assert not y[6].any()
    # the quiet runs of row 3 are not drowned by its loud one: leave the loud run
    # out on both sides and the rest still agrees to f32 accuracy
    xq = xh.copy()
    xq[3, 64:128] = 0.0
    yq = ops.gemv_w8a32(torch.from_numpy(xq).cuda(), packed, s, K, N).cpu().numpy()
    wq = (xq[3].astype(np.float64) @ qh.astype(np.float64)) * sh.astype(np.float64)
    check_close(yq[3], wq)


def test_int8_batch_kernel_shows_non_finite_activations():
    """A NaN or an infinity in a row gives that row NaN results (the f32 product
    would give NaN or infinity there) and leaves the other rows alone."""
    K, N, M = 1536, 256, 8
    q, s = ops.quantize_w8(make_weight(K, N, 78))
    packed = ops.pack_w8(q)
    rng = np.random.default_rng(6)
    xh = rng.standard_normal((M, K)).astype(np.float32)
    xh[2, 7] = np.nan
    xh[5, 1000] = -np.inf
    y = ops.gemv_w8a32(torch.from_numpy(xh).cuda(), packed, s, K, N).cpu().numpy()
    assert np.isnan(y[2]).all() and np.isnan(y[5]).all()
    assert np.isfinite(np.delete(y, [2, 5], 0)).all()


def test_gemv_accumulates_into_c(oracle):
    K, N, M = 1536, 1536, 2
    q, s = ops.quantize_w8(make_weight(K, N, 5))
    packed = ops.pack_w8(q)
    g = torch.Generator(device="cuda").manual_seed(9)
    x = torch.randn((M, K), generator=g, device="cuda")
    c0 = torch.randn((M, N), generator=g, device="cuda")
    c = c0.clone()
    ops.gemv_w8a32(x, packed, s, K, N, out=c, accumulate=True)
    # deterministic: a second launch gives the same bits
    c2 = c0.clone()
    ops.gemv_w8a32(x, packed, s, K, N, out=c2, accumulate=True)
    torch.cuda.synchronize()
    qh, sh, xh, ch = q.cpu().numpy(), s.cpu().numpy(), x.cpu().numpy(), c0.cpu().numpy()
    want = np.stack([oracle.dequant_gemv(xh[m], qh, sh, ch[m]) for m in range(M)])
    check_close(c.cpu().numpy(), want)
    np.testing.assert_array_equal(c.cpu().numpy(), c2.cpu().numpy())


def test_gemv_reference_known_answer_through_memref_abi(bh):
    # examples/BuddyMatmul/dequant-matmul-vectorization-decode.mlir:97-123,
    # host descriptors in, malloc'd host result out
    A = np.ones((1, 8), np.float32)
    W = np.zeros((8, 8), np.int8)
    W[:, :2] = 2
    S = np.full((1, 8), 0.5, np.float32)
    res = bma.MemRefF32_2D()
    a = bma.MemRef(A.ctypes.data, [1, 8])
    w = bma.MemRef(W.ctypes.data, [8, 8], ctype=ctypes.c_int8)
    s = bma.MemRef(S.ctypes.data, [1, 8])
    bh._mlir_ciface_buddy_dequant_matmul_i8_f32(ctypes.byref(res), ctypes.byref(a),
                                                ctypes.byref(w), ctypes.byref(s))
    assert res.aligned, bh.buddy_hip_last_error()
    assert list(res.sizes) == [1, 8] and list(res.strides) == [8, 1]
    out = np.ctypeslib.as_array(res.aligned, shape=(1, 8)).copy()
    ctypes.CDLL(None).free(res.allocated)
    assert out.tolist() == [[8, 8, 0, 0, 0, 0, 0, 0]]
    bh.buddy_hip_clear_weight_cache()


def test_memref_abi_strided_inputs_and_accumulate(bh, oracle):
    rng = np.random.default_rng(3)
    M, K, N = 3, 200, 48
    Abig = rng.normal(0, 1, (M, 2 * K)).astype(np.float32)  # A = every 2nd column
    W = rng.integers(-128, 128, (K, N)).astype(np.int8)
    S = rng.uniform(1e-4, 1e-3, (1, N)).astype(np.float32)
    C = rng.normal(0, 1, (M, N)).astype(np.float32)
    C0 = C.copy()
    a = bma.MemRef(Abig.ctypes.data, [M, K], strides=[2 * K, 2])
    w = bma.MemRef(W.ctypes.data, [K, N], ctype=ctypes.c_int8)
    s = bma.MemRef(S.ctypes.data, [1, N])
    c = bma.MemRef(C.ctypes.data, [M, N])
    bh._mlir_ciface_buddy_dequant_matmul_i8_f32_acc(ctypes.byref(c), ctypes.byref(a),
                                                    ctypes.byref(w), ctypes.byref(s))
    A = np.ascontiguousarray(Abig[:, ::2])
    want = np.stack([oracle.dequant_gemv(A[m], W, S, C0[m]) for m in range(M)])
    check_close(C, want)
    bh.buddy_hip_clear_weight_cache()


def test_memref_abi_block_of_rows_takes_the_matrix_cores(bh, oracle):
    # M above the GEMV's 16 rows: the prefill-shaped call through the operator
    # symbol; all f32 bits of the activations are carried, NaN propagates
    rng = np.random.default_rng(5)
    M, K, N = 77, 300, 200
    A = rng.normal(0, 1, (M, K)).astype(np.float32)
    A[3] *= 1e20
    A[5] *= 1e-20
    W = rng.integers(-128, 128, (K, N)).astype(np.int8)
    S = rng.uniform(1e-4, 1e-3, (1, N)).astype(np.float32)
    res = bma.MemRefF32_2D()
    a = bma.MemRef(A.ctypes.data, [M, K])
    w = bma.MemRef(W.ctypes.data, [K, N], ctype=ctypes.c_int8)
    s = bma.MemRef(S.ctypes.data, [1, N])
    bh._mlir_ciface_buddy_dequant_matmul_i8_f32(ctypes.byref(res), ctypes.byref(a),
                                                ctypes.byref(w), ctypes.byref(s))
    assert res.aligned, bh.buddy_hip_last_error()
    out = np.ctypeslib.as_array(res.aligned, shape=(M, N)).copy()
    ctypes.CDLL(None).free(res.allocated)
    want = oracle.blis_gemm_w8a32(A, W, S)
    for m in range(M):  # rows differ by 40 orders of magnitude: compare row by row
        check_close(out[m], want[m])
    # accumulate into a strided host C
    Cbig = rng.normal(0, 1, (M, N + 8)).astype(np.float32)
    C0 = Cbig[:, :N].copy()
    c = bma.MemRef(Cbig.ctypes.data, [M, N], strides=[N + 8, 1])
    A[3] /= 1e20
    A[5] /= 1e-20
    bh._mlir_ciface_buddy_dequant_matmul_i8_f32_acc(ctypes.byref(c), ctypes.byref(a),
                                                    ctypes.byref(w), ctypes.byref(s))
    check_close(Cbig[:, :N], oracle.blis_gemm_w8a32(A, W, S, C0.copy()))
    A[2, 7] = np.nan
    res = bma.MemRefF32_2D()
    bh._mlir_ciface_buddy_dequant_matmul_i8_f32(ctypes.byref(res), ctypes.byref(a),
                                                ctypes.byref(w), ctypes.byref(s))
    out = np.ctypeslib.as_array(res.aligned, shape=(M, N)).copy()
    ctypes.CDLL(None).free(res.allocated)
    assert np.isnan(out[2]).all() and not np.isnan(np.delete(out, 2, 0)).any()
    bh.buddy_hip_clear_weight_cache()


class WeightCacheInfo(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in ("entries", "bytes", "limit_bytes", "uploads",
                                              "evictions")]


def cache_info(bh):
    info = WeightCacheInfo()
    bh.buddy_hip_weight_cache_stats(ctypes.byref(info))
    return info


def dequant_matmul_host(bh, A, W, S):
    res = bma.MemRefF32_2D()
    a = bma.MemRef(A.ctypes.data, list(A.shape))
    w = bma.MemRef(W.ctypes.data, list(W.shape), ctype=ctypes.c_int8)
    s = bma.MemRef(S.ctypes.data, list(S.shape))
    bh._mlir_ciface_buddy_dequant_matmul_i8_f32(ctypes.byref(res), ctypes.byref(a),
                                                ctypes.byref(w), ctypes.byref(s))
    assert res.aligned, bh.buddy_hip_last_error()
    out = np.ctypeslib.as_array(res.aligned, shape=(A.shape[0], W.shape[1])).copy()
    ctypes.CDLL(None).free(res.allocated)
    return out


def test_weight_cache_sees_new_contents_at_the_same_address(bh, oracle):
    """The operator-level cache is keyed by the operands' addresses; a caller
    that frees a weight buffer and gets the same address back with other
    contents (or rewrites the buffer) must not be served the old packed copy."""
    bh.buddy_hip_clear_weight_cache()
    rng = np.random.default_rng(8)
    K, N = 320, 96
    A = rng.normal(0, 1, (2, K)).astype(np.float32)
    W = rng.integers(-128, 128, (K, N)).astype(np.int8)
    S = rng.uniform(1e-4, 1e-3, (1, N)).astype(np.float32)
    u0 = cache_info(bh).uploads
    out = dequant_matmul_host(bh, A, W, S)
    check_close(out, np.stack([oracle.dequant_gemv(A[m], W, S) for m in range(2)]))
    out = dequant_matmul_host(bh, A, W, S)          # a hit: no second upload
    assert cache_info(bh).uploads == u0 + 1 and cache_info(bh).entries == 1
    W[...] = rng.integers(-128, 128, (K, N)).astype(np.int8)   # same address, new weights
    out = dequant_matmul_host(bh, A, W, S)
    check_close(out, np.stack([oracle.dequant_gemv(A[m], W, S) for m in range(2)]))
    assert cache_info(bh).uploads == u0 + 2 and cache_info(bh).entries == 1
    S[...] = S[:, ::-1].copy()                      # new scales only
    out = dequant_matmul_host(bh, A, W, S)
    check_close(out, np.stack([oracle.dequant_gemv(A[m], W, S) for m in range(2)]))
    assert cache_info(bh).uploads == u0 + 3 and cache_info(bh).entries == 1
    # device-resident operands are fingerprinted too
    Wd, Sd = torch.from_numpy(W).cuda(), torch.from_numpy(S).cuda()
    w = bma.MemRef(Wd.data_ptr(), [K, N], ctype=ctypes.c_int8)
    s = bma.MemRef(Sd.data_ptr(), [1, N])
    a = bma.MemRef(A.ctypes.data, [2, K])

    def run_dev():
        res = bma.MemRefF32_2D()
        bh._mlir_ciface_buddy_dequant_matmul_i8_f32(ctypes.byref(res), ctypes.byref(a),
                                                    ctypes.byref(w), ctypes.byref(s))
        assert res.aligned, bh.buddy_hip_last_error()
        o = np.ctypeslib.as_array(res.aligned, shape=(2, N)).copy()
        ctypes.CDLL(None).free(res.allocated)
        return o

    check_close(run_dev(), np.stack([oracle.dequant_gemv(A[m], W, S) for m in range(2)]))
    W2 = rng.integers(-128, 128, (K, N)).astype(np.int8)
    Wd.copy_(torch.from_numpy(W2))
    torch.cuda.synchronize()
    check_close(run_dev(), np.stack([oracle.dequant_gemv(A[m], W2, S) for m in range(2)]))
    bh.buddy_hip_clear_weight_cache()
    assert cache_info(bh).entries == 0 and cache_info(bh).bytes == 0


def test_weight_cache_is_bounded_and_frees_the_least_recently_used(bh, oracle):
    bh.buddy_hip_clear_weight_cache()
    limit0 = cache_info(bh).limit_bytes
    rng = np.random.default_rng(9)
    K, N = 256, 64
    per_entry = bh.buddy_hip_w8_packed_bytes(K, N) + 4 * N
    bh.buddy_hip_set_weight_cache_limit(3 * per_entry)
    try:
        A = rng.normal(0, 1, (1, K)).astype(np.float32)
        Ws = [rng.integers(-128, 128, (K, N)).astype(np.int8) for _ in range(5)]
        S = rng.uniform(1e-4, 1e-3, (1, N)).astype(np.float32)
        Ss = [S.copy() for _ in range(5)]
        e0, u0 = cache_info(bh).evictions, cache_info(bh).uploads
        for i in range(3):
            dequant_matmul_host(bh, A, Ws[i], Ss[i])
        assert cache_info(bh).entries == 3 and cache_info(bh).bytes == 3 * per_entry
        dequant_matmul_host(bh, A, Ws[0], Ss[0])        # touch 0: 1 is now the oldest
        dequant_matmul_host(bh, A, Ws[3], Ss[3])        # evicts 1
        info = cache_info(bh)
        assert (info.entries, info.evictions - e0, info.uploads - u0) == (3, 1, 4)
        assert info.bytes <= info.limit_bytes
        dequant_matmul_host(bh, A, Ws[0], Ss[0])        # still cached
        assert cache_info(bh).uploads - u0 == 4
        out = dequant_matmul_host(bh, A, Ws[1], Ss[1])  # was freed: packed again, right result
        assert cache_info(bh).uploads - u0 == 5
        check_close(out, oracle.dequant_gemv(A[0], Ws[1], Ss[1])[None])
        bh.buddy_hip_set_weight_cache_limit(per_entry)   # shrinking frees at once
        assert cache_info(bh).entries == 1
    finally:
        bh.buddy_hip_set_weight_cache_limit(limit0)
        bh.buddy_hip_clear_weight_cache()


def test_bad_arguments_are_refused(bh):
    # null operands: message on stderr, result left null, nothing launched
    res = bma.MemRefF32_2D()
    bh._mlir_ciface_buddy_dequant_matmul_i8_f32(ctypes.byref(res), None, None, None)
    assert not res.aligned
    assert bh.buddy_hip_gemv_w8a32(None, None, None, None, 1, 64, 16, 0, None) != 0
    assert b"null" in bh.buddy_hip_last_error()
