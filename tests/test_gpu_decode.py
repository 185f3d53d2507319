"""GPU parity of the decode-step pieces and of whole decode steps against the
CPU oracle: attention (with fused RoPE + KV write), fused linear epilogues,
argmax, and the resident session (logits, KV rows written, greedy tokens)."""
import ctypes

import numpy as np
import pytest
import torch

import buddy_mlir_amd as bma
import oracle_lib
from buddy_mlir_amd import ops, synthetic
from buddy_mlir_amd.session import Shape
from parity import check_close

pytestmark = pytest.mark.gpu

EPS = np.float32(1e-6)


def dev(a, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda", dtype)


def linear(bh, **kw):
    torch.cuda.synchronize()
    ops.linear_w8a32(stream=None, **kw)
    torch.cuda.synchronize()


def mlp_block_oracle(oracle, xh, qg, sg, qu, su, qd, sd, norm_w=None, eps=None, y0=None):
    """The block on the CPU: M = 1 follows the decode GEMV kernel, more rows the
    BLIS kernel (the only vectorised reference kernel for M > 1)."""
    M = xh.shape[0]
    if norm_w is not None:
        xh = np.stack([oracle.rmsnorm(r, norm_w, eps, np.float32(1.0) / np.float32(xh.shape[1]))
                       for r in xh])
    if M == 1:
        g = oracle.dequant_gemv(xh[0], qg, sg)[None]
        u = oracle.dequant_gemv(xh[0], qu, su)[None]
    else:
        g = oracle.blis_gemm_w8a32(xh, qg, sg)
        u = oracle.blis_gemm_w8a32(xh, qu, su)
    hh = np.stack([oracle.silu_mul(g[m], u[m]) for m in range(M)])
    if M == 1:
        return oracle.dequant_gemv(hh[0], qd, sd, None if y0 is None else y0[0])[None]
    return oracle.blis_gemm_w8a32(hh, qd, sd, None if y0 is None else y0.copy())


@pytest.mark.parametrize("M", [1, 4, 5, 8, 9, 13, 16])
def test_mlp_block_entry_point_matches_oracle(bh, oracle, M):
    """BASELINE configs[1] through the one call made for it: 1536 <-> 8960,
    plain, and with the RMSNorm in front and the residual behind that a decoder
    layer has."""
    H, I = 1536, 8960
    qg, sg = synthetic.quantized_linear(H, I, 11)
    qu, su = synthetic.quantized_linear(H, I, 12)
    qd, sd = synthetic.quantized_linear(I, H, 13)
    g = torch.Generator(device="cuda").manual_seed(M)
    x = torch.randn((M, H), generator=g, device="cuda")
    if M > 2:
        x[1] *= 1e-6   # rows of very different size (h goes with the square): the
        x[2] *= 1e5    # steps are per row
    w = 1 + 0.1 * torch.randn(H, generator=g, device="cuda")
    y0 = torch.randn((M, H), generator=g, device="cuda")
    pg, pu, pd = ops.pack_w8(qg), ops.pack_w8(qu), ops.pack_w8(qd)
    torch.cuda.synchronize()
    y = ops.mlp_block_w8a32(x, pg, sg, pu, su, pd, sd, H, I)
    y2 = y0.clone()
    ops.mlp_block_w8a32(x, pg, sg, pu, su, pd, sd, H, I, y=y2, norm_w=w, norm_eps=1e-6,
                        accumulate=True)
    torch.cuda.synchronize()
    hq = [t.cpu().numpy() for t in (qg, sg, qu, su, qd, sd)]
    want = mlp_block_oracle(oracle, x.cpu().numpy(), *hq)
    want2 = mlp_block_oracle(oracle, x.cpu().numpy(), *hq, norm_w=w.cpu().numpy(),
                             eps=np.float32(1e-6), y0=y0.cpu().numpy())
    got, got2 = y.cpu().numpy(), y2.cpu().numpy()
    for m in range(M):
        check_close(got[m], want[m])
        check_close(got2[m], want2[m])


@pytest.mark.parametrize("M,H,I", [(7, 256, 100), (16, 64, 33), (5, 192, 70), (11, 320, 1000),
                                   (8, 128, 64), (16, 1536, 96)])
def test_mlp_block_ragged_shapes(bh, oracle, M, H, I):
    """Intermediate sizes that end inside a tile of 64 k or inside a channel
    group."""
    qg, sg = synthetic.quantized_linear(H, I, 21)
    qu, su = synthetic.quantized_linear(H, I, 22)
    qd, sd = synthetic.quantized_linear(I, H, 23)
    x = torch.randn((M, H), generator=torch.Generator(device="cuda").manual_seed(M + I),
                    device="cuda") * 3
    y = ops.mlp_block_w8a32(x, ops.pack_w8(qg), sg, ops.pack_w8(qu), su, ops.pack_w8(qd), sd, H, I)
    torch.cuda.synchronize()
    want = mlp_block_oracle(oracle, x.cpu().numpy(),
                            *[t.cpu().numpy() for t in (qg, sg, qu, su, qd, sd)])
    got = y.cpu().numpy()
    for m in range(M):
        check_close(got[m], want[m])


def test_mlp_block_non_finite_rows_and_refusals(bh, oracle):
    H, I, M = 256, 512, 9
    qg, sg = synthetic.quantized_linear(H, I, 31)
    qu, su = synthetic.quantized_linear(H, I, 32)
    qd, sd = synthetic.quantized_linear(I, H, 33)
    pg, pu, pd = ops.pack_w8(qg), ops.pack_w8(qu), ops.pack_w8(qd)
    x = torch.randn((M, H), generator=torch.Generator(device="cuda").manual_seed(3), device="cuda")
    clean = ops.mlp_block_w8a32(x, pg, sg, pu, su, pd, sd, H, I).cpu().numpy()
    x[2, 5] = float("nan")
    x[7, 0] = float("inf")
    got = ops.mlp_block_w8a32(x, pg, sg, pu, su, pd, sd, H, I).cpu().numpy()
    assert np.isnan(got[[2, 7]]).all()
    rest = [m for m in range(M) if m not in (2, 7)]
    np.testing.assert_array_equal(got[rest], clean[rest])
    # a workspace that is too small, and too many rows
    y = torch.empty((M, H), device="cuda")
    d, ws = ops.mlp_block_desc(x, pg, sg, pu, su, pd, sd, y, H, I)
    d.workspace_bytes = 16
    assert bh.buddy_hip_mlp_block_w8a32(ctypes.byref(d), None) != 0
    assert b"workspace" in bh.buddy_hip_last_error()
    assert bh.buddy_hip_mlp_block_workspace_bytes(17, I) == 0


@pytest.mark.parametrize("M", [1, 4, 16])
def test_mlp_block_matches_oracle(bh, oracle, M):
    """h = SiLU(x.G) * (x.U); y = h.D -- the fused gate|up kernel and the down
    projection.  M = 1 follows the decode GEMV kernel, M = 4 / 16 the BLIS
    kernel, the only vectorised reference kernel for M > 1."""
    H, I = 1536, 8960
    qg, sg = synthetic.quantized_linear(H, I, 11)
    qu, su = synthetic.quantized_linear(H, I, 12)
    qd, sd = synthetic.quantized_linear(I, H, 13)
    x = torch.randn((M, H), generator=torch.Generator(device="cuda").manual_seed(M),
                    device="cuda")
    h = torch.empty((M, I), device="cuda")
    y = torch.empty((M, H), device="cuda")
    linear(bh, A=x, lda=H, W0=ops.pack_w8(qg), scale0=sg, W1=ops.pack_w8(qu),
           scale1=su, C=h, ldc=I, M=M, K=H, N=I, epilogue=2)
    linear(bh, A=h, lda=I, W0=ops.pack_w8(qd), scale0=sd, C=y, ldc=H, M=M, K=I,
           N=H, epilogue=0)
    xh = x.cpu().numpy()
    qg, sg, qu, su, qd, sd = (t.cpu().numpy() for t in (qg, sg, qu, su, qd, sd))
    if M == 1:
        g = oracle.dequant_gemv(xh[0], qg, sg)[None]
        u = oracle.dequant_gemv(xh[0], qu, su)[None]
    else:
        g = oracle.blis_gemm_w8a32(xh, qg, sg)
        u = oracle.blis_gemm_w8a32(xh, qu, su)
    hh = np.stack([oracle.silu_mul(g[m], u[m]) for m in range(M)])
    want = (oracle.dequant_gemv(hh[0], qd, sd)[None] if M == 1
            else oracle.blis_gemm_w8a32(hh, qd, sd))
    check_close(h.cpu().numpy(), hh)
    check_close(y.cpu().numpy(), want)


def test_norm_prologue_and_residual_epilogue(bh, oracle):
    K, N = 1536, 2048
    q, s = synthetic.quantized_linear(K, N, 21)
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn((2, K), generator=g, device="cuda") * 3
    w = 1 + 0.1 * torch.randn(K, generator=g, device="cuda")
    bias = torch.randn(N, generator=g, device="cuda")
    out = torch.empty((2, N), device="cuda")
    linear(bh, A=x, lda=K, W0=ops.pack_w8(q), scale0=s, norm_w=w, norm_eps=float(EPS),
           bias=bias, C=out, ldc=N, M=2, K=K, N=N, epilogue=0)
    xh, wh, qh, sh, bh_ = (t.cpu().numpy() for t in (x, w, q, s, bias))
    want = np.stack([bh_ + oracle.dequant_gemv(oracle.rmsnorm(xh[m], wh, EPS), qh, sh)
                     for m in range(2)])
    check_close(out.cpu().numpy(), want)
    # narrow tiles (8 and 4 channels per tile) at M = 1: same result
    for tn in (8, 4):
        out1 = torch.empty((1, N), device="cuda")
        linear(bh, A=x, lda=K, W0=ops.pack_w8_tiles(q, tn), scale0=s, norm_w=w,
               norm_eps=float(EPS), bias=bias, C=out1, ldc=N, M=1, K=K, N=N, epilogue=0,
               tile_n=tn)
        check_close(out1.cpu().numpy()[0], want[0])
    # residual: C += ...
    c0 = torch.randn((2, N), generator=g, device="cuda")
    c = c0.clone()
    linear(bh, A=x, lda=K, W0=ops.pack_w8(q), scale0=s, C=c, ldc=N, M=2, K=K, N=N,
           epilogue=1)
    want = np.stack([oracle.dequant_gemv(xh[m], qh, sh, c0.cpu().numpy()[m])
                     for m in range(2)])
    check_close(c.cpu().numpy(), want)


# (192, 131072): a matrix wide enough for eight channel groups per wavefront
# with an odd number of chunks per wavefront: its last fetch of the ring is a
# repeat that is still in flight when the loop ends (a temporary of the RMSNorm
# reduction once landed in one of its registers)
@pytest.mark.parametrize("M", [3, 9, 16])
@pytest.mark.parametrize("K,N", [(1536, 2048), (8960, 1536), (200, 48), (192, 131072)])
def test_small_batch_fusions(bh, oracle, M, K, N):
    """RMSNorm + bias, residual add and SiLU*mul at batch sizes that run on the
    f32 FMA kernel (M <= 4) and on the matrix-core kernel (M >= 5)."""
    q, s = synthetic.quantized_linear(K, N, 31)
    q2, s2 = synthetic.quantized_linear(K, N, 32)
    g = torch.Generator(device="cuda").manual_seed(100 + M)
    x = torch.randn((M, K), generator=g, device="cuda") * 2
    w = 1 + 0.1 * torch.randn(K, generator=g, device="cuda")
    bias = torch.randn(N, generator=g, device="cuda")
    p, p2 = ops.pack_w8(q), ops.pack_w8(q2)
    xh, wh, qh, sh, q2h, s2h, bh_ = (t.cpu().numpy() for t in (x, w, q, s, q2, s2, bias))
    xn = np.stack([oracle.rmsnorm(xh[m], wh, EPS) for m in range(M)])
    # norm + bias
    out = torch.empty((M, N), device="cuda")
    linear(bh, A=x, lda=K, W0=p, scale0=s, norm_w=w, norm_eps=float(EPS), bias=bias,
           C=out, ldc=N, M=M, K=K, N=N, epilogue=0)
    want = np.stack([bh_ + oracle.dequant_gemv(xn[m], qh, sh) for m in range(M)])
    check_close(out.cpu().numpy(), want)
    # norm + SiLU(gate) * up
    h = torch.empty((M, N), device="cuda")
    linear(bh, A=x, lda=K, W0=p, scale0=s, W1=p2, scale1=s2, norm_w=w,
           norm_eps=float(EPS), C=h, ldc=N, M=M, K=K, N=N, epilogue=2)
    want = np.stack([oracle.silu_mul(oracle.dequant_gemv(xn[m], qh, sh),
                                     oracle.dequant_gemv(xn[m], q2h, s2h))
                     for m in range(M)])
    check_close(h.cpu().numpy(), want)
    # residual: C += ...
    c0 = torch.randn((M, N), generator=g, device="cuda")
    c = c0.clone()
    linear(bh, A=x, lda=K, W0=p, scale0=s, C=c, ldc=N, M=M, K=K, N=N, epilogue=1)
    want = np.stack([oracle.dequant_gemv(xh[m], qh, sh, c0.cpu().numpy()[m])
                     for m in range(M)])
    check_close(c.cpu().numpy(), want)


def test_standalone_elementwise_and_argmax(bh, oracle):
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn((3, 1536), generator=g, device="cuda") * 2
    w = 1 + 0.1 * torch.randn(1536, generator=g, device="cuda")
    y = torch.empty_like(x)
    torch.cuda.synchronize()
    bma.check(bh.buddy_hip_rmsnorm(x.data_ptr(), w.data_ptr(), y.data_ptr(), 3, 1536,
                                   float(EPS), None))
    torch.cuda.synchronize()
    for m in range(3):
        check_close(y[m].cpu().numpy(), oracle.rmsnorm(x[m].cpu().numpy(), w.cpu().numpy(), EPS))
    # RoPE
    inv = synthetic.inv_freq(128)
    qk = torch.randn((12, 128), generator=g, device="cuda")
    want_in = qk.cpu().numpy()
    pos = torch.tensor([777], dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    bma.check(bh.buddy_hip_rope(qk.data_ptr(), inv.data_ptr(), pos.data_ptr(), 12, 128, None))
    torch.cuda.synchronize()
    c, s = oracle.rope_cos_sin(inv.cpu().numpy(), 777)
    check_close(qk.cpu().numpy(), oracle.rope_apply(want_in, c, s))
    # SiLU*mul
    a = torch.randn(8960, generator=g, device="cuda") * 3
    b = torch.randn(8960, generator=g, device="cuda")
    h = torch.empty_like(a)
    torch.cuda.synchronize()
    bma.check(bh.buddy_hip_silu_mul(a.data_ptr(), b.data_ptr(), h.data_ptr(), 8960, None))
    torch.cuda.synchronize()
    check_close(h.cpu().numpy(), oracle.silu_mul(a.cpu().numpy(), b.cpu().numpy()))
    # argmax: first maximum on ties
    v = torch.randn(151936, generator=g, device="cuda")
    v[[100, 5000, 151935]] = 50.0
    ws = torch.empty(bh.buddy_hip_argmax_workspace_bytes(), dtype=torch.uint8, device="cuda")
    out = torch.zeros(1, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    bma.check(bh.buddy_hip_argmax(v.data_ptr(), 151936, ws.data_ptr(), out.data_ptr(), None))
    torch.cuda.synchronize()
    assert int(out.item()) == 100 == oracle.argmax_first(v.cpu().numpy())


def test_decode_attention_refuses_unaligned_operands(bh):
    """The kernels read qkv, inv_freq and the caches four floats at a time."""
    H, HKV, D, L = 4, 2, 128, 64
    t = torch.zeros((H + 2 * HKV) * D + 2 * HKV * L * D + D + 8, device="cuda")
    pos_t = torch.zeros(1, dtype=torch.int32, device="cuda")
    nb = bh.buddy_hip_attn_decode_workspace_bytes(H, L)
    ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
    out = torch.empty(H * D, device="cuda")
    p = t.data_ptr()
    for off in ((4, 0, 0), (0, 4, 0), (0, 0, 4)):
        rc = bh.buddy_hip_gqa_decode_attention(
            p + off[0], p + off[1], pos_t.data_ptr(), p + off[2], p, out.data_ptr(), None,
            H, HKV, D, L, 0.088, ws.data_ptr(), nb, None)
        assert rc == 1 and b"16-byte aligned" in bh.buddy_hip_last_error()


@pytest.mark.parametrize("pos", [0, 8, 31, 32, 36, 612, 1023, 1087])
def test_decode_attention_with_rope_and_kv_write(bh, oracle, pos):
    """valid lengths 9/37/613/1024 are the reference's own check points
    (frontend/Python/ops/tosa.py:14075-14080); 0/31/32 sit on chunk edges."""
    H, HKV, D, L = 12, 2, 128, 1088
    g = torch.Generator(device="cuda").manual_seed(pos + 1)
    qkv = torch.randn((H + 2 * HKV) * D, generator=g, device="cuda")
    kc = torch.randn((HKV, L, D), generator=g, device="cuda")
    vc = torch.randn((HKV, L, D), generator=g, device="cuda")
    kc[:, pos:, :] = 1e30  # rows at and beyond pos must not be read (pos is rewritten)
    vc[:, pos:, :] = 1e30
    inv = synthetic.inv_freq(D)
    out = torch.empty(H * D, device="cuda")
    lse = torch.empty(H, device="cuda")
    pos_t = torch.tensor([pos], dtype=torch.int32, device="cuda")
    nb = bh.buddy_hip_attn_decode_workspace_bytes(H, L)
    ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
    kch, vch, qh = kc.cpu().numpy().copy(), vc.cpu().numpy().copy(), qkv.cpu().numpy()
    scale = np.float32(0.0883883461)
    torch.cuda.synchronize()
    bma.check(bh.buddy_hip_gqa_decode_attention(
        qkv.data_ptr(), inv.data_ptr(), pos_t.data_ptr(), kc.data_ptr(), vc.data_ptr(),
        out.data_ptr(), lse.data_ptr(), H, HKV, D, L, float(scale), ws.data_ptr(), nb, None))
    torch.cuda.synchronize()
    # oracle: RoPE, cache write, then attention over the whole cache with the mask
    c, s = oracle.rope_cos_sin(inv.cpu().numpy(), pos)
    q = oracle.rope_apply(qh[:H * D].reshape(H, D), c, s)
    k = oracle.rope_apply(qh[H * D:(H + HKV) * D].reshape(HKV, D), c, s)
    v = qh[(H + HKV) * D:].reshape(HKV, D)
    kch[:, pos, :] = k
    vch[:, pos, :] = v
    kch[:, pos + 1:, :] = 0  # the oracle multiplies masked rows by exactly 0
    vch[:, pos + 1:, :] = 0
    mask = np.where(np.arange(L) <= pos, 0.0, -np.inf).astype(np.float32)
    want, want_lse = oracle.gqa_decode_attention(q, kch, vch, mask, scale, 4)
    check_close(out.cpu().numpy().reshape(H, D), want)
    # the op's second result: lse = m + log l per head (tosa.py:14576-14594)
    check_close(lse.cpu().numpy(), want_lse)
    # the new K/V rows landed in the cache, nothing else moved
    check_close(kc[:, pos, :].cpu().numpy(), k)
    np.testing.assert_array_equal(vc[:, pos, :].cpu().numpy(), v)
    if pos:
        np.testing.assert_array_equal(kc[:, :pos, :].cpu().numpy(), kch[:, :pos, :])


def oracle_model(oracle, shape: Shape, host):
    return oracle_lib.model_from_host(oracle, shape, host)


SMALL = Shape(layers=2, hidden=256, heads=4, kv_heads=2, head_dim=128, inter=512,
              vocab=1024, max_len=128, rms_eps=1e-6)


@pytest.mark.parametrize("graph", [False, True])
def test_small_model_logits_kv_and_tokens(oracle, graph):
    sess, host = synthetic.build_session(SMALL, context=40, keep_host=True, ln_jitter=0.1)
    sess.use_graph(graph)
    om = oracle_model(oracle, SMALL, host)
    kv = [a.copy() for a in host["kv"]]
    tok, toks_gpu, toks_cpu = 17, [], []
    for step in range(12):
        pos = 40 + step
        nxt, logits = sess.decode(tok, pos)
        otok, ologits = om.decode_step(tok, pos, kv)
        check_close(logits, ologits)
        toks_gpu.append(nxt)
        toks_cpu.append(otok)
        tok = otok
    assert toks_gpu == toks_cpu
    # every cache row the steps wrote matches the oracle's
    for j in range(2 * SMALL.layers):
        got = sess.get_kv(j)
        check_close(got[:, 40:52, :], kv[j][:, 40:52, :])
        np.testing.assert_array_equal(got[:, :40, :], host["kv"][j][:, :40, :])
    sess.close()


@pytest.mark.parametrize("pos", [4095, 4096, 8191])
def test_decode_attention_long_context(bh, oracle, pos):
    """Contexts far beyond the model's shipped 1024: more than 64 chunks per head."""
    H, HKV, D, L = 4, 2, 128, 8192
    g = torch.Generator(device="cuda").manual_seed(pos)
    qkv = torch.randn((H + 2 * HKV) * D, generator=g, device="cuda")
    kc = torch.randn((HKV, L, D), generator=g, device="cuda")
    vc = torch.randn((HKV, L, D), generator=g, device="cuda")
    inv = synthetic.inv_freq(D)
    out = torch.empty(H * D, device="cuda")
    pos_t = torch.tensor([pos], dtype=torch.int32, device="cuda")
    nb = bh.buddy_hip_attn_decode_workspace_bytes(H, L)
    ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
    kch, vch, qh = kc.cpu().numpy().copy(), vc.cpu().numpy().copy(), qkv.cpu().numpy()
    scale = np.float32(0.0883883461)
    torch.cuda.synchronize()
    bma.check(bh.buddy_hip_gqa_decode_attention(
        qkv.data_ptr(), inv.data_ptr(), pos_t.data_ptr(), kc.data_ptr(), vc.data_ptr(),
        out.data_ptr(), None, H, HKV, D, L, float(scale), ws.data_ptr(), nb, None))
    torch.cuda.synchronize()
    c, s = oracle.rope_cos_sin(inv.cpu().numpy(), pos)
    q = oracle.rope_apply(qh[:H * D].reshape(H, D), c, s)
    kch[:, pos, :] = oracle.rope_apply(qh[H * D:(H + HKV) * D].reshape(HKV, D), c, s)
    vch[:, pos, :] = qh[(H + HKV) * D:].reshape(HKV, D)
    kch[:, pos + 1:, :] = 0
    vch[:, pos + 1:, :] = 0
    mask = np.where(np.arange(L) <= pos, 0.0, -np.inf).astype(np.float32)
    want, _ = oracle.gqa_decode_attention(q, kch, vch, mask, scale, 4)
    check_close(out.cpu().numpy().reshape(H, D), want)


def test_small_model_decodes_at_long_context(oracle):
    """A cache of 4352 positions (68 chunks of 64: the o_proj kernel folds them in
    two passes) filled to 4300, then greedy steps against the oracle."""
    shape = Shape(layers=2, hidden=256, heads=4, kv_heads=2, head_dim=128, inter=512,
                  vocab=1024, max_len=4352, rms_eps=1e-6)
    sess, host = synthetic.build_session(shape, context=4300, keep_host=True, ln_jitter=0.1)
    om = oracle_model(oracle, shape, host)
    kv = [a.copy() for a in host["kv"]]
    tok = 9
    for step in range(6):
        nxt, logits = sess.decode(tok, 4300 + step)
        otok, ologits = om.decode_step(tok, 4300 + step, kv)
        check_close(logits, ologits)
        assert nxt == otok
        tok = otok
    sess.close()


@pytest.mark.parametrize("start", [100, 1140, 2296, 4596, 5110, 12535, 16375])
def test_small_model_steps_across_the_attention_chunk_sizes(oracle, start):
    """A step far into a long cache takes attention chunks of 128 or 256 positions
    (from positions 1152 and 2304 on), covers only the chunks up to its position,
    and from position 5120 on folds the partials in a launch of its own instead of
    in the o_proj launch: greedy steps that cross each boundary, a short context
    in a large cache, and the positions at which the launches that take the heads
    of a KV head together change their cut (12544 and 16384 with two KV
    heads), against the oracle -- every step's logits and the token fed back on
    the device."""
    shape = Shape(layers=2, hidden=256, heads=4, kv_heads=2, head_dim=128, inter=512,
                  vocab=1024, max_len=(start + 100 + 63) // 64 * 64 if start > 4400 else 4352,
                  rms_eps=1e-6)
    sess, host = synthetic.build_session(shape, context=start, keep_host=True, ln_jitter=0.1)
    om = oracle_model(oracle, shape, host)
    kv = [a.copy() for a in host["kv"]]
    tok = 7
    for step in range(20):
        nxt, logits = sess.decode(tok, start + step)
        otok, ologits = om.decode_step(tok, start + step, kv)
        check_close(logits, ologits)
        assert nxt == otok
        tok = otok
    # the same stretch again as one call (the cache rows are rewritten with the
    # same values)
    toks = sess.decode_greedy(7, start, 20)
    kv2 = [a.copy() for a in host["kv"]]
    t, want = 7, []
    for step in range(20):
        t, _ = om.decode_step(t, start + step, kv2)
        want.append(t)
    assert toks.tolist() == want
    sess.close()


@pytest.mark.parametrize("heads,kv_heads", [(1, 1), (3, 1), (5, 1), (6, 1), (8, 1), (12, 2), (8, 4)])
def test_long_context_steps_for_every_size_of_head_group(oracle, heads, kv_heads):
    """From position 5120 on a workgroup takes all the query heads of a KV head, or,
    where there are few KV heads, half of them (a group of 3 or 5 splits unevenly, a
    group of one not at all): steps that cross that position against the oracle."""
    start = 5114
    shape = Shape(layers=1, hidden=256, heads=heads, kv_heads=kv_heads, head_dim=128, inter=256,
                  vocab=512, max_len=5184, rms_eps=1e-6)
    sess, host = synthetic.build_session(shape, context=start, keep_host=True, ln_jitter=0.1)
    om = oracle_model(oracle, shape, host)
    kv = [a.copy() for a in host["kv"]]
    tok = 3
    for step in range(12):
        nxt, logits = sess.decode(tok, start + step)
        otok, ologits = om.decode_step(tok, start + step, kv)
        check_close(logits, ologits)
        assert nxt == otok
        tok = otok
    for j in range(2):
        check_close(sess.get_kv(j)[:, start:start + 12, :], kv[j][:, start:start + 12, :])
    sess.close()


@pytest.mark.parametrize("start", [17000, 66000])
def test_fold_of_more_partials_than_one_pass_takes(oracle, start):
    """The launch that folds the partials far into a long cache takes 128 of them
    per head in its first pass and keeps the (max, sum) pairs of up to 256 in
    registers: with one KV head 17000 positions are 136 partials of 128
    positions, 66000 are 260 of 256."""
    shape = Shape(layers=1, hidden=256, heads=2, kv_heads=1, head_dim=128, inter=256,
                  vocab=512, max_len=start + 64, rms_eps=1e-6)
    sess, host = synthetic.build_session(shape, context=start, keep_host=True, ln_jitter=0.1)
    om = oracle_model(oracle, shape, host)
    kv = [a.copy() for a in host["kv"]]
    tok = 3
    for step in range(4):
        nxt, logits = sess.decode(tok, start + step)
        otok, ologits = om.decode_step(tok, start + step, kv)
        check_close(logits, ologits)
        assert nxt == otok
        tok = otok
    sess.close()


def test_a_long_generation_outlives_the_captured_steps_it_keeps():
    """A session keeps a captured step per cut of the attention and lets the oldest
    go after eight: 5200 greedy steps from position 5000 pass more cuts than that
    (a new one every 512 positions), and must give the tokens of the same steps
    launched one by one without a graph."""
    shape = Shape(layers=1, hidden=256, heads=4, kv_heads=2, head_dim=128, inter=256,
                  vocab=512, max_len=10368, rms_eps=1e-6)
    start, steps = 5000, 5200
    toks = []
    for graph in (True, False):
        sess, _ = synthetic.build_session(shape, context=start, ln_jitter=0.1)
        sess.use_graph(graph)
        toks.append(sess.decode_greedy(3, start, steps))
        sess.close()
    assert toks[0].tolist() == toks[1].tolist()


def test_small_model_greedy_feedback_matches_stepwise(oracle):
    sess, host = synthetic.build_session(SMALL, context=16, keep_host=True, ln_jitter=0.1)
    toks = sess.decode_greedy(5, 16, 24)
    om = oracle_model(oracle, SMALL, host)
    kv = [a.copy() for a in host["kv"]]
    tok, want = 5, []
    for step in range(24):
        tok, _ = om.decode_step(tok, 16 + step, kv)
        want.append(tok)
    assert toks.tolist() == want
    sess.close()


def test_session_refuses_bad_arguments(bh):
    sess, _ = synthetic.build_session(SMALL, context=0)
    with pytest.raises(bma.BuddyHipError):
        sess.decode(5, SMALL.max_len)  # position beyond the cache
    with pytest.raises(bma.BuddyHipError):
        sess.decode(SMALL.vocab, 0)  # token id out of range
    with pytest.raises(bma.BuddyHipError):
        sess.decode_greedy(1, SMALL.max_len - 3, 8)  # would run off the cache
    # asynchronous steps are bounded on the host as well: the device advances
    # its own position and step counter, and nothing may run off the cache or
    # the token log
    with pytest.raises(bma.BuddyHipError):
        sess.enqueue_steps(1)  # no token / position set yet
    sess.set_state(5, SMALL.max_len - 4)
    with pytest.raises(bma.BuddyHipError):
        sess.enqueue_steps(5)  # the fifth step would write row max_len
    assert b"leave the cache" in bh.buddy_hip_last_error()
    sess.enqueue_steps(3)
    with pytest.raises(bma.BuddyHipError):
        sess.enqueue_steps(2)  # refused as a whole: one row is left
    sess.enqueue_steps(1)
    with pytest.raises(bma.BuddyHipError):
        sess.enqueue_steps(1)
    torch.cuda.synchronize()
    sess.close()
    bad = Shape(head_dim=64)
    with pytest.raises(bma.BuddyHipError):
        bma.session.DecoderSession(bad)


@pytest.mark.timeout(900)
def test_qwen2_1p5b_shape_64_greedy_steps(oracle):
    """BASELINE config 3: 28 layers, hidden 1536, 12/2 heads, inter 8960, vocab
    151936, context 1024, 64 greedy steps.  Token ids must match the oracle for
    all 64 steps; logits are compared on the first and last step."""
    shape = Shape()
    sess, host = synthetic.build_session(shape, context=1024, keep_host=True)
    first = int(synthetic.first_tokens(shape, 1)[0])
    _, logits0 = sess.decode(first, 1024)  # step 0 once more, for its logits
    toks = sess.decode_greedy(first, 1024, 64)
    om = oracle_model(oracle, shape, host)
    kv = host["kv"]
    tok, want, margins = first, [], []
    for step in range(64):
        tok, logits = om.decode_step(tok, 1024 + step, kv)
        if step == 0:
            check_close(logits0, logits)
        top2 = np.partition(logits, -2)[-2:]
        margins.append(float(top2[1] - top2[0]))
        want.append(tok)
    got = toks.tolist()
    diverge = next((i for i in range(64) if got[i] != want[i]), None)
    assert diverge is None, (f"first divergence at step {diverge}, top-2 logit margin "
                             f"there {margins[diverge]:.3e}")
    # the 64 cache rows the run wrote, last layer
    for j in (2 * shape.layers - 2, 2 * shape.layers - 1):
        check_close(sess.get_kv(j)[:, 1024:1088, :], kv[j][:, 1024:1088, :])
    sess.close()


def test_greedy_pick_taken_from_the_lm_head_launch_keeps_the_first_maximum(bh, oracle):
    """Where lm_head runs on the one-row f32 kernel (runs of more than 16 tiles:
    the shipped shape and this one) its launch leaves the first maximum of every
    16 logits behind and the step's last kernel picks among those.  Every
    vocabulary column here is the same int8 vector, so that the logits are the
    scales times one number and their maxima are ties: the token must be the
    first of them, whatever the sign of that number."""
    shape = Shape(layers=1, hidden=1152, heads=9, kv_heads=3, head_dim=128, inter=256,
                  vocab=70000, max_len=64)
    from test_gemv_plan import F32, plan as gemv_plan
    cut = gemv_plan(bh, 1, shape.hidden, shape.vocab)
    assert cut.kernel == F32 and cut.tiles_per_wavefront > 16 and not cut.split
    sess, _ = synthetic.build_session(shape, context=0)
    g = sess._globals
    w = g["w_lm"]
    w[:] = w[:, :1]
    s = torch.ones(shape.vocab, device="cuda")
    s[[123, 40000, 50001, 69999]] = 2.0  # the maxima when the common product is positive
    s[[7, 60000]] = 0.5                  # ... and when it is negative
    sess.set_globals(g["embed"], g["inv_freq"], g["ln_f"], w, s)
    tok, seen = 11, set()
    for pos in range(12):
        nxt, logits = sess.decode(tok, pos)
        assert (logits == logits.max()).sum() >= 2
        assert nxt == oracle.argmax_first(logits) == int(np.argmax(logits))
        assert nxt in (7, 123)
        seen.add(nxt)
        tok = (tok * 7919 + 13) % shape.vocab  # other rows of the embedding
    sess.close()
    assert len(seen) >= 1
