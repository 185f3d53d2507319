"""GPU parity of the prefill path: the MFMA int8 dequant matmul against the
oracle's BLIS restatement, the causal GQA attention against the oracle's
flash-attention restatement, and block prefill of the resident session against
token-by-token decode steps of the oracle."""
import numpy as np
import pytest
import torch

import buddy_mlir_amd as bma
from buddy_mlir_amd import ops, synthetic
from buddy_mlir_amd.session import Shape
from parity import check_close
from test_gpu_decode import SMALL, oracle_model

pytestmark = pytest.mark.gpu

SCALE = np.float32(0.0883883461)


def bf16_round(a: np.ndarray) -> np.ndarray:
    return torch.from_numpy(a).to(torch.bfloat16).to(torch.float32).numpy()


GEMM_SHAPES = [(512, 1536, 1536), (512, 1536, 256), (512, 1536, 8960), (512, 8960, 1536),
               (9, 4, 17), (65, 129, 257), (1, 64, 16), (130, 200, 130),
               # ragged in every dimension and wide enough for the kernel that does
               # not split K (64 x 256 workgroup tiles)
               (500, 200, 6500), (1000, 72, 3300)]


def fixed_point_round(a: np.ndarray, digits: int = 3):
    """What the int8 matmul multiplies: per row the smallest power-of-two step s
    with max|a| / s < 2^(8 digits - 2), and rint(a / s) * s."""
    mx = np.abs(a).max(axis=1, keepdims=True).astype(np.float64)
    e = np.floor(np.log2(np.where(mx > 0, mx, 1.0))) + 1 - (8 * digits - 2)
    step = np.exp2(np.maximum(e, -126))
    return (np.rint(a.astype(np.float64) / step) * step).astype(np.float32), step


@pytest.mark.parametrize("M,K,N", GEMM_SHAPES)
@pytest.mark.parametrize("mode", ["bf16", "exact", "digits", "digits2"])
def test_prefill_gemm_matches_blis_oracle(oracle, M, K, N, mode):
    q, s = synthetic.quantized_linear(K, N, M + K + N)
    packed = ops.pack_w8(q)
    g = torch.Generator(device="cuda").manual_seed(M)
    x = torch.randn((M, K), generator=g, device="cuda")
    if mode.startswith("digits") and M > 2:
        x[1] *= 1e-30   # rows of very different magnitude: the step is per row
        x[2, 0] = 300.0  # one large element in a row of small ones
    y = ops.gemm_w8a32(x, packed, s, K, N, exact=mode == "exact",
                       digits={"digits": 3, "digits2": 2}.get(mode, False))
    torch.cuda.synchronize()
    xh = x.cpu().numpy()
    if mode == "digits2":
        # two digit planes: 15 bits below each row's maximum, the fixed-point
        # counterpart of the bf16 cast.  Like that mode it is held to the oracle
        # fed the same rounded activations (only summation order is left) ...
        got = y.cpu().numpy()
        a_in, _ = fixed_point_round(xh, digits=2)
        want = oracle.blis_gemm_w8a32(a_in, q.cpu().numpy(), s.cpu().numpy())
        for m in range(M):
            check_close(got[m], want[m], normwise=4e-6)
        # ... and stays within the rounding it states of the plain f32 input:
        # norm-wise 2^-15 max|row| sqrt(K) / |row| at most, far inside the bf16
        # cast's 2^-9
        want = oracle.blis_gemm_w8a32(xh, q.cpu().numpy(), s.cpu().numpy())
        for m in range(M):
            if m != 2 or M <= 2:  # (the row with the 300 sigma outlier: its step is 2^-6)
                assert np.linalg.norm(got[m] - want[m]) <= 2e-4 * np.linalg.norm(want[m]) + 1e-30
        return
    if mode == "digits":
        # against the plain f32 input at the stated bar, per row (rows differ by
        # 30 orders of magnitude) ...
        want = oracle.blis_gemm_w8a32(xh, q.cpu().numpy(), s.cpu().numpy())
        got = y.cpu().numpy()
        for m in range(M):
            check_close(got[m], want[m])
        # ... and against the oracle fed the same fixed-point activations, where
        # what is left is summation order only
        a_in, _ = fixed_point_round(xh)
        want = oracle.blis_gemm_w8a32(a_in, q.cpu().numpy(), s.cpu().numpy())
        for m in range(M):
            check_close(got[m], want[m], normwise=4e-6)
        return
    # "activations cast to bf16": the oracle gets the same rounded activations
    a_in = xh if mode == "exact" else bf16_round(xh)
    want = oracle.blis_gemm_w8a32(a_in, q.cpu().numpy(), s.cpu().numpy())
    check_close(y.cpu().numpy(), want)


@pytest.mark.parametrize("M,K,N", [(512, 1536, 8960), (512, 8960, 1536), (70, 200, 48)])
def test_non_finite_activation_rows_come_out_nan_in_the_digit_mode(M, K, N):
    """The reference's prefill kernel is an f32 multiply-add chain
    (MatMulBlisVectorization.cpp:644-740): a NaN in a row of A makes that row of
    C NaN, an infinity makes it +-inf or NaN.  The digit-plane matmul gives such a
    row a NaN step: every element of the row is NaN, every other row is what it
    is without the poison, bit for bit."""
    q, s = synthetic.quantized_linear(K, N, 5)
    packed = ops.pack_w8(q)
    g = torch.Generator(device="cuda").manual_seed(M + K)
    x = torch.randn((M, K), generator=g, device="cuda")
    clean = ops.gemm_w8a32(x, packed, s, K, N, digits=True).cpu().numpy()
    x[3, K // 2] = float("nan")
    x[M - 2, 0] = float("-inf")
    x[5, K - 1] = float("inf")
    got = ops.gemm_w8a32(x, packed, s, K, N, digits=True).cpu().numpy()
    bad = [3, 5, M - 2]
    assert np.isnan(got[bad]).all()
    rest = np.delete(np.arange(M), bad)
    assert np.isfinite(got[rest]).all()
    np.testing.assert_array_equal(got[rest], clean[rest])
    # the paired gate|up form with SiLU*mul in its epilogue
    if N % 64 == 0:
        both = torch.cat([packed, packed])
        got = ops.gemm_w8a32(x, both, torch.cat([s, s]), K, N, digits=True,
                             silu_pair=True).cpu().numpy()
        assert np.isnan(got[bad]).all() and np.isfinite(got[rest]).all()


def test_non_finite_token_through_session_prefill():
    """A prompt whose last token's embedding row holds a NaN (then an infinity):
    that row's logits are NaN; the logits of every earlier row are those of the
    clean prompt bit for bit (causality), through every digit-plane producer of
    the block (RMSNorm rows, SiLU*mul rows, the slice-adding kernel that writes
    the next layer's rows).  The poisoned token is the first of a 16-row block of
    the attention kernel: a masked key still meets the queries of its own block
    in the P.V matrix product as 0 x NaN (in the reference the additive -inf
    mask lets a NaN key reach every query of the prompt)."""
    sess, _ = synthetic.build_session(SMALL, context=0, ln_jitter=0.1)
    lib = bma.lib()
    V = SMALL.vocab
    toks = synthetic.first_tokens(SMALL, 33, seed=5).astype(np.int32)
    poisoned = int(toks[-1])
    toks[:-1][toks[:-1] == poisoned] = (poisoned + 1) % V

    def all_logits():
        out = np.empty((toks.size, V), np.float32)
        bma.check(lib.buddy_hip_session_prefill_all_logits(
            sess._h, toks.ctypes.data, toks.size, 0, out.ctypes.data), "prefill_all_logits")
        return out

    clean = all_logits()
    assert np.isfinite(clean).all()
    embed = sess._globals["embed"]
    for poison in (float("nan"), float("-inf")):
        keep = embed[poisoned].clone()
        embed[poisoned, 7] = poison
        torch.cuda.synchronize()
        got = all_logits()
        embed[poisoned] = keep
        torch.cuda.synchronize()
        assert np.isnan(got[-1]).all()
        np.testing.assert_array_equal(got[:-1], clean[:-1])
    np.testing.assert_array_equal(all_logits(), clean)
    sess.close()


@pytest.mark.parametrize("M,K", [(1, 64), (5, 100), (70, 1536), (48, 8960)])
def test_digit_planes_are_the_rounded_fixed_point(M, K):
    """W = 127 I with scale 1/127 copies the activations: what comes out is
    rint(a / s) * s exactly, row by row."""
    g = torch.Generator(device="cuda").manual_seed(K)
    x = torch.randn((M, K), generator=g, device="cuda") * 3.0
    x[0, 0] = 0.0
    if M > 1:
        x[1] = 0.0  # an all-zero row
        x[M - 1] *= 2.0 ** -100
    q = (torch.eye(K, device="cuda") * 127).to(torch.int8)
    s = torch.full((K,), 1.0 / 127.0, device="cuda")
    y = ops.gemm_w8a32(x, ops.pack_w8(q), s, K, K, digits=True)
    torch.cuda.synchronize()
    want, step = fixed_point_round(x.cpu().numpy())
    got = y.cpu().numpy().astype(np.float64)
    # 127 * (1/127 rounded to f32) is 1 to within 1 ulp of f32
    np.testing.assert_allclose(got, want, rtol=2e-7, atol=0)
    xh = x.cpu().numpy().astype(np.float64)
    assert (np.abs(got - xh) <= 0.5 * step + 2e-7 * np.abs(xh)).all()


# gate and up in one launch with SiLU(gate) * up in its epilogue: the model's
# shape, one shape for each of the four workgroup tiles, single-tile and ragged rows
SILU_PAIR_SHAPES = [(512, 1536, 8960), (144, 256, 8192), (300, 256, 5120), (200, 192, 8192),
                    (512, 192, 4480), (17, 64, 16), (100, 100, 160)]


def silu_pair_case(oracle, M, K, N, digits=3):
    q0, s0 = synthetic.quantized_linear(K, N, M + K + N)
    q1, s1 = synthetic.quantized_linear(K, N, M + K + N + 1)
    packed = torch.cat([ops.pack_w8(q0), ops.pack_w8(q1)])
    scale = torch.cat([s0, s1])
    g = torch.Generator(device="cuda").manual_seed(M)
    x = torch.randn((M, K), generator=g, device="cuda")
    y = ops.gemm_w8a32(x, packed, scale, K, N, digits=digits, silu_pair=True)
    torch.cuda.synchronize()
    xh = x.cpu().numpy()
    if digits == 2:  # the oracle gets the same 15-bit fixed-point activations
        xh, _ = fixed_point_round(xh, digits=2)
    gate = oracle.blis_gemm_w8a32(xh, q0.cpu().numpy(), s0.cpu().numpy())
    up = oracle.blis_gemm_w8a32(xh, q1.cpu().numpy(), s1.cpu().numpy())
    got = y.cpu().numpy()
    assert got.shape == (M, N)
    for m in range(M):
        check_close(got[m], oracle.silu_mul(gate[m], up[m]))


@pytest.mark.parametrize("M,K,N", SILU_PAIR_SHAPES)
def test_prefill_gemm_silu_pair(oracle, M, K, N):
    silu_pair_case(oracle, M, K, N)


def test_prefill_gemm_silu_pair_refusals(bh):
    x = torch.zeros((32, 64), device="cuda")
    w = torch.zeros((2 * 64 * 64,), dtype=torch.int8, device="cuda")
    s = torch.ones((128,), device="cuda")
    c = torch.zeros((32, 64), device="cuda")
    # not without the digit planes, not with accumulation, not with a ragged N
    assert bh.buddy_hip_gemm_w8a32(x.data_ptr(), w.data_ptr(), s.data_ptr(), c.data_ptr(),
                                   32, 64, 64, ops.GEMM_SILU_PAIR, None) != 0
    assert bh.buddy_hip_gemm_w8a32(x.data_ptr(), w.data_ptr(), s.data_ptr(), c.data_ptr(),
                                   32, 64, 64, ops.GEMM_SILU_PAIR | ops.GEMM_A_I8_DIGITS |
                                   ops.GEMV_ACCUMULATE, None) != 0
    assert bh.buddy_hip_gemm_w8a32(x.data_ptr(), w.data_ptr(), s.data_ptr(), c.data_ptr(),
                                   32, 64, 40, ops.GEMM_SILU_PAIR | ops.GEMM_A_I8_DIGITS,
                                   None) != 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("exact", [True, False])
@pytest.mark.parametrize("M,K,N", [(100, 256, 96), (490, 136, 6600)])
def test_prefill_gemm_accumulates(oracle, M, K, N, exact):
    q, s = synthetic.quantized_linear(K, N, 77)
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn((M, K), generator=g, device="cuda")
    c0 = torch.randn((M, N), generator=g, device="cuda")
    c = c0.clone()
    ops.gemm_w8a32(x, ops.pack_w8(q), s, K, N, out=c, accumulate=True, exact=exact,
                   digits=not exact)
    torch.cuda.synchronize()
    want = oracle.blis_gemm_w8a32(x.cpu().numpy(), q.cpu().numpy(), s.cpu().numpy(),
                                  c0.cpu().numpy())
    check_close(c.cpu().numpy(), want)


def run_attn(bh, q, k, v, mask, heads, kv_heads, Lq, Lk):
    out = torch.empty_like(q)
    torch.cuda.synchronize()
    bma.check(bh.buddy_hip_prefill_attention(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), None if mask is None else mask.data_ptr(),
        out.data_ptr(), heads, kv_heads, 128, Lq, Lk, float(SCALE), None))
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("L", [16, 40, 512])
def test_prefill_attention_reference_shape(bh, oracle, L):
    """q, k, v all [12, L, 128] with an additive causal mask, the call shape of
    flash_attention_for_cpu_prefill_op; also the implicit causal mask."""
    H = 12
    g = torch.Generator(device="cuda").manual_seed(L)
    q, k, v = (torch.randn((H, L, 128), generator=g, device="cuda") for _ in range(3))
    mh = np.where(np.tril(np.ones((L, L), bool)), 0.0, -np.inf).astype(np.float32)
    want = oracle.prefill_flash_attention(q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy(),
                                          mh, SCALE)
    got_mask = run_attn(bh, q, k, v, torch.from_numpy(mh).cuda(), H, H, L, L)
    got_causal = run_attn(bh, q, k, v, None, H, H, L, L)
    check_close(got_mask, want)
    check_close(got_causal, want)


def test_prefill_attention_gqa_and_longer_keys(bh, oracle):
    """2 KV heads read in place = 12 repeated heads; 37 queries over 100 keys
    (a prompt continuing after 63 cached positions)."""
    H, HKV, Lq, Lk = 12, 2, 37, 100
    g = torch.Generator(device="cuda").manual_seed(5)
    q = torch.randn((H, Lq, 128), generator=g, device="cuda")
    k = torch.randn((HKV, Lk, 128), generator=g, device="cuda")
    v = torch.randn((HKV, Lk, 128), generator=g, device="cuda")
    kk = k.repeat_interleave(H // HKV, dim=0).cpu().numpy()
    vv = v.repeat_interleave(H // HKV, dim=0).cpu().numpy()
    qi = np.arange(Lq)[:, None] + (Lk - Lq)
    mh = np.where(np.arange(Lk)[None, :] <= qi, 0.0, -np.inf).astype(np.float32)
    want = oracle.prefill_flash_attention(q.cpu().numpy(), kk, vv, mh, SCALE)
    check_close(run_attn(bh, q, k, v, None, H, HKV, Lq, Lk), want)


@pytest.mark.parametrize("Lq,Lk", [(1, 1), (5, 5), (17, 17), (33, 33), (95, 95), (129, 129),
                                   (1, 300), (16, 130), (50, 51), (200, 333)])
def test_prefill_attention_ragged_lengths(bh, oracle, Lq, Lk):
    """A workgroup takes a query block and its mirror image, and its wavefronts
    split the key blocks of the two: one query block alone, an odd number of
    them (the middle one on its own), a last block of 1 row, fewer key blocks than
    wavefronts, and prompts that continue behind cached positions -- with the
    implicit causal mask and with the same mask passed as a tensor."""
    H, HKV = 4, 2
    g = torch.Generator(device="cuda").manual_seed(1000 * Lq + Lk)
    q = torch.randn((H, Lq, 128), generator=g, device="cuda")
    k = torch.randn((HKV, Lk, 128), generator=g, device="cuda")
    v = torch.randn((HKV, Lk, 128), generator=g, device="cuda")
    kk = k.repeat_interleave(H // HKV, dim=0).cpu().numpy()
    vv = v.repeat_interleave(H // HKV, dim=0).cpu().numpy()
    qi = np.arange(Lq)[:, None] + (Lk - Lq)
    mh = np.where(np.arange(Lk)[None, :] <= qi, 0.0, -np.inf).astype(np.float32)
    want = oracle.prefill_flash_attention(q.cpu().numpy(), kk, vv, mh, SCALE)
    check_close(run_attn(bh, q, k, v, None, H, HKV, Lq, Lk), want)
    check_close(run_attn(bh, q, k, v, torch.from_numpy(mh).cuda(), H, HKV, Lq, Lk), want)


@pytest.mark.parametrize("H,HKV,Lq,Lk", [(32, 8, 272, 272), (12, 2, 600, 700)])
def test_prefill_attention_launches_of_several_rounds(bh, oracle, H, HKV, Lq, Lk):
    """More workgroups than compute units: the launch takes the form with four
    wavefronts per workgroup (two workgroups per compute unit)."""
    g = torch.Generator(device="cuda").manual_seed(H + Lq)
    q = torch.randn((H, Lq, 128), generator=g, device="cuda")
    k = torch.randn((HKV, Lk, 128), generator=g, device="cuda")
    v = torch.randn((HKV, Lk, 128), generator=g, device="cuda")
    kk = k.repeat_interleave(H // HKV, dim=0).cpu().numpy()
    vv = v.repeat_interleave(H // HKV, dim=0).cpu().numpy()
    qi = np.arange(Lq)[:, None] + (Lk - Lq)
    mh = np.where(np.arange(Lk)[None, :] <= qi, 0.0, -np.inf).astype(np.float32)
    want = oracle.prefill_flash_attention(q.cpu().numpy(), kk, vv, mh, SCALE)
    check_close(run_attn(bh, q, k, v, None, H, HKV, Lq, Lk), want)
    check_close(run_attn(bh, q, k, v, torch.from_numpy(mh).cuda(), H, HKV, Lq, Lk), want)


def test_prefill_attention_refuses_unaligned_operands(bh):
    t = torch.zeros(4 * 16 * 128 + 4, device="cuda")
    p = t.data_ptr()
    rc = bh.buddy_hip_prefill_attention(p + 4, p, p, None, p, 4, 4, 128, 16, 16, float(SCALE), None)
    assert rc == 1 and b"16-byte aligned" in bh.buddy_hip_last_error()


@pytest.mark.parametrize("precision", ["digits", "exact", "bf16", "digits2"])
def test_small_model_block_prefill_equals_token_by_token(oracle, precision):
    """Prefill of 40 prompt tokens as one block against 40 oracle decode steps:
    last-token logits, greedy token and every cache row written; then decode
    continues from the prefilled cache."""
    sess, host = synthetic.build_session(SMALL, context=0, keep_host=True, ln_jitter=0.1)
    om = oracle_model(oracle, SMALL, host)
    kv = [a.copy() for a in host["kv"]]
    toks = synthetic.first_tokens(SMALL, 40, seed=3).tolist()
    for pos, t in enumerate(toks):
        otok, ologits = om.decode_step(t, pos, kv)
    nxt, logits = sess.prefill(toks, 0, precision=precision)
    if precision not in ("bf16", "digits2"):
        check_close(logits, ologits)
        assert nxt == otok
        for j in range(2 * SMALL.layers):
            check_close(sess.get_kv(j)[:, :40, :], kv[j][:, :40, :])
        # decoding on from the prefilled cache
        tok = otok
        for step in range(6):
            n2, lg = sess.decode(tok, 40 + step)
            tok, olg = om.decode_step(tok, 40 + step, kv)
            check_close(lg, olg)
            assert n2 == tok
    elif precision == "digits2":
        # activations rounded to 2^-15 of their row's maximum in every matmul
        check_close(logits, ologits, rtol=5e-3, atol_frac=1e-3, normwise=1e-3)
        assert nxt == otok
    else:
        # activations cast to bf16 in every matmul of every layer: compared at
        # the looser bound that rounding allows
        check_close(logits, ologits, rtol=5e-2, atol_frac=2e-2, normwise=2e-2)
    sess.close()


def test_prefill_in_two_blocks_and_after_decode_steps(oracle):
    """A prompt fed as two blocks (the second starts at position 24 and attends
    to the cache rows of the first), then decode steps, then a third block: the
    same logits and cache rows as 53 oracle decode steps."""
    sess, host = synthetic.build_session(SMALL, context=0, keep_host=True, ln_jitter=0.1)
    om = oracle_model(oracle, SMALL, host)
    kv = [a.copy() for a in host["kv"]]
    toks = synthetic.first_tokens(SMALL, 53, seed=11).tolist()
    want = []
    for pos, t in enumerate(toks):
        otok, ologits = om.decode_step(t, pos, kv)
        want.append((otok, ologits))
    nxt, logits = sess.prefill(toks[:24], 0)
    check_close(logits, want[23][1])
    assert nxt == want[23][0]
    nxt, logits = sess.prefill(toks[24:40], 24)
    check_close(logits, want[39][1])
    assert nxt == want[39][0]
    for pos in range(40, 43):  # three tokens one by one
        n2, lg = sess.decode(toks[pos], pos)
        check_close(lg, want[pos][1])
        assert n2 == want[pos][0]
    nxt, logits = sess.prefill(toks[43:53], 43)  # a ragged block of 10
    check_close(logits, want[52][1])
    assert nxt == want[52][0]
    for j in range(2 * SMALL.layers):
        check_close(sess.get_kv(j)[:, :53, :], kv[j][:, :53, :])
    sess.close()


def test_wide_hidden_size_through_the_slice_adding_norm_kernel(oracle):
    """hidden = 9216: the kernel that adds the K slices of o_proj / down and
    writes the next RMSNorm's digit planes keeps two copies of a row in LDS,
    72 KiB here -- more than the 64 KiB a kernel gets without asking.  A
    prompt of 64 tokens (one row tile: the matmuls then split K over
    workgroups) against 64 oracle decode steps."""
    shape = Shape(layers=2, hidden=9216, heads=8, kv_heads=2, head_dim=128, inter=2048,
                  vocab=512, max_len=128, rms_eps=1e-6)
    sess, host = synthetic.build_session(shape, context=0, keep_host=True, ln_jitter=0.1)
    om = oracle_model(oracle, shape, host)
    kv = [a.copy() for a in host["kv"]]
    toks = synthetic.first_tokens(shape, 64, seed=23).tolist()
    for pos, t in enumerate(toks):
        otok, ologits = om.decode_step(t, pos, kv)
    nxt, logits = sess.prefill(toks, 0)
    check_close(logits, ologits)
    assert nxt == otok
    for j in range(2 * shape.layers):
        check_close(sess.get_kv(j)[:, :64, :], kv[j][:, :64, :])
    sess.close()


@pytest.mark.timeout(900)
def test_qwen2_1p5b_shape_512_token_prefill(oracle):
    """The full 28-layer shape, a prompt of 512 tokens as one block (digit-plane
    matmuls, the default) against 512 oracle decode steps: last-row logits, the
    greedy token, and the cache rows of the first and the last layer; then the
    last-row logits of the three other activation modes."""
    shape = Shape()
    sess, host = synthetic.build_session(shape, context=0, keep_host=True)
    om = oracle_model(oracle, shape, host)
    kv = host["kv"]
    toks = synthetic.first_tokens(shape, 512, seed=21).tolist()
    for pos, t in enumerate(toks):
        otok, ologits = om.decode_step(t, pos, kv)
    nxt, logits = sess.prefill(toks, 0)
    check_close(logits, ologits)
    top2 = np.partition(ologits, -2)[-2:]
    assert nxt == otok, f"top-2 logit margin {float(top2[1] - top2[0]):.3e}"
    for j in (0, 1, 2 * shape.layers - 2, 2 * shape.layers - 1):
        check_close(sess.get_kv(j)[:, :512, :], kv[j][:, :512, :])
    # one decode step on from the prefilled cache
    n2, lg = sess.decode(otok, 512)
    t2, olg = om.decode_step(otok, 512, kv)
    check_close(lg, olg)
    assert n2 == t2
    # the same prompt in the other activation modes, at the bound each one's
    # rounding allows over 28 layers: every f32 bit (three bf16 terms) at the f32
    # bar, two digit planes (2^-15 of a row's maximum per matmul), activations cast
    # to bf16 (2^-9 per element: the precision BASELINE's prefill case names)
    _, exact = sess.prefill(toks, 0, precision="exact")
    check_close(exact, ologits)
    _, two = sess.prefill(toks, 0, precision="digits2")
    nw2 = check_close(two, ologits, rtol=2e-2, atol_frac=3e-3, normwise=3e-3)
    _, cast = sess.prefill(toks, 0, precision="bf16")
    nwc = check_close(cast, ologits, rtol=5e-2, atol_frac=2e-2, normwise=2e-2)
    print(f"norm-wise error of the last-row logits: two planes {nw2:.2e}, bf16 cast {nwc:.2e}")
    assert nw2 < nwc
    for lg_mode in (exact, two, cast):
        assert int(np.argmax(lg_mode)) == otok or float(top2[1] - top2[0]) < 0.05 * float(
            np.abs(ologits).max())
    sess.close()


def test_session_prefill_refuses_overflow(bh):
    sess, _ = synthetic.build_session(SMALL, context=0)
    with pytest.raises(bma.BuddyHipError):
        sess.prefill(list(range(10)), SMALL.max_len - 5)
    sess.close()
