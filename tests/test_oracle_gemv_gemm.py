"""Pins the oracle's decode GEMV kernels (a4, a5, a6) and BLIS GEMM (a7)."""
import numpy as np
import pytest


def test_dequant_gemv_reference_known_answer(oracle):
    # examples/BuddyMatmul/dequant-matmul-vectorization-decode.mlir:97-123
    A = np.ones(8, np.float32)
    W = np.zeros((8, 8), np.int8)
    W[:, :2] = 2
    y = oracle.dequant_gemv(A, W, np.full(8, 0.5, np.float32))
    assert y.tolist() == [8, 8, 0, 0, 0, 0, 0, 0]


@pytest.mark.parametrize("K,N", [(8, 8), (64, 32), (100, 70), (1536, 256)])
def test_dequant_gemv_closed_form(oracle, K, N):
    rng = np.random.default_rng(K + N)
    A = rng.normal(0, 1, K).astype(np.float32)
    W = rng.integers(-128, 128, (K, N)).astype(np.int8)
    s = rng.uniform(1e-4, 1e-3, N).astype(np.float32)
    C0 = rng.normal(0, 1, N).astype(np.float32)
    y = oracle.dequant_gemv(A, W, s, C0)
    ref = C0.astype(np.float64) + (A.astype(np.float64) @ W.astype(np.float64)) * s
    np.testing.assert_allclose(y, ref, rtol=2e-5, atol=2e-5)
    # transposed operand / dropped scale / missing C would each be far off
    assert not np.allclose(y, ref - C0, rtol=1e-3, atol=1e-3)


def test_dequant_gemv_sequential_fma_order_is_exact(oracle):
    # the loop is acc = fma(a, w, acc) in k order, then acc*scale, then C + ...
    rng = np.random.default_rng(7)
    K, N = 50, 5
    A = rng.normal(0, 1, K).astype(np.float32)
    W = rng.integers(-128, 128, (K, N)).astype(np.int8)
    s = rng.uniform(0.001, 0.01, N).astype(np.float32)
    C0 = rng.normal(0, 1, N).astype(np.float32)
    y = oracle.dequant_gemv(A, W, s, C0)
    for n in range(N):
        acc = np.float32(0)
        for k in range(K):
            # an fma of f32 operands = the f64 product-sum rounded once
            acc = np.float32(np.float64(A[k]) * np.float64(W[k, n]) + np.float64(acc))
        want = np.float32(C0[n] + np.float32(acc * s[n]))
        assert y[n] == want


def test_dequant_gemv_panels_equals_plain(oracle):
    rng = np.random.default_rng(9)
    K, N = 192, 128
    A = rng.normal(0, 1, K).astype(np.float32)
    W = rng.integers(-128, 128, (K, N)).astype(np.int8)
    s = rng.uniform(1e-4, 1e-3, N).astype(np.float32)
    y0 = oracle.dequant_gemv(A, W, s)
    y1 = oracle.dequant_gemv_panels(A, oracle.pack_panels(W, 32), s, K, N)
    np.testing.assert_array_equal(y0, y1)


@pytest.mark.parametrize("zero_init", [False, True])
def test_f32_gemv_plain_and_packed(oracle, zero_init):
    # tests/Conversion/matmul-vectorization-decode-zero-init.mlir:16-23:
    # a proven-zero C is not read; otherwise the accumulator starts at C
    rng = np.random.default_rng(11)
    K, N, V = 128, 64, 32
    A = rng.normal(0, 1, K).astype(np.float32)
    B = rng.normal(0, 1, (K, N)).astype(np.float32)
    C0 = rng.normal(0, 1, N).astype(np.float32)
    y_plain = oracle.gemv_f32(A, B, C0, V, zero_init)
    y_packed = oracle.gemv_packed_f32(A, oracle.pack_panels(B, V), C0, K, N, V, zero_init)
    np.testing.assert_array_equal(y_plain, y_packed)
    ref = A.astype(np.float64) @ B.astype(np.float64) + (0 if zero_init else C0)
    np.testing.assert_allclose(y_plain, ref, rtol=1e-5, atol=1e-5)


def test_blis_reference_known_answers(oracle):
    # tests/Conversion/matmul-blis-vectorization.mlir:23-57 (M=9,N=17,K=4)
    C = oracle.blis_gemm_f32(np.ones((9, 4), np.float32), np.ones((4, 17), np.float32),
                             np.full((9, 17), 10, np.float32))
    assert (C == 14).all()
    # examples/BuddyMatmul/dequant-matmul-vectorization-blis-prefill.mlir:90-115
    C = oracle.blis_gemm_w8a32(np.ones((4, 4), np.float32), np.full((4, 4), 2, np.int8),
                               np.ones(4, np.float32))
    assert (C == 8).all()


@pytest.mark.parametrize("M", [7, 8, 9, 64, 65])
@pytest.mark.parametrize("N", [31, 32, 33, 256, 257])
@pytest.mark.parametrize("K", [127, 128, 129])
def test_blis_tails_vs_float64(oracle, M, N, K):
    rng = np.random.default_rng(M * 1000 + N * 10 + K)
    A = rng.normal(0, 1, (M, K)).astype(np.float32)
    W = rng.integers(-128, 128, (K, N)).astype(np.int8)
    s = rng.uniform(1e-4, 1e-3, N).astype(np.float32)
    C0 = rng.normal(0, 1, (M, N)).astype(np.float32)
    C = oracle.blis_gemm_w8a32(A, W, s, C0)
    ref = C0 + A.astype(np.float64) @ (W.astype(np.float64) * s[None, :])
    np.testing.assert_allclose(C, ref, rtol=3e-5, atol=3e-5)


def test_blis_scale_before_sum_and_kc_rounding(oracle):
    # full 8x32 tile, K = 256 = two kc blocks: B is dequantised (rounded f32)
    # before the fma chain and C is rounded once per kc block
    rng = np.random.default_rng(21)
    M, N, K = 8, 32, 256
    A = rng.normal(0, 1, (M, K)).astype(np.float32)
    W = rng.integers(-128, 128, (K, N)).astype(np.int8)
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    C = oracle.blis_gemm_w8a32(A, W, s)
    Bp = (W.astype(np.float32) * s[None, :]).astype(np.float32)
    for (i, j) in [(0, 0), (3, 17), (7, 31)]:
        c = np.float32(0)
        for pc in (0, 128):
            acc = np.float32(0)
            for k in range(pc, pc + 128):
                acc = np.float32(np.float64(A[i, k]) * np.float64(Bp[k, j]) + np.float64(acc))
            c = np.float32(c + acc)
        assert C[i, j] == c


def test_w8a8_int32_exact(oracle):
    rng = np.random.default_rng(31)
    M, K, N = 3, 200, 40
    A = rng.normal(0, 1, (M, K)).astype(np.float32)
    W = rng.integers(-128, 128, (K, N)).astype(np.int8)
    ws = rng.uniform(1e-4, 1e-3, N).astype(np.float32)
    C, acc = oracle.w8a8_matmul(A, W, ws)
    xq, sa = oracle.w8a8_quantize_activation(A)
    assert np.abs(xq).max() == 127  # the largest |x| maps to +-127
    ref_acc = xq.astype(np.int64) @ W.astype(np.int64)
    np.testing.assert_array_equal(acc.astype(np.int64), ref_acc)
    np.testing.assert_array_equal(C, acc.astype(np.float32) * (sa * ws)[None, :])
    z, sz = oracle.w8a8_quantize_activation(np.zeros((2, 4), np.float32))
    assert sz == np.float32(1e-10) and (z == 0).all()
