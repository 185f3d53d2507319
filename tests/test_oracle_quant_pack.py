"""Pins the oracle's quantizer (a1) and reference panel packing (a3).

Quantizer recipe: tools/buddy-codegen/import_model.py:837-848,874-880.
Panel layout: frontend/Python/graph/transform/pack_decode_weights.py:102-108,
address arithmetic pinned by tests/Conversion/matmul-vectorization-decode-packed
.mlir:19-25 (K=128, N=64, V=32: flat size 8192, panel base n*128, k offset k*32).
"""
import numpy as np
import pytest
import torch


def test_quant_zero_channel_clamps_scale(oracle):
    W = np.zeros((16, 4), np.float32)
    W[:, 1] = np.linspace(-1, 1, 16)
    q, s = oracle.quantize_w8(W)
    assert s[0] == np.float32(1e-10) and s[2] == np.float32(1e-10)
    assert (q[:, 0] == 0).all() and (q[:, 2] == 0).all() and (q[:, 3] == 0).all()


def test_quant_extremes_hit_127_never_minus_128(oracle):
    rng = np.random.default_rng(1)
    W = rng.normal(0, 0.02, (256, 64)).astype(np.float32)
    q, s = oracle.quantize_w8(W)
    amax_idx = np.abs(W).argmax(axis=0)
    for n in range(64):
        v = W[amax_idx[n], n]
        assert q[amax_idx[n], n] == (127 if v > 0 else -127)
    assert q.min() >= -127  # a symmetric range never produces -128
    np.testing.assert_array_equal(s, (np.abs(W).max(axis=0) / np.float32(127.0)))


def test_quant_round_half_to_even(oracle):
    # amax = 127 -> scale exactly 1.0, so W/scale are the halves themselves
    col = np.array([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5], np.float32)
    q, s = oracle.quantize_w8(col[:, None])
    assert s[0] == 1.0
    assert q[:, 0].tolist() == [127, 0, 2, 2, 0, -2, -2, 4]


def test_quant_idempotent_on_dequantized(oracle):
    rng = np.random.default_rng(2)
    W = rng.normal(0, 0.02, (128, 48)).astype(np.float32)
    q, s = oracle.quantize_w8(W)
    deq = q.astype(np.float32) * s[None, :]
    q2, s2 = oracle.quantize_w8(deq)
    np.testing.assert_array_equal(q, q2)


@pytest.mark.parametrize("shape", [(64, 32), (1536, 96), (33, 7)])
def test_quant_matches_torch_library_ops(oracle, shape):
    # the reference's recipe written with the library routines it calls
    # (torch abs/amax/div/clamp/round on CPU f32), executed here on our inputs
    g = torch.Generator().manual_seed(shape[0] * 131 + shape[1])
    W = torch.randn(shape, generator=g) * 0.02
    W[3, 1] = 0.0
    amax = W.abs().amax(dim=[0], keepdim=True)
    scale = (amax / 127.0).clamp(min=1e-10)
    ref_q = torch.clamp(torch.round(W / scale), -128, 127).to(torch.int8).numpy()
    q, s = oracle.quantize_w8(W.numpy())
    np.testing.assert_array_equal(q, ref_q)
    np.testing.assert_array_equal(s, scale.numpy().reshape(-1))


def test_quant_w4_range(oracle):
    rng = np.random.default_rng(5)
    W = rng.normal(0, 1, (64, 8)).astype(np.float32)
    q, s = oracle.quantize_w4(W)
    assert q.min() >= -7 and q.max() <= 7
    np.testing.assert_array_equal(s, np.abs(W).max(axis=0) / np.float32(7.0))


def test_pack_reference_lit_vector(oracle):
    # matmul-vectorization-decode-packed.mlir: K=128, N=64, V=32
    K, N, V = 128, 64, 32
    B = np.arange(K * N, dtype=np.float32).reshape(K, N)
    flat = oracle.pack_panels(B, V).reshape(-1)
    assert flat.size == 8192
    for n0 in (0, 32):
        for k in (0, 1, 77, 127):
            lin = n0 * K + k * V  # muli %n,%c128 ; muli %k,%c32 ; addi
            np.testing.assert_array_equal(flat[lin:lin + V], B[k, n0:n0 + V])


@pytest.mark.parametrize("K,N,V,dt", [(4, 8, 4, np.float32), (3, 64, 32, np.int8),
                                      (128, 128, 128, np.float32), (5, 6, 2, np.int8)])
def test_pack_closed_form_and_roundtrip(oracle, K, N, V, dt):
    rng = np.random.default_rng(K * N)
    B = rng.integers(-100, 100, (K, N)).astype(dt)
    P = oracle.pack_panels(B, V)
    assert P.shape == B.shape and P.dtype == B.dtype
    flat = P.reshape(-1)
    for nt in range(N // V):
        for k in range(K):
            for v in range(V):
                assert flat[nt * K * V + k * V + v] == B[k, nt * V + v]
    # same bytes, permuted; equals torch's reshape/permute recipe
    np.testing.assert_array_equal(np.sort(flat), np.sort(B.reshape(-1)))
    ref = torch.from_numpy(B).reshape(K, N // V, V).permute(1, 0, 2).contiguous().reshape(K, N)
    np.testing.assert_array_equal(P, ref.numpy())
    np.testing.assert_array_equal(oracle.unpack_panels(P, V), B)


def test_pack_refuses_ragged_n(oracle):
    with pytest.raises(ValueError):
        oracle.pack_panels(np.zeros((4, 33), np.float32), 32)
