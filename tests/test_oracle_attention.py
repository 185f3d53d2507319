"""Pins the oracle's attention kernels (a8, a9) against the textbook two-pass
softmax in float64 and the cases the reference states for its own kernel
(frontend/Python/ops/tosa.py:14075-14080: valid_len 9/37/613/1024, splits
1/2/4/8, true -inf mask, max err ~1e-7, no NaN)."""
import numpy as np
import pytest
import torch

H, HKV, D = 12, 2, 128
SCALE = np.float32(0.0883883461)  # subgraph0_decode_simplify.mlir:17


def ref_decode(q, kc, vc, mask):
    g = H // HKV
    out = np.empty((H, D))
    lse = np.empty(H)
    for h in range(H):
        s = (kc[h // g].astype(np.float64) @ q[h].astype(np.float64)) * np.float64(SCALE)
        s = s + mask.astype(np.float64)
        m = s.max()
        p = np.exp(s - m)
        out[h] = (p[:, None] * vc[h // g].astype(np.float64)).sum(0) / p.sum()
        lse[h] = m + np.log(p.sum())
    return out, lse


@pytest.mark.parametrize("valid", [9, 37, 613, 1024])
@pytest.mark.parametrize("splits", [1, 2, 4, 8])
def test_decode_attention_reference_cases(oracle, valid, splits):
    L = 1024
    rng = np.random.default_rng(valid * 10 + splits)
    q = rng.normal(0, 1, (H, D)).astype(np.float32)
    kc = rng.normal(0, 1, (HKV, L, D)).astype(np.float32)
    vc = rng.normal(0, 1, (HKV, L, D)).astype(np.float32)
    mask = np.where(np.arange(L) < valid, 0.0, -np.inf).astype(np.float32)
    out, lse = oracle.gqa_decode_attention(q, kc, vc, mask, SCALE, splits)
    assert np.isfinite(out).all() and np.isfinite(lse).all()
    ro, rl = ref_decode(q, kc, vc, mask)
    assert np.abs(out - ro).max() < 2e-6
    assert np.abs(lse - rl).max() < 2e-5


def test_decode_attention_split_independent_and_masked_split_is_zero(oracle):
    L = 256
    rng = np.random.default_rng(3)
    q = rng.normal(0, 1, (H, D)).astype(np.float32)
    kc = rng.normal(0, 1, (HKV, L, D)).astype(np.float32)
    vc = rng.normal(0, 1, (HKV, L, D)).astype(np.float32)
    mask = np.where(np.arange(L) < 40, 0.0, -np.inf).astype(np.float32)
    o1, _ = oracle.gqa_decode_attention(q, kc, vc, mask, SCALE, 1)
    o4, _ = oracle.gqa_decode_attention(q, kc, vc, mask, SCALE, 4)
    assert np.abs(o1 - o4).max() < 1e-6
    # poison the masked tail: fully masked splits must contribute exactly 0
    vc2 = vc.copy()
    vc2[:, 64:, :] = 1e30
    o4b, _ = oracle.gqa_decode_attention(q, kc, vc2, mask, SCALE, 4)
    np.testing.assert_array_equal(o4, o4b)


def test_decode_attention_gqa_head_mapping(oracle):
    # heads 0..5 read KV head 0, heads 6..11 read KV head 1 (h / group)
    L = 64
    rng = np.random.default_rng(4)
    q = np.tile(rng.normal(0, 1, (1, D)).astype(np.float32), (H, 1))
    kc = rng.normal(0, 1, (HKV, L, D)).astype(np.float32)
    vc = rng.normal(0, 1, (HKV, L, D)).astype(np.float32)
    out, _ = oracle.gqa_decode_attention(q, kc, vc, np.zeros(L, np.float32), SCALE, 4)
    for h in range(1, 6):
        np.testing.assert_array_equal(out[h], out[0])
    for h in range(7, 12):
        np.testing.assert_array_equal(out[h], out[6])
    assert not np.allclose(out[0], out[6])


@pytest.mark.parametrize("Lq", [16, 40, 128])
def test_prefill_attention_vs_float64_and_sdpa(oracle, Lq):
    rng = np.random.default_rng(Lq)
    q = rng.normal(0, 1, (H, Lq, D)).astype(np.float32)
    k = rng.normal(0, 1, (H, Lq, D)).astype(np.float32)
    v = rng.normal(0, 1, (H, Lq, D)).astype(np.float32)
    mask = np.where(np.tril(np.ones((Lq, Lq), bool)), 0.0, -np.inf).astype(np.float32)
    out = oracle.prefill_flash_attention(q, k, v, mask, SCALE)
    s = np.einsum("hqd,hkd->hqk", q.astype(np.float64), k.astype(np.float64)) * float(SCALE)
    s = s + mask[None]
    p = np.exp(s - s.max(-1, keepdims=True))
    ref = np.einsum("hqk,hkd->hqd", p / p.sum(-1, keepdims=True), v.astype(np.float64))
    assert np.abs(out - ref).max() < 3e-6
    # library routine: torch SDPA with a causal mask
    tq, tk, tv = (torch.from_numpy(a)[None] for a in (q, k, v))
    sd = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True,
                                                          scale=float(SCALE))[0].numpy()
    assert np.abs(out - sd).max() < 1e-5
