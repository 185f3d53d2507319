"""Pins the oracle's element-wise chain (a10), argmax (a11) with the constants
of examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:8,17,38."""
import numpy as np

EPS = np.float32(9.99999997e-7)
INV_1536 = np.float32(6.51041686e-4)


def test_rmsnorm_closed_form(oracle):
    rng = np.random.default_rng(0)
    x = rng.normal(0, 3, 1536).astype(np.float32)
    w = rng.normal(1, 0.1, 1536).astype(np.float32)
    assert np.float32(1.0) / np.float32(1536) == INV_1536
    y = oracle.rmsnorm(x, w, EPS)
    x64 = x.astype(np.float64)
    ref = w * (x64 / np.sqrt((x64 ** 2).mean() + float(EPS)))
    np.testing.assert_allclose(y, ref, rtol=3e-6, atol=1e-6)
    # with unit weights the output has unit RMS
    y1 = oracle.rmsnorm(x, np.ones(1536, np.float32), EPS)
    assert abs(np.sqrt((y1.astype(np.float64) ** 2).mean()) - 1.0) < 1e-5


def test_rope_rotate_half_convention(oracle):
    half = 64
    inv_freq = (1.0 / (1e6 ** (np.arange(half, dtype=np.float64) / half))).astype(np.float32)
    rng = np.random.default_rng(1)
    x = rng.normal(0, 1, (12, 128)).astype(np.float32)
    c0, s0 = oracle.rope_cos_sin(inv_freq, 0)
    np.testing.assert_array_equal(oracle.rope_apply(x, c0, s0), x)  # pos 0 = identity
    pos = 777
    c, s = oracle.rope_cos_sin(inv_freq, pos)
    ang = inv_freq.astype(np.float32) * np.float32(pos)
    np.testing.assert_allclose(c[:half], np.cos(ang.astype(np.float64)), atol=1e-6)
    np.testing.assert_array_equal(c[:half], c[half:])
    y = oracle.rope_apply(x, c, s)
    # rotate-half: y = x*cos + cat(-x[64:], x[:64])*sin
    rot = np.concatenate([-x[:, half:], x[:, :half]], axis=1)
    np.testing.assert_allclose(y, x * c + rot * s, rtol=1e-6, atol=1e-6)
    # a rotation preserves the norm of each (j, j+64) pair
    n_in = x[:, :half] ** 2 + x[:, half:] ** 2
    n_out = y[:, :half] ** 2 + y[:, half:] ** 2
    np.testing.assert_allclose(n_out, n_in, rtol=1e-5)
    # interleaved (GPT-J) pairing would not preserve these pairs
    assert not np.allclose(y[:, 0::2] ** 2 + y[:, 1::2] ** 2,
                           x[:, 0::2] ** 2 + x[:, 1::2] ** 2, rtol=1e-3)


def test_silu_mul(oracle):
    rng = np.random.default_rng(2)
    g = rng.normal(0, 3, 8960).astype(np.float32)
    u = rng.normal(0, 1, 8960).astype(np.float32)
    h = oracle.silu_mul(g, u)
    g64 = g.astype(np.float64)
    np.testing.assert_allclose(h, g64 / (1 + np.exp(-g64)) * u, rtol=1e-6, atol=1e-7)
    assert oracle.silu_mul(np.zeros(1), np.ones(1))[0] == 0.0


def test_argmax_first_on_ties(oracle):
    x = np.array([1, 5, 3, 5, 5, 2], np.float32)
    assert oracle.argmax_first(x) == 1
    assert oracle.argmax_first(np.zeros(10, np.float32)) == 0
    assert oracle.argmax_first(np.array([-3, -1, -2], np.float32)) == 1
