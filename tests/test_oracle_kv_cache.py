"""Pins the CPU restatement of the reference's KV-cache overflow handling
(runtime/include/buddy/runtime/llm/KVCacheManager.h:150-268) by what the
arithmetic fixes, not by retyping its loops:

* the move is a plain slice assignment (numpy) with a zero tail;
* rotating a key that carries the RoPE of position p by -d gives the key with
  the RoPE of position p - d (angle addition), checked against the RoPE
  restatement that is itself pinned by the model IR's constants;
* the rotation is orthogonal (pair norms survive) and -d followed by +d is the
  identity within rounding;
* the reference's refusals (bad keep / discard) leave the cache untouched.
"""
import numpy as np
import pytest


def inv_freq(dim, theta=1e6):
    return (1.0 / theta ** (np.arange(0, dim, 2, dtype=np.float32) / np.float32(dim))).astype(np.float32)


@pytest.mark.parametrize("heads,L,D,keep,discard,count",
                         [(2, 64, 128, 4, 16, 64), (1, 16, 8, 0, 1, 2), (3, 40, 16, 5, 10, 33),
                          (2, 32, 128, 0, 31, 32)])
def test_discard_is_a_slice_move_with_zero_tail(oracle, heads, L, D, keep, discard, count):
    rng = np.random.default_rng(1)
    c = rng.standard_normal((heads, L, D)).astype(np.float32)
    rc, got = oracle.kv_discard(c, keep, discard, count)
    assert rc == 0
    tail = count - keep - discard
    want = np.zeros_like(c)
    want[:, :keep] = c[:, :keep]
    want[:, keep:keep + tail] = c[:, keep + discard:count]
    assert np.array_equal(got, want)


@pytest.mark.parametrize("keep,discard,count", [(4, 0, 10), (-1, 2, 10), (10, 2, 10), (4, 6, 10),
                                                (4, 7, 10)])
def test_discard_refusals_leave_the_cache_alone(oracle, keep, discard, count):
    c = np.arange(2 * 12 * 4, dtype=np.float32).reshape(2, 12, 4)
    rc, got = oracle.kv_discard(c, keep, discard, count)
    assert rc == -1 and np.array_equal(got, c)


def test_count_is_clamped_to_the_cache_length(oracle):
    c = np.arange(1 * 8 * 2, dtype=np.float32).reshape(1, 8, 2)
    rc, got = oracle.kv_discard(c, 1, 2, 100)  # behaves like count = 8
    rc2, want = oracle.kv_discard(c, 1, 2, 8)
    assert rc == 0 and rc2 == 0 and np.array_equal(got, want)


def test_adjust_equals_rope_at_the_new_position(oracle):
    heads, L, D, keep, discard, count = 2, 48, 128, 3, 12, 40
    f = inv_freq(D)
    rng = np.random.default_rng(2)
    raw = rng.standard_normal((heads, L, D)).astype(np.float32)  # keys before RoPE
    roped = np.zeros_like(raw)
    for p in range(count):
        cs, sn = oracle.rope_cos_sin(f, p)
        roped[:, p] = oracle.rope_apply(raw[:, p], cs, sn)
    rc, moved = oracle.kv_discard(roped, keep, discard, count)
    assert rc == 0
    got = oracle.kv_adjust_rope(moved, keep, discard, count, f)
    tail = count - keep - discard
    for t in range(tail):
        new_pos = keep + t          # where the token sits now
        cs, sn = oracle.rope_cos_sin(f, new_pos)
        want = oracle.rope_apply(raw[:, keep + discard + t], cs, sn)
        # two rotations against one: a few ulp of the pair norm
        np.testing.assert_allclose(got[:, new_pos], want, rtol=0, atol=3e-5)
    # the kept prefix and the cleared tail are not touched
    assert np.array_equal(got[:, :keep], roped[:, :keep])
    assert not got[:, keep + tail:].any()


def test_adjust_is_orthogonal_and_invertible(oracle):
    heads, L, D, keep, discard, count = 1, 20, 16, 2, 5, 18
    f = inv_freq(D, 10000.0)
    rng = np.random.default_rng(3)
    k = rng.standard_normal((heads, L, D)).astype(np.float32)
    got = oracle.kv_adjust_rope(k, keep, discard, count, f)
    half = D // 2
    n0 = k[..., :half] ** 2 + k[..., half:] ** 2
    n1 = got[..., :half] ** 2 + got[..., half:] ** 2
    np.testing.assert_allclose(n1, n0, rtol=2e-6, atol=1e-7)
    # rows outside [keep, keep + count - keep - discard) are untouched
    rows = count - keep - discard
    assert np.array_equal(got[:, :keep], k[:, :keep])
    assert np.array_equal(got[:, keep + rows:], k[:, keep + rows:])
    # rotate forward again: a key rotated by -d then by +d (a RoPE of position d
    # in pair form) is itself
    cs, sn = oracle.rope_cos_sin(f, discard)
    back = oracle.rope_apply(got[0, keep:keep + rows], cs, sn)
    np.testing.assert_allclose(back, k[0, keep:keep + rows], rtol=0, atol=2e-6)


def test_adjust_with_nothing_to_do(oracle):
    k = np.ones((1, 8, 4), np.float32)
    f = inv_freq(4)
    assert np.array_equal(oracle.kv_adjust_rope(k, 2, 0, 8, f), k)
    assert np.array_equal(oracle.kv_adjust_rope(k, 2, 6, 8, f), k)
