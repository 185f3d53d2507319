"""The cut of a decode step's attention (buddy_hip_attn_step_plan) is host
arithmetic that the kernels trust: the partials a step launches and folds must
cover its position, fit the cache's workspace (sized for chunks of 64) and stay
within what the fold that is chosen can take.  No device needed."""
import ctypes

import numpy as np
import pytest

import buddy_mlir_amd as bma


def plan(bh, pos, max_len, kv_heads):
    c, u, f = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    bma.check(bh.buddy_hip_attn_step_plan(pos, max_len, kv_heads, ctypes.byref(c),
                                          ctypes.byref(u), ctypes.byref(f)))
    return c.value, u.value, bool(f.value)


@pytest.mark.parametrize("kv_heads", [1, 2, 4, 8])
def test_partials_cover_the_position_and_fit(bh, kv_heads):
    rng = np.random.default_rng(kv_heads)
    cases = [(p, m) for m in (1, 64, 65, 1088, 1152, 1153, 4352, 9472, 32768, 131072, 262144, 1 << 20)
             for p in {0, m - 1, m // 2, min(m - 1, 1151), min(m - 1, 1152), min(m - 1, 2303),
                       min(m - 1, 2304), min(m - 1, 5119), min(m - 1, 5120), min(m - 1, 12544),
                       min(m - 1, 16384)}]
    cases += [(int(p), int(m)) for m in rng.integers(1, 1 << 20, 300)
              for p in rng.integers(0, m, 3)]
    for pos, max_len in cases:
        chunk, used, own = plan(bh, pos, max_len, kv_heads)
        assert chunk in (64, 128, 256)
        all_chunks = -(-max_len // chunk)
        assert pos // chunk + 1 <= used <= all_chunks, (pos, max_len, chunk, used)
        # the workspace holds one partial per 64 positions of the cache
        assert used <= -(-max_len // 64)
        if own:
            assert used <= 4096  # what the fold of its own takes per head
        else:
            assert used <= 36    # what the o_proj launch requests in one trip
        # a cache of up to 1152 positions keeps the one cut of 64-position chunks
        if max_len <= 1152:
            assert (chunk, used, own) == (64, all_chunks, False)


def test_bad_arguments_are_refused(bh):
    c = ctypes.c_int()
    for pos, max_len, kv in ((-1, 10, 2), (10, 10, 2), (0, 0, 2), (0, 10, 0)):
        assert bh.buddy_hip_attn_step_plan(pos, max_len, kv, ctypes.byref(c), ctypes.byref(c),
                                           ctypes.byref(c)) != 0
