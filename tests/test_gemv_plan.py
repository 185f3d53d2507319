"""How the one-to-four-row GEMV cuts a launch (host arithmetic behind
buddy_hip_gemv_w8a32_plan; nothing is launched).

A wrong cut is an out-of-bounds access on the device, so the invariants the
kernels rely on are checked here over many shapes, and the launch shapes of the
decode step are pinned."""
import ctypes

import numpy as np
import pytest

TWO, FOLD, UNALIGNED = 1, 2, 4
DIGITS, F32, BATCH_INT8, BATCH_BF16 = 0, 1, 2, 3


class Plan(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in
                ("kernel", "rows_compiled", "channel_groups", "tiles", "groups_per_workgroup",
                 "k_slices", "wavefronts", "workgroups", "split", "tiles_per_wavefront", "slots",
                 "reserved")] + [("lds_bytes", ctypes.c_int64)]


def plan(bh, M, K, N, flags=0):
    p = Plan()
    assert bh.buddy_hip_gemv_w8a32_plan(M, K, N, flags, ctypes.byref(p)) == 0, \
        bh.buddy_hip_last_error()
    return p


SINGLE = {1: [2, 3, 4, 5, 6, 7, 8, 9, 10, 12, 14, 16], 2: [2, 3, 4, 6, 8, 10, 12],
          4: [2, 3, 4, 6, 8]}
DUAL = {1: [2, 3, 4, 5, 6, 7, 8, 9], 2: [2, 3, 4, 6, 8], 4: [2, 3, 4, 6]}


def check_invariants(p, M, K, N, flags):
    assert p.channel_groups == -(-N // 16) and p.tiles == -(-K // 64)
    assert p.wavefronts == p.groups_per_workgroup * p.k_slices
    assert p.wavefronts in (4, 8, 16)
    # every channel group has a workgroup (two when split), every tile a wavefront
    assert (p.workgroups >> p.split) * p.groups_per_workgroup >= p.channel_groups
    assert p.k_slices * p.tiles_per_wavefront >= p.tiles
    assert p.tiles_per_wavefront == -(-p.tiles // p.k_slices)
    assert p.lds_bytes <= 160 * 1024
    if p.split:
        assert not flags & (TWO | FOLD) and M <= 4 and p.groups_per_workgroup == 1
    if p.kernel == DIGITS:
        assert M <= 4 and not flags & UNALIGNED
        assert p.slots >= p.tiles_per_wavefront
        if p.split:
            assert p.slots in (4, 6, 8, 10)
        elif flags & FOLD:
            assert p.slots in (2, 3, 4) and M == 1
        else:
            assert p.slots in (DUAL if flags & TWO else SINGLE)[p.rows_compiled]
        # the planes of four tiles per wavefront and the meeting place of the k-slices
        assert p.lds_bytes == p.wavefronts * p.rows_compiled * (4 * 256 + 33 * 4)
    else:
        assert p.kernel == F32 and p.slots == 0


def test_invariants_over_many_shapes(bh):
    rng = np.random.default_rng(0)
    shapes = [(1, 1), (1, 17), (64, 16), (63, 15), (65, 17), (100, 70), (1536, 8960),
              (8960, 1536), (1536, 151936), (4096, 128256), (14336, 4096), (16384, 2064),
              (11264, 64), (1 << 20, 16), (16, 1 << 20)]
    shapes += [(int(rng.integers(1, 20000)), int(rng.integers(1, 40000))) for _ in range(400)]
    seen = set()
    for K, N in shapes:
        for M in (1, 2, 3, 4):
            for flags in (0, TWO, UNALIGNED, FOLD if M == 1 else 0):
                p = plan(bh, M, K, N, flags)
                check_invariants(p, M, K, N, flags)
                seen.add((p.kernel, p.split))
    assert seen == {(DIGITS, 0), (DIGITS, 1), (F32, 0), (F32, 1)}


def test_decode_step_launch_shapes(bh):
    """Qwen2-1.5B: every per-layer GEMV of a decode step runs the digit-plane
    kernel with all its workgroups resident at once; lm_head keeps the f32 one."""
    p = plan(bh, 1, 1536, 2048)                       # RMSNorm + q|k|v
    assert (p.kernel, p.workgroups, p.wavefronts, p.slots) == (DIGITS, 128, 8, 3)
    p = plan(bh, 1, 1536, 1536, FOLD)                 # fold + o_proj
    assert (p.kernel, p.workgroups, p.wavefronts, p.slots) == (DIGITS, 96, 16, 2)
    p = plan(bh, 1, 1536, 8960, TWO)                  # RMSNorm + gate|up + SiLU*mul
    assert (p.kernel, p.workgroups, p.wavefronts, p.slots) == (DIGITS, 560, 8, 3)
    p = plan(bh, 1, 8960, 1536)                       # down: two workgroups per channel group
    assert (p.kernel, p.workgroups, p.wavefronts, p.slots, p.split) == (DIGITS, 192, 16, 10, 1)
    p = plan(bh, 1, 1536, 151936)                     # lm_head: 24 tiles per wavefront
    assert (p.kernel, p.workgroups, p.wavefronts, p.tiles_per_wavefront) == (F32, 2374, 4, 24)
    # the same matrices at four rows
    p = plan(bh, 4, 1536, 8960, TWO)
    assert (p.kernel, p.rows_compiled, p.slots) == (DIGITS, 4, 3)
    p = plan(bh, 4, 8960, 1536)
    assert (p.kernel, p.rows_compiled, p.slots, p.split) == (DIGITS, 4, 10, 1)


def test_other_kernels_and_refusals(bh):
    assert plan(bh, 8, 1536, 8960).kernel == BATCH_INT8
    assert plan(bh, 8, 1534, 8960).kernel == F32          # K % 4 != 0: f32 kernel, 8 rows
    assert plan(bh, 3, 1536, 8960, UNALIGNED).kernel == F32
    p = Plan()
    for M, K, N, flags in [(0, 64, 16, 0), (17, 64, 16, 0), (1, 0, 16, 0), (1, 64, 0, 0),
                           (2, 64, 16, FOLD), (1, 64, 16, FOLD | TWO)]:
        assert bh.buddy_hip_gemv_w8a32_plan(M, K, N, flags, ctypes.byref(p)) != 0
    assert bh.buddy_hip_gemv_w8a32_plan(1, 64, 16, 0, None) != 0
