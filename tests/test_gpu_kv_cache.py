"""KV-cache overflow handling on the device against the CPU restatement of
kvcache::discardKVCache / adjustKeyCacheRope
(runtime/include/buddy/runtime/llm/KVCacheManager.h:150-268).

The move is byte work and the rotation uses the host's cos/sin with unfused
multiplies and adds, so everything here is compared bit for bit."""
import ctypes

import numpy as np
import pytest
import torch

import buddy_mlir_amd as bma
from buddy_mlir_amd import synthetic
from buddy_mlir_amd.session import Shape

import oracle_lib
from parity import check_close

pytestmark = pytest.mark.gpu


def run_discard(bh, tensors, heads, L, D, keep, discard, count, inv_freq):
    ptrs = (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])
    f = None if inv_freq is None else np.ascontiguousarray(inv_freq, np.float32)
    torch.cuda.synchronize()
    rc = bh.buddy_hip_kv_discard(ptrs, len(tensors), heads, L, D, keep, discard, count,
                                 None if f is None else f.ctypes.data, None)
    torch.cuda.synchronize()
    return rc


@pytest.mark.parametrize("heads,L,D,keep,discard,count",
                         [(2, 1088, 128, 4, 256, 1088), (2, 64, 128, 0, 1, 64),
                          (3, 40, 16, 5, 10, 33), (1, 300, 256, 7, 3, 299),
                          (2, 128, 128, 16, 100, 120)])
@pytest.mark.parametrize("rotate", [True, False])
def test_discard_and_rerotate_bit_exact(bh, oracle, heads, L, D, keep, discard, count, rotate):
    g = torch.Generator(device="cuda").manual_seed(keep + discard + count)
    n = 6  # three layers: k0 v0 k1 v1 k2 v2
    tensors = [torch.randn((heads, L, D), generator=g, device="cuda") for _ in range(n)]
    host = [t.cpu().numpy() for t in tensors]
    f = synthetic.inv_freq(D).cpu().numpy()
    assert run_discard(bh, tensors, heads, L, D, keep, discard, count, f if rotate else None) == 0
    for i, (t, h) in enumerate(zip(tensors, host)):
        rc, want = oracle.kv_discard(h, keep, discard, count)
        assert rc == 0
        if rotate and i % 2 == 0:
            want = oracle.kv_adjust_rope(want, keep, discard, count, f)
        np.testing.assert_array_equal(t.cpu().numpy(), want, err_msg=f"tensor {i}")


@pytest.mark.parametrize("keep,discard,count", [(4, 0, 10), (-1, 2, 10), (10, 2, 10), (4, 6, 10)])
def test_refused_parameters_leave_the_cache_alone(bh, keep, discard, count):
    t = torch.randn((2, 12, 128), device="cuda")
    before = t.clone()
    rc = run_discard(bh, [t, t.clone()], 2, 12, 128, keep, discard, count, None)
    assert rc != 0 and b"kv_discard" in bh.buddy_hip_last_error()
    assert torch.equal(t, before)


SMALL = Shape(layers=2, hidden=256, heads=4, kv_heads=2, head_dim=128, inter=512,
              vocab=1024, max_len=64, rms_eps=1e-6)


def test_generation_across_a_discard_matches_the_reference_loop(oracle):
    """The reference's decode loop when the cache fills up
    (runtime/include/buddy/runtime/llm/TextGeneration.cpp:231-237): discard,
    re-rotate, continue at position count - discard."""
    sess, host = synthetic.build_session(SMALL, context=56, keep_host=True, ln_jitter=0.1)
    om = oracle_lib.model_from_host(oracle, SMALL, host)
    kv = [a.copy() for a in host["kv"]]
    f = host["globals"]["inv_freq"]
    tok, pos = 11, 56
    got, want = [], []

    def step(tok_in, pos_in):
        nxt, logits = sess.decode(tok_in, pos_in)
        otok, ologits = om.decode_step(tok_in, pos_in, kv)
        check_close(logits, ologits)
        got.append(nxt)
        want.append(otok)
        return otok

    for _ in range(8):  # fills positions 56..63: the cache is full
        tok = step(tok, pos)
        pos += 1
    keep, discard, count = 4, 24, 64
    sess.discard_kv(keep, discard, count)
    for j in range(len(kv)):
        rc, moved = oracle.kv_discard(kv[j], keep, discard, count)
        assert rc == 0
        kv[j][...] = oracle.kv_adjust_rope(moved, keep, discard, count, f) if j % 2 == 0 else moved
    for j in range(len(kv)):  # the prompt rows (the same bits on both sides) moved bit for bit
        got_kv = sess.get_kv(j)
        np.testing.assert_array_equal(got_kv[:, :keep], kv[j][:, :keep])
        np.testing.assert_array_equal(got_kv[:, keep:56 - discard], kv[j][:, keep:56 - discard])
        assert not got_kv[:, count - discard:].any()
    pos = count - discard
    for _ in range(6):
        tok = step(tok, pos)
        pos += 1
    assert got == want
    sess.close()
