"""The decode attention entry point that allocates nothing
(buddy_hip_gqa_decode_attention_static: partials in a buffer built into the
library) against the entry point that takes a workspace, through the C ABI:
same kernels, so the results must be identical bit for bit -- on two calls in a
row, the second with a smaller input, because the built-in buffer keeps the
first call's contents."""
import numpy as np
import pytest
import torch

import buddy_mlir_amd as bma
from buddy_mlir_amd import synthetic

pytestmark = pytest.mark.gpu

SCALE = float(np.float32(0.0883883461))


def both(bh, H, HKV, L, pos, seed):
    D = 128
    g = torch.Generator(device="cuda").manual_seed(seed)
    qkv = torch.randn((H + 2 * HKV) * D, generator=g, device="cuda")
    kc = torch.randn((HKV, L, D), generator=g, device="cuda")
    vc = torch.randn((HKV, L, D), generator=g, device="cuda")
    inv = synthetic.inv_freq(D)
    pos_t = torch.tensor([pos], dtype=torch.int32, device="cuda")
    res = []
    for static in (False, True):
        k, v = kc.clone(), vc.clone()
        out = torch.full((H * D,), float("nan"), device="cuda")
        lse = torch.full((H,), float("nan"), device="cuda")
        torch.cuda.synchronize()
        if static:
            bma.check(bh.buddy_hip_gqa_decode_attention_static(
                qkv.data_ptr(), inv.data_ptr(), pos_t.data_ptr(), k.data_ptr(), v.data_ptr(),
                out.data_ptr(), lse.data_ptr(), H, HKV, D, L, SCALE, None))
        else:
            nb = bh.buddy_hip_attn_decode_workspace_bytes(H, L)
            ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
            bma.check(bh.buddy_hip_gqa_decode_attention(
                qkv.data_ptr(), inv.data_ptr(), pos_t.data_ptr(), k.data_ptr(), v.data_ptr(),
                out.data_ptr(), lse.data_ptr(), H, HKV, D, L, SCALE, ws.data_ptr(), nb, None))
        torch.cuda.synchronize()
        res.append((out.cpu().numpy(), lse.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy()))
    return res


def test_static_scratch_entry_point_matches_the_workspace_one(bh):
    # a long cache first (68 chunks per head), then a smaller call that leaves
    # most of the first call's partials behind in the built-in buffer
    for H, HKV, L, pos, seed in ((12, 2, 4352, 4300, 1), (4, 2, 1088, 70, 2), (12, 2, 1088, 0, 3)):
        (o0, l0, k0, v0), (o1, l1, k1, v1) = both(bh, H, HKV, L, pos, seed)
        assert np.isfinite(o0).all() and np.isfinite(l0).all()
        np.testing.assert_array_equal(o1, o0)
        np.testing.assert_array_equal(l1, l0)
        np.testing.assert_array_equal(k1, k0)
        np.testing.assert_array_equal(v1, v0)


def test_static_scratch_entry_point_refuses_what_does_not_fit(bh):
    t = torch.zeros(8, device="cuda")
    p = t.data_ptr()
    # 64 heads x 16384 positions = 16384 (head, chunk) pairs > 8192
    rc = bh.buddy_hip_gqa_decode_attention_static(p, p, p, p, p, p, None, 64, 8, 128, 16384,
                                                  SCALE, None)
    assert rc == 1
    assert b"exceeds the built-in scratch" in bh.buddy_hip_last_error()


def test_static_scratch_entry_point_recorded_into_a_graph(bh):
    """The use the entry point exists for: after buddy_hip_static_scratch_init()
    the call is captured into a HIP graph (no allocation, no address lookup
    under capture) and replayed with new inputs in the same buffers; every
    replay, with eager work and synchronisations of the program's own between
    them, equals the workspace entry point bit for bit."""
    H, HKV, L, D = 12, 2, 1088, 128
    bma.check(bh.buddy_hip_static_scratch_init())
    g = torch.Generator(device="cuda").manual_seed(5)
    qkv = torch.randn((H + 2 * HKV) * D, generator=g, device="cuda")
    kc = torch.randn((HKV, L, D), generator=g, device="cuda")
    vc = torch.randn((HKV, L, D), generator=g, device="cuda")
    inv = synthetic.inv_freq(D)
    pos_t = torch.tensor([900], dtype=torch.int32, device="cuda")
    out = torch.zeros(H * D, device="cuda")
    lse = torch.zeros(H, device="cuda")
    nb = bh.buddy_hip_attn_decode_workspace_bytes(H, L)
    ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
    k2, v2 = kc.clone(), vc.clone()
    out2, lse2 = torch.zeros_like(out), torch.zeros_like(lse)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.graph(graph, stream=side):
        bma.check(bh.buddy_hip_gqa_decode_attention_static(
            qkv.data_ptr(), inv.data_ptr(), pos_t.data_ptr(), kc.data_ptr(), vc.data_ptr(),
            out.data_ptr(), lse.data_ptr(), H, HKV, D, L, SCALE, side.cuda_stream))
    torch.cuda.synchronize()
    for replay, pos in enumerate((900, 17, 1087, 333)):
        qkv.copy_(torch.randn(qkv.shape, generator=g, device="cuda"))
        pos_t.fill_(pos)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        bma.check(bh.buddy_hip_gqa_decode_attention(
            qkv.data_ptr(), inv.data_ptr(), pos_t.data_ptr(), k2.data_ptr(), v2.data_ptr(),
            out2.data_ptr(), lse2.data_ptr(), H, HKV, D, L, SCALE, ws.data_ptr(), nb, None))
        torch.cuda.synchronize()
        assert torch.isfinite(out).all(), replay
        assert torch.equal(out, out2) and torch.equal(lse, lse2), replay
        assert torch.equal(kc, k2) and torch.equal(vc, v2), replay
