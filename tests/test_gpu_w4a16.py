"""The int4 weight-only decode path on the device against the CPU restatement of
tools/buddy-codegen/import_model.py:800-815,838-842 and
Int4DequantMatMulVectorizationDecode.cpp:385-468.  Everything is compared bit
for bit: the kernel keeps the reference's order of f16 operations."""
import numpy as np
import pytest
import torch

import buddy_mlir_amd as bma

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("K,N", [(64, 16), (1536, 8960), (8960, 1536), (100, 70), (1, 2), (3000, 130),
                                 (17, 64), (263, 128), (511, 192), (256, 64), (272, 66)])
def test_quantize_pack_gemv_bit_exact(bh, oracle, K, N):
    g = torch.Generator(device="cuda").manual_seed(K * 7 + N)
    W = torch.randn((K, N), generator=g, device="cuda") * 0.02
    q = torch.empty((K, N), dtype=torch.int8, device="cuda")
    s = torch.empty(N, dtype=torch.float32, device="cuda")
    packed = torch.empty((K, N // 2), dtype=torch.int8, device="cuda")
    torch.cuda.synchronize()
    bma.check(bh.buddy_hip_quantize_w4(W.data_ptr(), K, N, q.data_ptr(), s.data_ptr(), None))
    bma.check(bh.buddy_hip_pack_int4(q.data_ptr(), K * N, packed.data_ptr(), None))
    torch.cuda.synchronize()
    qh, sh = oracle.quantize_w4(W.cpu().numpy())
    np.testing.assert_array_equal(q.cpu().numpy(), qh)
    np.testing.assert_array_equal(s.cpu().numpy(), sh)
    ph = oracle.pack_int4(qh)
    np.testing.assert_array_equal(packed.cpu().numpy(), ph)

    rng = np.random.default_rng(K + N)
    a = rng.standard_normal(K).astype(np.float16)
    scale = sh.astype(np.float16)
    c0 = rng.standard_normal(N).astype(np.float16)
    a_d, s_d, c_d = dev(a.view(np.int16)), dev(scale.view(np.int16)), dev(c0.view(np.int16))
    torch.cuda.synchronize()
    bma.check(bh.buddy_hip_gemv_w4a16(a_d.data_ptr(), packed.data_ptr(), s_d.data_ptr(),
                                      c_d.data_ptr(), K, N, None))
    torch.cuda.synchronize()
    want = oracle.w4a16_gemv(a, ph, scale, c0)
    got = c_d.cpu().numpy().view(np.float16)
    np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))


def test_reference_example_inputs_on_device(bh):
    """examples/BuddyMatmul/int4-dequant-matmul-vectorization-decode.mlir:177-190:
    A = 1, every byte = 2, scale = 1, K = 4, N = 4 -> [8, 0, 8, 0]."""
    a = dev(np.ones(4, np.float16).view(np.int16))
    s = dev(np.ones(4, np.float16).view(np.int16))
    c = dev(np.zeros(4, np.float16).view(np.int16))
    packed = dev(np.full((4, 2), 2, np.int8))
    torch.cuda.synchronize()
    bma.check(bh.buddy_hip_gemv_w4a16(a.data_ptr(), packed.data_ptr(), s.data_ptr(),
                                      c.data_ptr(), 4, 4, None))
    torch.cuda.synchronize()
    assert c.cpu().numpy().view(np.float16).astype(np.float32).tolist() == [8.0, 0.0, 8.0, 0.0]


def test_bad_arguments_are_refused(bh):
    x = torch.zeros(8, dtype=torch.int16, device="cuda")
    p = torch.zeros(8, dtype=torch.int8, device="cuda")
    assert bh.buddy_hip_gemv_w4a16(x.data_ptr(), p.data_ptr(), x.data_ptr(), x.data_ptr(), 4, 3, None) != 0
    assert bh.buddy_hip_pack_int4(p.data_ptr(), 7, p.data_ptr(), None) != 0
    assert bh.buddy_hip_gemv_w4a16(None, p.data_ptr(), x.data_ptr(), x.data_ptr(), 4, 4, None) != 0
