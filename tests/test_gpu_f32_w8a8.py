"""GPU parity of the remaining kernels on the path: plain and panel-packed f32
decode GEMV, the reference panel packing on device, the w8a8 matmul with exact
int32 partial sums, and the f32 matmul behind `_mlir_ciface_buddy_matmul_f32`."""
import ctypes

import numpy as np
import pytest
import torch

import buddy_mlir_amd as bma
from buddy_mlir_amd import ops, synthetic
from parity import check_close

pytestmark = pytest.mark.gpu


def sync_check(rc):
    bma.check(rc)
    torch.cuda.synchronize()


# 4096 columns and more take 32-column strips, 8192 and more 64-column strips;
# 4099 and 8197 leave a ragged last strip and rows that are not 16-byte aligned
@pytest.mark.parametrize("K,N", [(1536, 1536), (1536, 256), (128, 64), (100, 70), (8960, 1536),
                                 (1536, 4096), (300, 4099), (1536, 8960), (77, 8197)])
def test_f32_gemv_with_bias(bh, oracle, K, N):
    g = torch.Generator(device="cuda").manual_seed(K + N)
    x = torch.randn(K, generator=g, device="cuda")
    B = torch.randn((K, N), generator=g, device="cuda") * 0.02
    bias = torch.randn(N, generator=g, device="cuda")
    y = torch.empty(N, device="cuda")
    torch.cuda.synchronize()
    sync_check(bh.buddy_hip_gemv_f32(x.data_ptr(), B.data_ptr(), bias.data_ptr(),
                                     y.data_ptr(), K, N, 0, None))
    want = bias.cpu().numpy() + oracle.gemv_f32(x.cpu().numpy(), B.cpu().numpy(),
                                                np.zeros(N, np.float32), 32, True)
    check_close(y.cpu().numpy(), want)


@pytest.mark.parametrize("norm", [False, True])
@pytest.mark.parametrize("K,N", [(1536, 2048), (1536, 256), (128, 64), (100, 70), (33, 9),
                                 (8960, 1536), (1, 1)])
def test_f32_gemv_over_tiles(bh, oracle, K, N, norm):
    g = torch.Generator(device="cuda").manual_seed(K + 2 * N)
    x = torch.randn(K, generator=g, device="cuda")
    B = torch.randn((K, N), generator=g, device="cuda") * 0.02
    bias = torch.randn(N, generator=g, device="cuda")
    nw = torch.rand(K, generator=g, device="cuda") + 0.5
    eps = 1e-6
    nbytes = bh.buddy_hip_f32_tiles_bytes(K, N)
    assert nbytes == ((K + 31) // 32 * 32) * ((N + 7) // 8 * 8) * 4
    T = torch.full((nbytes // 4,), float("nan"), device="cuda")
    y = torch.empty(N, device="cuda")
    torch.cuda.synchronize()
    sync_check(bh.buddy_hip_tile_f32(B.data_ptr(), K, N, T.data_ptr(), None))
    # closed form of the layout, padding zero
    Th, Bh = T.cpu().numpy(), B.cpu().numpy()
    blocks = (K + 31) // 32
    rng = np.random.default_rng(K)
    for _ in range(200):
        k, n = int(rng.integers(K)), int(rng.integers(N))
        assert Th[((n // 8) * blocks + k // 32) * 256 + (k % 32) * 8 + n % 8] == Bh[k, n]
    assert not np.isnan(Th).any() and np.count_nonzero(Th) == np.count_nonzero(Bh)
    sync_check(bh.buddy_hip_gemv_f32_tiles(x.data_ptr(), T.data_ptr(), bias.data_ptr(),
                                           nw.data_ptr() if norm else None, eps,
                                           y.data_ptr(), K, N, 0, None))
    xh = x.cpu().numpy()
    if norm:
        xh = oracle.rmsnorm(xh, nw.cpu().numpy(), eps)
    want = bias.cpu().numpy() + oracle.gemv_f32(xh, Bh, np.zeros(N, np.float32), 32, True)
    check_close(y.cpu().numpy(), want)
    # accumulate flag: y += ..., deterministic
    y2 = y.clone()
    sync_check(bh.buddy_hip_gemv_f32_tiles(x.data_ptr(), T.data_ptr(), None,
                                           nw.data_ptr() if norm else None, eps,
                                           y2.data_ptr(), K, N, 1, None))
    check_close(y2.cpu().numpy(), y.cpu().numpy() + (want - bias.cpu().numpy()))


@pytest.mark.parametrize("K,N", [(128, 64), (1536, 8960), (1536, 256)])
def test_panel_pack_and_packed_gemv(bh, oracle, K, N):
    g = torch.Generator(device="cuda").manual_seed(K)
    B = torch.randn((K, N), generator=g, device="cuda")
    P = torch.empty_like(B)
    U = torch.empty_like(B)
    torch.cuda.synchronize()
    sync_check(bh.buddy_hip_pack_panels_f32(B.data_ptr(), K, N, 32, P.data_ptr(), None))
    sync_check(bh.buddy_hip_unpack_panels_f32(P.data_ptr(), K, N, 32, U.data_ptr(), None))
    Bh = B.cpu().numpy()
    np.testing.assert_array_equal(P.cpu().numpy(), oracle.pack_panels(Bh, 32))  # bit-exact
    np.testing.assert_array_equal(U.cpu().numpy(), Bh)
    x = torch.randn(K, generator=g, device="cuda")
    y0 = torch.randn(N, generator=g, device="cuda")
    for accumulate in (False, True):
        y = y0.clone()
        sync_check(bh.buddy_hip_gemv_f32_panels(x.data_ptr(), P.data_ptr(), y.data_ptr(), K, N,
                                                1 if accumulate else 0, None))
        want = oracle.gemv_packed_f32(x.cpu().numpy(), P.cpu().numpy(), y0.cpu().numpy(), K, N,
                                      32, zero_init=not accumulate)
        check_close(y.cpu().numpy(), want)
    # a ragged last panel is refused, as in the reference
    assert bh.buddy_hip_pack_panels_f32(B.data_ptr(), K, N - 1, 32, P.data_ptr(), None) != 0


# up to 16 rows: the dot-product GEMV; above: one int8 plane through the prefill
# matmul (ragged M, K and N, the four tile shapes, the full MLP shapes)
@pytest.mark.parametrize("M,K,N", [(1, 1536, 8960), (3, 200, 40), (16, 1536, 256), (1, 8960, 1536),
                                   (17, 64, 64), (50, 100, 30), (144, 256, 16384),
                                   (300, 256, 10240), (200, 192, 16384), (512, 1536, 8960),
                                   (512, 8960, 1536)])
def test_w8a8_int32_partial_sums_bit_exact(bh, oracle, M, K, N):
    q, s = synthetic.quantized_linear(K, N, M + K)
    packed = ops.pack_w8(q)
    g = torch.Generator(device="cuda").manual_seed(N)
    A = torch.randn((M, K), generator=g, device="cuda")
    C = torch.empty((M, N), device="cuda")
    acc = torch.empty((M, N), dtype=torch.int32, device="cuda")
    nb = bh.buddy_hip_w8a8_workspace_bytes(M, K)
    ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    sync_check(bh.buddy_hip_w8a8_matmul(A.data_ptr(), packed.data_ptr(), s.data_ptr(),
                                        C.data_ptr(), acc.data_ptr(), M, K, N, ws.data_ptr(),
                                        nb, None))
    wC, wacc = oracle.w8a8_matmul(A.cpu().numpy(), q.cpu().numpy(), s.cpu().numpy())
    np.testing.assert_array_equal(acc.cpu().numpy(), wacc)  # integers: exact
    np.testing.assert_array_equal(C.cpu().numpy(), wC)      # same f32 ops on them
    # the integer sums are optional
    C2 = torch.empty((M, N), device="cuda")
    sync_check(bh.buddy_hip_w8a8_matmul(A.data_ptr(), packed.data_ptr(), s.data_ptr(),
                                        C2.data_ptr(), None, M, K, N, ws.data_ptr(), nb, None))
    np.testing.assert_array_equal(C2.cpu().numpy(), wC)


def test_w8a8_many_rows_extremes(bh, oracle):
    """All-zero activations (the 1e-10 floor of the scale), and +-127 everywhere
    with weights of +-128: the largest sums the int32 accumulators meet."""
    M, K, N = 40, 1024, 48
    q = torch.full((K, N), -128, dtype=torch.int8, device="cuda")
    q[:, 1::2] = 127
    s = torch.full((N,), 0.01, device="cuda")
    packed = ops.pack_w8(q)
    nb = bh.buddy_hip_w8a8_workspace_bytes(M, K)
    ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
    for A in (torch.zeros((M, K), device="cuda"), torch.full((M, K), -3.0, device="cuda")):
        C = torch.empty((M, N), device="cuda")
        acc = torch.empty((M, N), dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        sync_check(bh.buddy_hip_w8a8_matmul(A.data_ptr(), packed.data_ptr(), s.data_ptr(),
                                            C.data_ptr(), acc.data_ptr(), M, K, N,
                                            ws.data_ptr(), nb, None))
        wC, wacc = oracle.w8a8_matmul(A.cpu().numpy(), q.cpu().numpy(), s.cpu().numpy())
        np.testing.assert_array_equal(acc.cpu().numpy(), wacc)
        np.testing.assert_array_equal(C.cpu().numpy(), wC)
    assert abs(int(wacc[0, 0])) == K * 127 * 128


def test_buddy_matmul_f32_entry_point(bh):
    # tests/Conversion/matmul-blis-vectorization.mlir shape: 9x4 . 4x17 of ones
    A = np.ones((9, 4), np.float32)
    B = np.ones((4, 17), np.float32)
    res = bma.MemRefF32_2D()
    bh._mlir_ciface_buddy_matmul_f32(ctypes.byref(res), ctypes.byref(bma.MemRef(A.ctypes.data, [9, 4])),
                                     ctypes.byref(bma.MemRef(B.ctypes.data, [4, 17])))
    assert res.aligned and list(res.sizes) == [9, 17] and list(res.strides) == [17, 1]
    out = np.ctypeslib.as_array(res.aligned, shape=(9, 17)).copy()
    ctypes.CDLL(None).free(res.allocated)
    assert (out == 4).all()
    # strided operands, random values
    rng = np.random.default_rng(0)
    Abig = rng.normal(0, 1, (70, 2 * 130)).astype(np.float32)
    Bm = rng.normal(0, 1, (130, 90)).astype(np.float32)
    res = bma.MemRefF32_2D()
    bh._mlir_ciface_buddy_matmul_f32(
        ctypes.byref(res), ctypes.byref(bma.MemRef(Abig.ctypes.data, [70, 130], strides=[260, 2])),
        ctypes.byref(bma.MemRef(Bm.ctypes.data, [130, 90])))
    out = np.ctypeslib.as_array(res.aligned, shape=(70, 90)).copy()
    ctypes.CDLL(None).free(res.allocated)
    check_close(out, Abig[:, ::2].astype(np.float64) @ Bm.astype(np.float64))
