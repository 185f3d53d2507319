"""The int4 weight-only decode path on the device against the CPU restatement of
tools/buddy-codegen/import_model.py:800-815,838-842 and
Int4DequantMatMulVectorizationDecode.cpp:385-468.  Everything is compared bit
for bit: the kernel keeps the reference's order of f16 operations.  The opt-in
streaming kernel (buddy_hip_gemv_w4a16_fast: exact products, f32-class sum, one
rounding to f16) cannot equal that chain bit for bit; it is held to the real-number
sum instead: every element within half an f16 unit in the last place of it, and
as a whole no further from it than the reference's own chain is."""
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


def w4_tiles_closed_form(packed, K, N):
    """int4 wave tiles by their definition: tile (g, c) of 1 KiB, lane L byte b =
    low nibble w[128 c + 16 (L / 16) + b][16 g + L % 16], high nibble the same k + 64."""
    q = np.zeros((-(-K // 128) * 128, -(-N // 16) * 16), np.uint8)
    q[:K, 0:N:2] = packed.view(np.uint8) & 0x0F
    q[:K, 1:N:2] = packed.view(np.uint8) >> 4
    groups, chunks = q.shape[1] // 16, q.shape[0] // 128
    t = q.reshape(chunks, 2, 4, 16, groups, 16)       # [c][half][L/16][b][g][L%16]
    lo, hi = t[:, 0], t[:, 1]                         # [c][L/16][b][g][L%16]
    by = (lo | (hi << 4)).transpose(3, 0, 1, 4, 2)    # [g][c][L/16][L%16][b]
    return np.ascontiguousarray(by).reshape(-1).view(np.int8)


@pytest.mark.parametrize("K,N", [(1536, 8960), (8960, 1536), (100, 70), (1, 2), (3000, 130),
                                 (263, 128), (4096, 4096), (20000, 48), (129, 16)])
def test_fast_kernel_against_the_real_number_sum(bh, oracle, K, N):
    rng = np.random.default_rng(K * 3 + N)
    qh = rng.integers(-8, 8, (K, N)).astype(np.int8)
    ph = oracle.pack_int4(qh)
    a = rng.standard_normal(K).astype(np.float16)
    if K > 200:
        a[7] = np.float16(300.0)          # an outlier inside a run
        a[K // 2:K // 2 + 40] *= np.float16(1e-3)
    scale = (rng.uniform(0.5, 1.5, N) * 0.02 / 7).astype(np.float16)
    c0 = rng.standard_normal(N).astype(np.float16)
    packed = dev(ph)
    tiles = torch.empty(bh.buddy_hip_w4_tiles_bytes(K, N), dtype=torch.int8, device="cuda")
    a_d, s_d, c_d = dev(a.view(np.int16)), dev(scale.view(np.int16)), dev(c0.view(np.int16))
    torch.cuda.synchronize()
    bma.check(bh.buddy_hip_pack_w4_tiles(packed.data_ptr(), K, N, tiles.data_ptr(), None))
    bma.check(bh.buddy_hip_gemv_w4a16_fast(a_d.data_ptr(), tiles.data_ptr(), s_d.data_ptr(),
                                           c_d.data_ptr(), K, N, None))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(tiles.cpu().numpy(), w4_tiles_closed_form(ph, K, N))
    got = c_d.cpu().numpy().view(np.float16).astype(np.float64)
    dot = a.astype(np.float64) @ qh.astype(np.float64)
    exact = c0.astype(np.float64) + dot * scale.astype(np.float64)
    # the best an f16 result can be: half a unit in the last place of the exact
    # value (plus the f32 roundings of the finishing multiply-add).  The sums of
    # a wavefront's run (exact integers) and of the k-slices meet in f32: where an
    # outlier makes a slice's sum large and the result is a cancellation, those
    # roundings (2^-24 of the largest partial sum each) show.  With that term at
    # its worst case over the whole row the bound holds for every element; without
    # it for all but a few in a thousand.
    ulp = np.spacing(np.abs(exact).astype(np.float16)).astype(np.float64)
    slack = 4e-7 * (np.abs(c0.astype(np.float64)) + np.abs(dot * scale.astype(np.float64)))
    tight = 0.5 * ulp * (1 + 2.0 ** -9) + slack
    fixed = (float(np.abs(a.astype(np.float64)).max()) * 2.0 ** -23 *
             (np.abs(qh.astype(np.float64)).sum(axis=0) * scale.astype(np.float64)))
    err = np.abs(got - exact)
    assert (err <= tight + fixed).all()
    assert (err > tight).sum() <= max(1, N // 300), int((err > tight).sum())
    # and no further from it than the reference's f16 chain
    ref = oracle.w4a16_gemv(a, ph, scale, c0).astype(np.float64)
    assert np.linalg.norm(got - exact) <= np.linalg.norm(ref - exact) + 1e-12


def test_fast_kernel_special_values(bh, oracle):
    K, N = 512, 64
    rng = np.random.default_rng(1)
    qh = rng.integers(-8, 8, (K, N)).astype(np.int8)
    tiles = torch.empty(bh.buddy_hip_w4_tiles_bytes(K, N), dtype=torch.int8, device="cuda")
    bma.check(bh.buddy_hip_pack_w4_tiles(dev(oracle.pack_int4(qh)).data_ptr(), K, N,
                                         tiles.data_ptr(), None))
    scale = dev(np.ones(N, np.float16).view(np.int16))

    def run(a):
        c = dev(np.zeros(N, np.float16).view(np.int16))
        torch.cuda.synchronize()
        bma.check(bh.buddy_hip_gemv_w4a16_fast(dev(a.view(np.int16)).data_ptr(), tiles.data_ptr(),
                                               scale.data_ptr(), c.data_ptr(), K, N, None))
        torch.cuda.synchronize()
        return c.cpu().numpy().view(np.float16)

    assert (run(np.zeros(K, np.float16)) == 0).all()
    one = np.zeros(K, np.float16)
    one[300] = 1.0                                  # picks row 300 of the weights exactly
    np.testing.assert_array_equal(run(one).astype(np.float32), qh[300].astype(np.float32))
    tiny = np.zeros(K, np.float16)
    tiny[5] = np.float16(6e-8)                      # the smallest subnormal
    np.testing.assert_array_equal(run(tiny), (qh[5].astype(np.float64) * float(tiny[5])).astype(np.float16))
    for poison in (np.nan, np.inf, -np.inf):
        bad = rng.standard_normal(K).astype(np.float16)
        bad[77] = poison
        assert np.isnan(run(bad)).all()


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
    assert bh.buddy_hip_gemv_w4a16_fast(None, p.data_ptr(), x.data_ptr(), x.data_ptr(), 4, 4, None) != 0
    assert bh.buddy_hip_pack_w4_tiles(p.data_ptr(), 4, 3, p.data_ptr(), None) != 0
    assert bh.buddy_hip_w4_tiles_bytes(129, 17) == 2 * 2 * 1024
