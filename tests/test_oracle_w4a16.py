"""Pins the CPU restatement of the reference's W4A16 decode path
(tools/buddy-codegen/import_model.py:810-815;
midend/lib/Conversion/MatMulOptimization/Int4DequantMatMulVectorizationDecode.cpp
:385-468) with checks that do not retype its loops:

* f32 <-> f16 conversions against numpy.float16 (an independent library routine),
  ties and subnormals included;
* nibble packing against its closed form on all 256 byte values, and the
  round trip over the whole int4 range;
* the kernel against a numpy.float16 emulation of the sequential accumulation
  (numpy rounds every float16 operation from float32, which is what the
  reference's x86 target does), and against float64 within the f16 error bound;
* the inputs of the reference's own example, whose result follows in closed
  form: A = 1, every byte = 2 (low nibble 2, high nibble 0), scale = 1, K = 4
  -> [8, 0, 8, 0].
"""
import numpy as np
import pytest


def test_f16_conversion_matches_numpy(oracle):
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(4096).astype(np.float32) * 10,
        np.float32([0, -0.0, 1, 65504, 65520, 1e-8, 6e-8, 6.1e-5, 2049, 2051, 1 + 2**-11,
                    1 + 3 * 2**-11, -2.5e-7, np.inf, -np.inf]),
    ])
    got = oracle.f32_to_f16(x)
    want = x.astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_pack_closed_form_and_round_trip(oracle):
    q = np.array([[v, w] for v in range(-8, 8) for w in range(-8, 8)], np.int8).reshape(-1)
    packed = oracle.pack_int4(q)
    lo, hi = q[0::2].astype(np.int32), q[1::2].astype(np.int32)
    want = (((lo & 0xF) | ((hi & 0xF) << 4)) & 0xFF).astype(np.uint8).view(np.int8)
    assert np.array_equal(packed, want)
    assert np.array_equal(oracle.unpack_int4(packed), q)
    # every byte value decodes to (low, high) = sign-extended nibbles
    b = np.arange(256, dtype=np.uint8).view(np.int8)
    u = oracle.unpack_int4(b).astype(np.int32)
    bb = np.arange(256)
    sext = lambda v: np.where(v >= 8, v - 16, v)
    assert np.array_equal(u[0::2], sext(bb & 0xF)) and np.array_equal(u[1::2], sext(bb >> 4))


def test_reference_example_inputs(oracle):
    """examples/BuddyMatmul/int4-dequant-matmul-vectorization-decode.mlir:177-190"""
    a = np.ones(4, np.float16)
    packed = np.full((4, 2), 2, np.int8)
    scale = np.ones(4, np.float16)
    got = oracle.w4a16_gemv(a, packed, scale)
    assert got.astype(np.float32).tolist() == [8.0, 0.0, 8.0, 0.0]


def numpy_f16_kernel(a, q, scale, c):
    K, N = q.shape
    out = c.copy()
    for n in range(N):
        acc = np.float16(0)
        for k in range(K):
            # the product of an f16 and a 4-bit integer is exact in f32, so one
            # f32 addition rounds like the fused multiply-add does
            acc = np.float16(np.float32(a[k]) * np.float32(np.float16(q[k, n])) + np.float32(acc))
        scaled = np.float16(np.float32(acc) * np.float32(scale[n]))
        out[n] = np.float16(np.float32(out[n]) + np.float32(scaled))
    return out


@pytest.mark.parametrize("K,N", [(64, 16), (300, 10), (1, 2), (777, 6)])
def test_kernel_matches_numpy_float16_emulation(oracle, K, N):
    rng = np.random.default_rng(K + N)
    W = rng.standard_normal((K, N)).astype(np.float32) * 0.02
    q, s = oracle.quantize_w4(W)
    assert q.min() >= -8 and q.max() <= 7
    packed = oracle.pack_int4(q)
    a = rng.standard_normal(K).astype(np.float16)
    scale = s.astype(np.float16)
    c0 = rng.standard_normal(N).astype(np.float16)
    got = oracle.w4a16_gemv(a, packed, scale, c0)
    want = numpy_f16_kernel(a, q, scale, c0)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    # and it is the dot product, up to what f16 accumulation costs
    exact = c0.astype(np.float64) + (a.astype(np.float64) @ q.astype(np.float64)) * scale.astype(np.float64)
    bound = 2.0 ** -10 * (np.abs(a.astype(np.float64)) @ np.abs(q.astype(np.float64))) * K ** 0.5 * scale.astype(np.float64) + 2e-3 * np.abs(exact) + 1e-3
    assert np.all(np.abs(got.astype(np.float64) - exact) <= bound)


def test_w4_quantizer_recipe(oracle):
    """amax / 7, clamp to [-8, 7] (import_model.py:802,838-842)."""
    W = np.float32([[7.0, -14.0, 0.0], [-7.0, 14.0, 0.0], [3.49, 7.1, 0.0]])
    q, s = oracle.quantize_w4(W)
    assert np.allclose(s, [1.0, 2.0, 1e-10])
    assert q.tolist() == [[7, -7, 0], [-7, 7, 0], [3, 4, 0]]
