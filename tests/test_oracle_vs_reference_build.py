"""The restated sampler and KV-cache functions of the oracle, and the memref
descriptor of the C interface, against the reference's own code: runtime/include/buddy/runtime/llm/Sampler.h and
KVCacheManager.h are header-only C++ that needs the standard library only, so
`make -C oracle ref` compiles them from the reference tree into
oracle/_ref/libref_llm.so (oracle/ref_llm.cpp is the C interface around them).
Where that library has not been built these tests skip."""
import numpy as np
import pytest

import oracle_lib

ref = oracle_lib.load_reference_runtime()
pytestmark = pytest.mark.skipif(ref is None, reason="oracle/_ref/libref_llm.so not built "
                                "(needs the reference tree: make -C oracle ref)")

CONFIGS = [
    dict(temperature=0.0, top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=1.0, repeat_last_n=64),
    dict(temperature=0.0, top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=1.3, repeat_last_n=8),
    dict(temperature=0.8, top_k=40, top_p=0.95, min_p=0.05, repeat_penalty=1.1, repeat_last_n=64),
    dict(temperature=1.5, top_k=5, top_p=1.0, min_p=0.0, repeat_penalty=1.0, repeat_last_n=64),
    dict(temperature=0.7, top_k=0, top_p=0.9, min_p=0.0, repeat_penalty=1.0, repeat_last_n=64),
    dict(temperature=1.0, top_k=1, top_p=1.0, min_p=0.0, repeat_penalty=1.0, repeat_last_n=64),
    dict(temperature=2.0, top_k=64, top_p=0.5, min_p=0.2, repeat_penalty=2.0, repeat_last_n=3),
    dict(temperature=1.0, top_k=0, top_p=1.0, min_p=0.3, repeat_penalty=0.8, repeat_last_n=100),
]


@pytest.mark.parametrize("cfg", CONFIGS)
@pytest.mark.parametrize("seed", [1, 2**32 + 5])  # the generator takes the seed modulo 2^32
@pytest.mark.parametrize("vocab", [1000, 151936])
def test_sampler_tokens_equal_the_reference_sampler(oracle, cfg, seed, vocab):
    rng = np.random.default_rng(seed % 1000 + cfg["top_k"] + vocab)
    a = oracle_lib.OracleSampler(oracle, seed=seed, **cfg)
    b = ref.sampler(seed=seed, **cfg)
    recent = []
    for step in range(40 if vocab == 1000 else 6):
        logits = (rng.standard_normal(vocab) * 3).astype(np.float32)
        if step % 7 == 3:
            logits[rng.integers(0, vocab, 5)] = logits.max()  # equal logits at the top
        ta = a.sample(logits, recent)[0]
        tb = b.sample(logits, recent)
        assert ta == tb, (step, cfg, vocab)
        recent.append(ta)
        if step == 9:
            recent += [-1, vocab + 3]


@pytest.mark.parametrize("heads,L,D,keep,discard,count",
                         [(2, 1088, 128, 4, 256, 1088), (2, 64, 128, 0, 1, 64),
                          (3, 40, 16, 5, 10, 33), (1, 300, 256, 7, 3, 299),
                          (2, 128, 128, 16, 100, 120),
                          # refused by the reference: nothing may change
                          (2, 64, 32, 10, 0, 50), (2, 64, 32, 60, 5, 50), (2, 64, 32, 10, 45, 50)])
def test_discard_and_rope_adjust_equal_the_reference_bit_for_bit(oracle, heads, L, D, keep,
                                                                 discard, count):
    rng = np.random.default_rng(heads * 1000 + L + keep)
    tensors = [rng.standard_normal((heads, L, D)).astype(np.float32) for _ in range(4)]
    inv_freq = ref.inverse_rope_freqs(1e6, D)
    want = [t.copy() for t in tensors]
    ref.kv_discard(want, keep, discard, count)
    got = [oracle.kv_discard(t, keep, discard, count)[1] for t in tensors]
    for g, w in zip(got, want):
        np.testing.assert_array_equal(g.view(np.uint32), w.view(np.uint32))
    ref.kv_adjust_rope(want, keep, discard, count, inv_freq)
    for i, (g, w) in enumerate(zip(got, want)):
        if i % 2 == 0:  # keys: even tensors
            g = oracle.kv_adjust_rope(g, keep, discard, count, inv_freq)
        np.testing.assert_array_equal(g.view(np.uint32), w.view(np.uint32))


def test_discard_clamps_a_count_beyond_the_cache_like_the_reference(oracle):
    # discardKVCache clamps the token count to the cache length
    # (KVCacheManager.h:154); adjustKeyCacheRope does not and would run past the
    # tensor, so only the move is compared here
    rng = np.random.default_rng(3)
    t = rng.standard_normal((2, 64, 32)).astype(np.float32)
    want = [t.copy()]
    ref.kv_discard(want, 10, 20, 5000)
    rc, got = oracle.kv_discard(t, 10, 20, 5000)
    np.testing.assert_array_equal(got.view(np.uint32), want[0].view(np.uint32))
    assert not np.array_equal(got, t)
    # a negative prefix is refused by the move (and likewise not checked by the
    # reference's rotation): nothing changes
    want = [t.copy()]
    ref.kv_discard(want, -1, 5, 50)
    rc, got = oracle.kv_discard(t, -1, 5, 50)
    assert rc != 0
    np.testing.assert_array_equal(got, t)
    np.testing.assert_array_equal(want[0], t)


def test_inverse_frequencies_of_the_reference_are_the_models(oracle):
    # the decode graph carries inv_freq as a parameter computed by the importer
    # as 1 / theta^(2i/d) in f32; the runtime helper rebuilds it with powf
    f = ref.inverse_rope_freqs(1e6, 128)
    i = np.arange(64, dtype=np.float64)
    np.testing.assert_allclose(f, 1.0 / 1e6 ** (2 * i / 128), rtol=3e-7)
    assert f[0] == 1.0 and f.dtype == np.float32


@pytest.mark.parametrize("kind,ctype,dtype,rank", [
    (0, "c_float", np.float32, 1), (0, "c_float", np.float32, 2), (0, "c_float", np.float32, 3),
    (0, "c_float", np.float32, 4), (1, "c_int8", np.int8, 1), (1, "c_int8", np.int8, 2),
    (2, "c_longlong", np.int64, 1), (2, "c_longlong", np.int64, 2)])
def test_descriptor_structs_have_the_layout_of_the_reference_memref_object(kind, ctype, dtype,
                                                                           rank):
    """_mlir_ciface_* symbols are handed the address of a MemRef<T, N> object
    (frontend/Interfaces/buddy/Core/Container.h:126-137): read through this
    library's descriptor struct, the object of the reference's own class must
    show its pointers, offset, sizes and row-major strides."""
    import ctypes

    import buddy_mlir_amd as bma

    sizes = [3, 5, 2, 4][:rank]
    data = np.arange(int(np.prod(sizes)), dtype=dtype)
    n, raw = ref.memref_object(kind, data, sizes, offset=7)
    T = bma.memref_type(getattr(ctypes, ctype), rank)
    assert n == ctypes.sizeof(T) == 24 + 16 * rank
    d = T.from_buffer_copy(raw[:n].tobytes())
    alloc = ctypes.cast(d.allocated, ctypes.c_void_p).value
    align = ctypes.cast(d.aligned, ctypes.c_void_p).value
    assert alloc and alloc == align
    assert d.offset == 7
    assert list(d.sizes) == sizes
    strides = [int(np.prod(sizes[i + 1:])) for i in range(rank)]
    assert list(d.strides) == strides
