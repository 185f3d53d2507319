"""ctypes/numpy binding of oracle/liboracle.so (the CPU checker).

Test infrastructure: used by tests/, the smoke check and the benchmark's
cpu_baseline leg only.
"""
from __future__ import annotations

import ctypes
import subprocess
from ctypes import POINTER, Structure, c_float, c_int, c_int64, c_size_t, c_void_p
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
SO = ROOT / "oracle" / "liboracle.so"


def build():
    subprocess.run(["make", "-C", str(ROOT / "oracle"), "-s"], check=True)


def _p(a):
    return a.ctypes.data_as(c_void_p) if a is not None else None


class Shape(Structure):
    _fields_ = [(n, c_int64) for n in
                ("layers", "hidden", "heads", "kv_heads", "head_dim", "inter",
                 "vocab", "max_len")] + [("eps", c_float), ("attn_splits", c_int64)]


class Layer(Structure):
    _fields_ = [(n, c_void_p) for n in
                ("ln1", "ln2", "wq", "wk", "wv", "wo", "sq", "sk", "sv", "so",
                 "bq", "bk", "bv", "wg", "wu", "wd", "sg", "su", "sd",
                 "fq", "fk", "fv")]


class Model(Structure):
    _fields_ = [("shape", Shape), ("embed", c_void_p), ("inv_freq", c_void_p),
                ("layer", POINTER(Layer)), ("ln_f", c_void_p),
                ("w_lm", c_void_p), ("s_lm", c_void_p)]


class Oracle:
    def __init__(self, lib):
        self.lib = lib
        lib.oracle_argmax_first.restype = c_int64
        lib.oracle_decode_step.restype = c_int64
        lib.oracle_num_threads.restype = c_int

    # -- a1
    def quantize_w8(self, W):
        W = np.ascontiguousarray(W, dtype=np.float32)
        K, N = W.shape
        q = np.empty((K, N), np.int8)
        s = np.empty((N,), np.float32)
        self.lib.oracle_quantize_w8(_p(W), c_int64(K), c_int64(N), _p(q), _p(s))
        return q, s

    def quantize_w4(self, W):
        W = np.ascontiguousarray(W, dtype=np.float32)
        K, N = W.shape
        q = np.empty((K, N), np.int8)
        s = np.empty((N,), np.float32)
        self.lib.oracle_quantize_w4(_p(W), c_int64(K), c_int64(N), _p(q), _p(s))
        return q, s

    # -- a3
    def pack_panels(self, B, V=32):
        B = np.ascontiguousarray(B)
        K, N = B.shape
        out = np.empty_like(B)
        rc = self.lib.oracle_pack_panels(_p(B), c_int64(K), c_int64(N), c_int64(V),
                                         c_size_t(B.itemsize), _p(out))
        if rc:
            raise ValueError("N not divisible by V")
        return out

    def unpack_panels(self, P, V=32):
        P = np.ascontiguousarray(P)
        K, N = P.shape
        out = np.empty_like(P)
        rc = self.lib.oracle_unpack_panels(_p(P), c_int64(K), c_int64(N),
                                           c_int64(V), c_size_t(P.itemsize), _p(out))
        if rc:
            raise ValueError("N not divisible by V")
        return out

    # -- a4/a6
    def gemv_packed_f32(self, A, flatB, C, K, N, V=32, zero_init=False):
        A = np.ascontiguousarray(A, np.float32).reshape(-1)
        flatB = np.ascontiguousarray(flatB, np.float32).reshape(-1)
        C = np.array(C, np.float32).reshape(-1)
        self.lib.oracle_gemv_packed_f32(_p(A), _p(flatB), _p(C), c_int64(K),
                                        c_int64(N), c_int64(V), c_int(zero_init))
        return C

    def gemv_f32(self, A, B, C, V=32, zero_init=False):
        B = np.ascontiguousarray(B, np.float32)
        K, N = B.shape
        A = np.ascontiguousarray(A, np.float32).reshape(-1)
        C = np.array(C, np.float32).reshape(-1)
        self.lib.oracle_gemv_f32(_p(A), _p(B), _p(C), c_int64(K), c_int64(N),
                                 c_int64(V), c_int(zero_init))
        return C

    # -- a5
    def dequant_gemv(self, A, W, scale, C=None):
        W = np.ascontiguousarray(W, np.int8)
        K, N = W.shape
        A = np.ascontiguousarray(A, np.float32).reshape(-1)
        scale = np.ascontiguousarray(scale, np.float32).reshape(-1)
        C = np.zeros(N, np.float32) if C is None else np.array(C, np.float32).reshape(-1)
        assert A.size == K and scale.size == N and C.size == N
        self.lib.oracle_dequant_gemv_w8a32(_p(A), _p(W), _p(scale), _p(C),
                                           c_int64(K), c_int64(N))
        return C

    def dequant_gemv_panels(self, A, Wp, scale, K, N, C=None):
        Wp = np.ascontiguousarray(Wp, np.int8)
        A = np.ascontiguousarray(A, np.float32).reshape(-1)
        scale = np.ascontiguousarray(scale, np.float32).reshape(-1)
        C = np.zeros(N, np.float32) if C is None else np.array(C, np.float32).reshape(-1)
        self.lib.oracle_dequant_gemv_w8a32_panels(_p(A), _p(Wp), _p(scale), _p(C),
                                                  c_int64(K), c_int64(N))
        return C

    # -- a7
    def blis_gemm_f32(self, A, B, C):
        A = np.ascontiguousarray(A, np.float32)
        B = np.ascontiguousarray(B, np.float32)
        C = np.array(C, np.float32)
        M, K = A.shape
        N = B.shape[1]
        self.lib.oracle_blis_gemm_f32(_p(A), _p(B), _p(C), c_int64(M), c_int64(N),
                                      c_int64(K))
        return C

    def blis_gemm_w8a32(self, A, W, scale, C=None):
        A = np.ascontiguousarray(A, np.float32)
        W = np.ascontiguousarray(W, np.int8)
        scale = np.ascontiguousarray(scale, np.float32).reshape(-1)
        M, K = A.shape
        N = W.shape[1]
        C = np.zeros((M, N), np.float32) if C is None else np.array(C, np.float32)
        self.lib.oracle_blis_gemm_w8a32(_p(A), _p(W), _p(scale), _p(C), c_int64(M),
                                        c_int64(N), c_int64(K))
        return C

    # -- a8
    def gqa_decode_attention(self, q, kc, vc, mask, scale, num_splits=4):
        q = np.ascontiguousarray(q, np.float32)
        kc = np.ascontiguousarray(kc, np.float32)
        vc = np.ascontiguousarray(vc, np.float32)
        H, D = q.shape
        HKV, L, _ = kc.shape
        mask = None if mask is None else np.ascontiguousarray(mask, np.float32)
        out = np.empty((H, D), np.float32)
        lse = np.empty((H,), np.float32)
        self.lib.oracle_gqa_decode_attention(
            _p(q), _p(kc), _p(vc), _p(mask), _p(out), _p(lse), c_int64(H),
            c_int64(HKV), c_int64(L), c_int64(D), c_float(scale),
            c_int64(num_splits))
        return out, lse

    # -- a9
    def prefill_flash_attention(self, q, k, v, mask, scale):
        q = np.ascontiguousarray(q, np.float32)
        k = np.ascontiguousarray(k, np.float32)
        v = np.ascontiguousarray(v, np.float32)
        H, Lq, D = q.shape
        Lk = k.shape[1]
        mask = None if mask is None else np.ascontiguousarray(mask, np.float32)
        out = np.empty((H, Lq, D), np.float32)
        self.lib.oracle_prefill_flash_attention(
            _p(q), _p(k), _p(v), _p(mask), _p(out), c_int64(H), c_int64(Lq),
            c_int64(Lk), c_int64(D), c_float(scale))
        return out

    # -- a10
    def rmsnorm(self, x, w, eps=9.99999997e-7, inv_n=None):
        x = np.ascontiguousarray(x, np.float32).reshape(-1)
        w = np.ascontiguousarray(w, np.float32).reshape(-1)
        n = x.size
        inv_n = np.float32(1.0) / np.float32(n) if inv_n is None else inv_n
        y = np.empty(n, np.float32)
        self.lib.oracle_rmsnorm(_p(x), _p(w), _p(y), c_int64(n), c_float(inv_n),
                                c_float(eps))
        return y

    def rope_cos_sin(self, inv_freq, pos):
        inv_freq = np.ascontiguousarray(inv_freq, np.float32)
        half = inv_freq.size
        c = np.empty(2 * half, np.float32)
        s = np.empty(2 * half, np.float32)
        self.lib.oracle_rope_cos_sin(_p(inv_freq), c_int64(half), c_int64(pos),
                                     _p(c), _p(s))
        return c, s

    def rope_apply(self, x, cosv, sinv):
        x = np.array(x, np.float32)
        H, D = x.shape
        cosv = np.ascontiguousarray(cosv, np.float32)
        sinv = np.ascontiguousarray(sinv, np.float32)
        self.lib.oracle_rope_apply(_p(x), c_int64(H), c_int64(D), _p(cosv), _p(sinv))
        return x

    # -- W4A16 (f16 values are numpy.float16 arrays; bits go through uint16 views)
    def f32_to_f16(self, x):
        x = np.ascontiguousarray(x, np.float32).reshape(-1)
        y = np.empty(x.size, np.uint16)
        self.lib.oracle_f32_to_f16(_p(x), c_int64(x.size), _p(y))
        return y.view(np.float16)

    def pack_int4(self, q):
        q = np.ascontiguousarray(q, np.int8)
        out = np.empty(q.size // 2, np.int8)
        rc = self.lib.oracle_pack_int4(_p(q), c_int64(q.size), _p(out))
        assert rc == 0
        return out.reshape(q.shape[:-1] + (q.shape[-1] // 2,))

    def unpack_int4(self, packed):
        packed = np.ascontiguousarray(packed, np.int8)
        out = np.empty(packed.size * 2, np.int8)
        self.lib.oracle_unpack_int4(_p(packed), c_int64(out.size), _p(out))
        return out.reshape(packed.shape[:-1] + (packed.shape[-1] * 2,))

    def w4a16_gemv(self, a, packed, scale, c=None):
        """a [K] f16, packed [K, N/2] int8, scale [N] f16, c [N] f16 (or zeros)."""
        a = np.ascontiguousarray(a, np.float16).reshape(-1)
        packed = np.ascontiguousarray(packed, np.int8)
        K, N = packed.shape[0], packed.shape[1] * 2
        scale = np.ascontiguousarray(scale, np.float16).reshape(-1)
        out = np.zeros(N, np.float16) if c is None else np.array(c, np.float16).reshape(-1)
        self.lib.oracle_w4a16_gemv(_p(a.view(np.uint16)), _p(packed), _p(scale.view(np.uint16)),
                                   _p(out.view(np.uint16)), c_int64(K), c_int64(N))
        return out

    def kv_discard(self, cache, keep, discard, count):
        """discardKVCache on one [heads, max_len, dim] tensor; returns (rc, new)."""
        c = np.array(cache, np.float32)
        H, L, D = c.shape
        rc = self.lib.oracle_kv_discard(_p(c), c_int64(H), c_int64(L), c_int64(D),
                                        c_int64(keep), c_int64(discard), c_int64(count))
        return rc, c

    def kv_adjust_rope(self, kcache, keep, discard, count, inv_freq):
        c = np.array(kcache, np.float32)
        H, L, D = c.shape
        inv_freq = np.ascontiguousarray(inv_freq, np.float32)
        self.lib.oracle_kv_adjust_rope(_p(c), c_int64(H), c_int64(L), c_int64(D),
                                       c_int64(keep), c_int64(discard), c_int64(count),
                                       _p(inv_freq))
        return c

    def silu_mul(self, g, u):
        g = np.ascontiguousarray(g, np.float32).reshape(-1)
        u = np.ascontiguousarray(u, np.float32).reshape(-1)
        h = np.empty_like(g)
        self.lib.oracle_silu_mul(_p(g), _p(u), _p(h), c_int64(g.size))
        return h

    # -- a11
    def argmax_first(self, x):
        x = np.ascontiguousarray(x, np.float32).reshape(-1)
        return int(self.lib.oracle_argmax_first(_p(x), c_int64(x.size)))

    # -- a14
    def w8a8_quantize_activation(self, x):
        x = np.ascontiguousarray(x, np.float32)
        xq = np.empty(x.shape, np.int8)
        s = c_float()
        self.lib.oracle_w8a8_quantize_activation(_p(x), c_int64(x.size), _p(xq),
                                                 ctypes.byref(s))
        return xq, np.float32(s.value)

    def w8a8_matmul(self, A, W, wscale):
        A = np.ascontiguousarray(A, np.float32)
        W = np.ascontiguousarray(W, np.int8)
        wscale = np.ascontiguousarray(wscale, np.float32).reshape(-1)
        M, K = A.shape
        N = W.shape[1]
        C = np.empty((M, N), np.float32)
        acc = np.empty((M, N), np.int32)
        self.lib.oracle_w8a8_matmul(_p(A), _p(W), _p(wscale), _p(C), _p(acc),
                                    c_int64(M), c_int64(N), c_int64(K))
        return C, acc

    def num_threads(self):
        return int(self.lib.oracle_num_threads())


class OracleSampler:
    """The restated reference sampler (oracle/sampler.cpp)."""

    def __init__(self, oracle, temperature=0.0, top_k=0, top_p=1.0, min_p=0.0,
                 repeat_penalty=1.0, repeat_last_n=64, seed=1):
        lib = oracle.lib
        lib.oracle_sampler_create.restype = c_void_p
        lib.oracle_sampler_sample.restype = c_int
        self.lib = lib
        self.h = c_void_p(lib.oracle_sampler_create(
            c_float(temperature), c_int(top_k), c_float(top_p), c_float(min_p),
            c_float(repeat_penalty), c_int(repeat_last_n), ctypes.c_uint64(seed)))

    def sample(self, logits, recent=()):
        logits = np.ascontiguousarray(logits, np.float32)
        rec = np.ascontiguousarray(recent, np.int32)
        kept = c_int64(0)
        tok = self.lib.oracle_sampler_sample(self.h, _p(logits), c_int64(logits.size),
                                             _p(rec) if rec.size else None, c_int64(rec.size),
                                             ctypes.byref(kept))
        return int(tok), int(kept.value)

    def __del__(self):
        if getattr(self, "h", None):
            self.lib.oracle_sampler_destroy(self.h)
            self.h = None


class OracleModel:
    """Holds numpy weights and the ctypes structs that point at them."""

    def __init__(self, oracle: Oracle, shape: dict, embed, inv_freq, layers, ln_f,
                 w_lm, s_lm):
        self.o = oracle
        self.keep = [embed, inv_freq, ln_f, w_lm, s_lm, layers]
        self.shape = shape
        arr = (Layer * len(layers))()
        for i, L in enumerate(layers):
            for name, _ in Layer._fields_:
                a = L.get(name)
                setattr(arr[i], name, None if a is None else a.ctypes.data)
        self.arr = arr
        m = Model()
        for k, v in shape.items():
            setattr(m.shape, k, v)
        m.embed = embed.ctypes.data
        m.inv_freq = inv_freq.ctypes.data
        m.layer = arr
        m.ln_f = ln_f.ctypes.data
        m.w_lm = w_lm.ctypes.data
        m.s_lm = s_lm.ctypes.data
        self.m = m

    def decode_step(self, token, pos, kv):
        V = self.shape["vocab"]
        logits = np.empty(V, np.float32)
        ptrs = (c_void_p * len(kv))(*[a.ctypes.data for a in kv])
        tok = self.o.lib.oracle_decode_step(ctypes.byref(self.m), c_int64(token),
                                            c_int64(pos), ptrs, _p(logits))
        return int(tok), logits


def model_from_host(oracle: Oracle, shape, host) -> OracleModel:
    """OracleModel over the numpy copies made by
    buddy_mlir_amd.synthetic.build_session(keep_host=True)."""
    g = host["globals"]
    od = dict(layers=shape.layers, hidden=shape.hidden, heads=shape.heads,
              kv_heads=shape.kv_heads, head_dim=shape.head_dim, inter=shape.inter,
              vocab=shape.vocab, max_len=shape.max_len, eps=shape.rms_eps,
              attn_splits=4)
    return OracleModel(oracle, od, g["embed"], g["inv_freq"], host["layers"],
                       g["ln_f"], g["w_lm"], g["s_lm"])


_cached = None


def load() -> Oracle:
    global _cached
    if _cached is None:
        if not SO.exists():
            build()
        _cached = Oracle(ctypes.CDLL(str(SO)))
    return _cached


REF_SO = ROOT / "oracle" / "_ref" / "libref_llm.so"


class ReferenceRuntime:
    """The reference's own header-only sampler and KV-cache manager, as built by
    `make -C oracle ref` from the reference tree (oracle/ref_llm.cpp).  Only there
    where that build exists; the tests that use it skip otherwise."""

    def __init__(self):
        lib = ctypes.CDLL(str(REF_SO))
        lib.ref_sampler_create.restype = c_void_p
        lib.ref_sampler_sample.restype = c_int
        lib.ref_inverse_rope_freqs_count.restype = c_int
        self.lib = lib

    def sampler(self, temperature=0.0, top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=1.0,
                repeat_last_n=64, seed=1):
        lib = self.lib
        h = c_void_p(lib.ref_sampler_create(
            c_float(temperature), c_int(top_k), c_float(top_p), c_float(min_p),
            c_float(repeat_penalty), c_int(repeat_last_n), ctypes.c_uint64(seed)))

        class _S:
            def sample(_, logits, recent=()):
                lg = np.ascontiguousarray(logits, np.float32)
                rec = np.ascontiguousarray(recent, np.int32)
                return int(lib.ref_sampler_sample(h, _p(lg), c_int64(lg.size),
                                                  _p(rec) if rec.size else None,
                                                  c_int64(rec.size)))

            def __del__(_):
                lib.ref_sampler_destroy(h)

        return _S()

    def _ptrs(self, tensors):
        return (c_void_p * len(tensors))(*[t.ctypes.data for t in tensors])

    def kv_discard(self, tensors, keep, discard, count):
        """In place on a list of [heads, max_len, dim] f32 arrays."""
        H, L, D = tensors[0].shape
        self.lib.ref_kv_discard(self._ptrs(tensors), c_int(len(tensors)), c_int(H), c_int(L),
                                c_int(D), c_int(keep), c_int(discard), c_int(count))

    def kv_adjust_rope(self, tensors, keep, discard, count, inv_freq):
        H, L, D = tensors[0].shape
        f = np.ascontiguousarray(inv_freq, np.float32)
        self.lib.ref_kv_adjust_rope(self._ptrs(tensors), c_int(len(tensors)), c_int(H), c_int(L),
                                    c_int(D), c_int(keep), c_int(discard), c_int(count), _p(f))

    def memref_object(self, kind, data, sizes, offset=0):
        """Bytes of the reference's MemRef<T, N> object built over `data`
        (kind 0 = f32, 1 = int8, 2 = int64)."""
        sz = np.ascontiguousarray(sizes, np.int64)
        buf = np.zeros(256, np.uint8)
        n = self.lib.ref_memref_object(c_int(kind), c_int(sz.size), _p(data), _p(sz),
                                       c_int64(offset), _p(buf), c_int(buf.size))
        return n, buf

    def inverse_rope_freqs(self, theta, head_dim):
        n = self.lib.ref_inverse_rope_freqs_count(c_float(theta), c_int(head_dim))
        out = np.empty(n, np.float32)
        self.lib.ref_inverse_rope_freqs(c_float(theta), c_int(head_dim), _p(out))
        return out


def load_reference_runtime():
    return ReferenceRuntime() if REF_SO.exists() else None
