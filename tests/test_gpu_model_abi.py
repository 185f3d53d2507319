"""The reference's w8a32 package through the drop-in boundary: the blob layout
(f32 q/k/v with bias, int8 o/gate/up/down/lm_head) loaded into a session, and
the model-level `_mlir_ciface_forward_prefill` / `_mlir_ciface_forward_decode`
entry points called with the descriptors the generated ModelSession passes
(tools/buddy-codegen/gen_session.py:974-1007, 1345-1452)."""
import ctypes

import numpy as np
import pytest

import buddy_mlir_amd as bma
import oracle_lib
from buddy_mlir_amd.session import ModelShape, Shape
from parity import check_close

pytestmark = pytest.mark.gpu


def make_blobs(bh, shape: Shape, seed=0):
    """Random blobs in the documented order, plus the per-tensor views."""
    cs = shape.c()
    n_f32, n_i8 = ctypes.c_int64(), ctypes.c_int64()
    bh.buddy_hip_w8a32_blob_sizes(ctypes.byref(cs), ctypes.byref(n_f32), ctypes.byref(n_i8))
    rng = np.random.default_rng(seed)
    f32 = np.empty(n_f32.value, np.float32)
    i8 = rng.integers(-127, 128, n_i8.value, dtype=np.int8)
    H, D, I, V = shape.hidden, shape.head_dim, shape.inter, shape.vocab
    QN, KVN = shape.heads * D, shape.kv_heads * D
    off = [0]

    def take(n, kind):
        a = f32[off[0]:off[0] + n]
        if kind == "w":
            a[:] = rng.standard_normal(n, dtype=np.float32) * 0.02
        elif kind == "ln":
            a[:] = 1 + 0.1 * rng.standard_normal(n, dtype=np.float32)
        elif kind == "b":
            a[:] = 0.1 * rng.standard_normal(n, dtype=np.float32)
        elif kind == "s":  # scales of N(0,0.02) weights: ~ 4 sigma / 127
            a[:] = rng.uniform(5e-4, 8e-4, n).astype(np.float32)
        off[0] += n
        return a

    g = {"embed": take(V * H, "w").reshape(V, H)}
    inv = take(D // 2, None)
    inv[:] = (1.0 / (1e6 ** (np.arange(0, D, 2, dtype=np.float64) / D))).astype(np.float32)
    g["inv_freq"] = inv
    layers = [dict() for _ in range(shape.layers)]
    for L in layers:
        L["ln1"] = take(H, "ln")
        L["bq"] = take(QN, "b"); L["fq"] = take(H * QN, "w").reshape(H, QN)
        L["bk"] = take(KVN, "b"); L["fk"] = take(H * KVN, "w").reshape(H, KVN)
        L["bv"] = take(KVN, "b"); L["fv"] = take(H * KVN, "w").reshape(H, KVN)
        L["ln2"] = take(H, "ln")
    g["ln_f"] = take(H, "ln")
    for L in layers:
        L["so"], L["sg"], L["su"], L["sd"] = take(H, "s"), take(I, "s"), take(I, "s"), take(H, "s")
    g["s_lm"] = take(V, "s")
    assert off[0] == n_f32.value
    o = 0
    for L in layers:
        for name, (k, n) in (("wo", (QN, H)), ("wg", (H, I)), ("wu", (H, I)), ("wd", (I, H))):
            L[name] = i8[o:o + k * n].reshape(k, n)
            o += k * n
    g["w_lm"] = i8[o:o + H * V].reshape(H, V)
    assert o + H * V == n_i8.value
    return f32, i8, {"globals": g, "layers": layers}


SMALL = Shape(layers=2, hidden=256, heads=4, kv_heads=2, head_dim=128, inter=512,
              vocab=1024, max_len=64, rms_eps=1e-6)


def test_blob_sizes_match_reference_constants(bh):
    cs = Shape(max_len=1024).c()
    a, b = ctypes.c_int64(), ctypes.c_int64()
    bh.buddy_hip_w8a32_blob_sizes(ctypes.byref(cs), ctypes.byref(a), ctypes.byref(b))
    # examples/BuddyDeepSeekR1/buddy-deepseek-r1-w8a32-main.cpp:32-33
    assert (a.value, b.value) == (322338752, 1455489024)


def test_small_model_from_blobs_matches_oracle(bh, oracle):
    f32, i8, host = make_blobs(bh, SMALL, seed=1)
    cs = SMALL.c()
    h = bh.buddy_hip_session_create_from_w8a32_blobs(ctypes.byref(cs), f32.ctypes.data,
                                                     f32.size, i8.ctypes.data, i8.size)
    assert h, bh.buddy_hip_last_error()
    om = oracle_lib.model_from_host(oracle, SMALL, host)
    kv = [np.zeros((SMALL.kv_heads, SMALL.max_len, SMALL.head_dim), np.float32)
          for _ in range(2 * SMALL.layers)]
    tok = 3
    for pos in range(10):
        logits = np.empty(SMALL.vocab, np.float32)
        nxt = ctypes.c_int(-1)
        bma.check(bh.buddy_hip_session_decode(h, tok, pos, logits.ctypes.data, ctypes.byref(nxt)))
        otok, ologits = om.decode_step(tok, pos, kv)
        check_close(logits, ologits)
        assert nxt.value == otok
        tok = otok
    # a wrong-size blob is refused
    assert not bh.buddy_hip_session_create_from_w8a32_blobs(
        ctypes.byref(cs), f32.ctypes.data, f32.size - 1, i8.ctypes.data, i8.size)
    bh.buddy_hip_session_destroy(h)


class DecodeResult(ctypes.Structure):
    _fields_ = ([("pos_out", bma.MemRefI64_1D), ("kv0", bma.MemRefF32_4D),
                 ("kv1", bma.MemRefF32_4D)] +
                [(f"g{i}", type(f"G{i}", (ctypes.Structure,),
                                {"_fields_": [("dummy", bma.MemRefI64_1D),
                                              ("k", bma.MemRefF32_4D),
                                              ("v", bma.MemRefF32_4D)]}))
                 for i in range(27)] +
                [("logits", bma.MemRefF32_3D)])


class PrefillResult(ctypes.Structure):
    _fields_ = [("kv", bma.MemRefF32_4D * 56), ("logits", bma.MemRefF32_3D)]


@pytest.mark.timeout(900)
def test_model_level_entry_points_full_shape(bh, oracle):
    """28-layer Qwen2-1.5B-shaped package, cache length 64: forward_prefill on a
    20-token prompt padded to 64, then forward_decode for 3 tokens, against the
    oracle run token by token on the same blobs."""
    assert ctypes.sizeof(DecodeResult) == 40 + 2 * 88 + 27 * (40 + 2 * 88) + 72
    assert ctypes.sizeof(PrefillResult) == 56 * 88 + 72
    L = 64
    shape = Shape(max_len=L)
    f32, i8, host = make_blobs(bh, shape, seed=2)
    om = oracle_lib.model_from_host(oracle, shape, host)
    okv = [np.zeros((2, L, 128), np.float32) for _ in range(56)]
    rng = np.random.default_rng(9)
    prompt = rng.integers(0, shape.vocab, 20)
    tokens = np.zeros((1, L), np.int64)
    tokens[0, :20] = prompt
    ologits = []
    for pos in range(20):
        t, lg = om.decode_step(int(prompt[pos]), pos, okv)
        ologits.append(lg)
    free = ctypes.CDLL(None).free
    free.argtypes = [ctypes.c_void_p]

    mf = bma.MemRef(f32.ctypes.data, [f32.size])
    mi = bma.MemRef(i8.ctypes.data, [i8.size], ctype=ctypes.c_int8)
    mt = bma.MemRef(tokens.ctypes.data, [1, L], ctype=ctypes.c_longlong)
    pres = PrefillResult()
    bh._mlir_ciface_forward_prefill(ctypes.byref(pres), ctypes.byref(mf), ctypes.byref(mi),
                                    ctypes.byref(mt))
    assert pres.logits.aligned, bh.buddy_hip_last_error()
    assert list(pres.logits.sizes) == [1, L, shape.vocab]
    assert list(pres.kv[0].sizes) == [1, 2, L, 128]
    got = np.ctypeslib.as_array(pres.logits.aligned, shape=(L, shape.vocab))
    for pos in (0, 7, 19):
        check_close(got[pos], ologits[pos])
    assert int(got[19].argmax()) == int(ologits[19].argmax())
    # the caller copies KV into its own state tensors (gen_session.py:1352-1358)
    state_kv = [np.ctypeslib.as_array(pres.kv[j].aligned, shape=(2, L, 128)).copy()
                for j in range(56)]
    for j in (0, 1, 54, 55):
        check_close(state_kv[j][:, :20, :], okv[j][:, :20, :])
    for j in range(56):
        free(ctypes.cast(pres.kv[j].allocated, ctypes.c_void_p))
    free(ctypes.cast(pres.logits.allocated, ctypes.c_void_p))

    # decode: device cache continues from the prefill; oracle continues from its own
    kvm = [bma.MemRef(a.ctypes.data, [1, 2, L, 128]) for a in state_kv]
    posbuf = np.zeros(1, np.int64)
    tokbuf = np.zeros((1, 1), np.int64)
    dummies = [np.zeros(1, np.int64) for _ in range(27)]
    mpos = bma.MemRef(posbuf.ctypes.data, [1], ctype=ctypes.c_longlong)
    mtok = bma.MemRef(tokbuf.ctypes.data, [1, 1], ctype=ctypes.c_longlong)
    mdum = [bma.MemRef(d.ctypes.data, [1], ctype=ctypes.c_longlong) for d in dummies]
    tok = int(ologits[19].argmax())
    for step in range(3):
        pos = 20 + step
        tokbuf[0, 0], posbuf[0] = tok, pos
        for d in dummies:
            d[0] = pos
        res = DecodeResult()
        args = [ctypes.byref(res), ctypes.byref(mf), ctypes.byref(mi), ctypes.byref(mtok),
                ctypes.byref(mpos), ctypes.byref(kvm[0]), ctypes.byref(kvm[1])]
        for i in range(27):
            args += [ctypes.byref(mdum[i]), ctypes.byref(kvm[2 + 2 * i]),
                     ctypes.byref(kvm[3 + 2 * i])]
        assert len(args) == 88
        bh._mlir_ciface_forward_decode(*args)
        assert res.logits.aligned, bh.buddy_hip_last_error()
        assert list(res.logits.sizes) == [1, 1, shape.vocab]
        # state tensors alias the caller's buffers (so the caller frees nothing)
        assert ctypes.addressof(res.kv0.aligned.contents) == state_kv[0].ctypes.data
        assert ctypes.addressof(res.g26.v.aligned.contents) == state_kv[55].ctypes.data
        assert ctypes.addressof(res.pos_out.aligned.contents) == posbuf.ctypes.data
        lg = np.ctypeslib.as_array(res.logits.aligned, shape=(shape.vocab,)).copy()
        free(ctypes.cast(res.logits.allocated, ctypes.c_void_p))
        otok, olg = om.decode_step(tok, pos, okv)
        check_close(lg, olg)
        assert int(lg.argmax()) == otok
        tok = otok
    bh.buddy_hip_forward_reset()


def decode_args(res, mf, mi, mtok, mpos, kvm, mdum):
    args = [ctypes.byref(res), ctypes.byref(mf), ctypes.byref(mi), ctypes.byref(mtok),
            ctypes.byref(mpos), ctypes.byref(kvm[0]), ctypes.byref(kvm[1])]
    for i in range(27):
        args += [ctypes.byref(mdum[i]), ctypes.byref(kvm[2 + 2 * i]),
                 ctypes.byref(kvm[3 + 2 * i])]
    assert len(args) == 88
    return args


@pytest.mark.timeout(900)
def test_forward_decode_survives_the_callers_own_overflow_handling(bh, oracle):
    """The generated ModelSession handles a full cache on its HOST tensors
    (gen_session.py:1471-1511: discardKVCache, adjustKeyCacheRope, position
    lowered) and goes on calling forward_decode.  forward_decode writes every new
    row through to the caller's tensors and reloads the device cache when the
    position is not the one that follows, so such a caller needs no change: a
    64-row cache decoded from empty, overflowed, edited on the host with the
    restated KVCacheManager, and decoded on, yields the oracle's tokens."""
    L = 64
    shape = Shape(max_len=L)
    f32, i8, host = make_blobs(bh, shape, seed=2)
    om = oracle_lib.model_from_host(oracle, shape, host)
    okv = [np.zeros((2, L, 128), np.float32) for _ in range(56)]
    state_kv = [np.zeros((2, L, 128), np.float32) for _ in range(56)]
    free = ctypes.CDLL(None).free
    free.argtypes = [ctypes.c_void_p]
    mf = bma.MemRef(f32.ctypes.data, [f32.size])
    mi = bma.MemRef(i8.ctypes.data, [i8.size], ctype=ctypes.c_int8)
    kvm = [bma.MemRef(a.ctypes.data, [1, 2, L, 128]) for a in state_kv]
    posbuf = np.zeros(1, np.int64)
    tokbuf = np.zeros((1, 1), np.int64)
    dummies = [np.zeros(1, np.int64) for _ in range(27)]
    mpos = bma.MemRef(posbuf.ctypes.data, [1], ctype=ctypes.c_longlong)
    mtok = bma.MemRef(tokbuf.ctypes.data, [1, 1], ctype=ctypes.c_longlong)
    mdum = [bma.MemRef(d.ctypes.data, [1], ctype=ctypes.c_longlong) for d in dummies]
    inv_freq = host["globals"]["inv_freq"]
    keep = L // 4                       # TextGeneration.cpp:164
    discard = max(1, (L - keep) // 2)   # gen_session.py:1477-1479

    def step(tok, pos):
        tokbuf[0, 0], posbuf[0] = tok, pos
        for d in dummies:
            d[0] = pos
        res = DecodeResult()
        bh._mlir_ciface_forward_decode(*decode_args(res, mf, mi, mtok, mpos, kvm, mdum))
        assert res.logits.aligned, bh.buddy_hip_last_error()
        lg = np.ctypeslib.as_array(res.logits.aligned, shape=(shape.vocab,)).copy()
        free(ctypes.cast(res.logits.allocated, ctypes.c_void_p))
        return lg

    bh.buddy_hip_forward_reset()
    tok, pos, got, want = 11, 0, [], []
    for n in range(L + 12):
        if pos >= L:  # the caller edits ITS tensors; the oracle edits its own
            for kvset in (state_kv, okv):
                for j in range(56):
                    _, new = oracle.kv_discard(kvset[j], keep, discard, L)
                    if j % 2 == 0:
                        new = oracle.kv_adjust_rope(new, keep, discard, L, inv_freq)
                    kvset[j][...] = new
            pos = L - discard
        lg = step(tok, pos)
        otok, olg = om.decode_step(tok, pos, okv)
        if n in (0, L - 1, L, L + 11):
            check_close(lg, olg)
            # the row the step wrote is in the caller's tensors
            for j in (0, 1, 54, 55):
                check_close(state_kv[j][:, pos, :], okv[j][:, pos, :])
        got.append(int(lg.argmax()))
        want.append(otok)
        tok, pos = otok, pos + 1
    assert got == want
    bh.buddy_hip_forward_reset()


@pytest.mark.timeout(900)
def test_device_side_discard_keeps_the_device_cache_at_any_later_position(bh, oracle):
    """After buddy_hip_forward_discard_kv the caller's tensors are stale (never
    shifted), so no later decode may reload them, whatever its position: decode
    16 tokens, discard on the device, decode the position that follows, then
    decode that same position again with another token (a rewind).  Every step
    must give the oracle's logits on the oracle's own shifted cache."""
    L = 64
    shape = Shape(max_len=L)
    f32, i8, host = make_blobs(bh, shape, seed=4)
    om = oracle_lib.model_from_host(oracle, shape, host)
    okv = [np.zeros((2, L, 128), np.float32) for _ in range(56)]
    state_kv = [np.zeros((2, L, 128), np.float32) for _ in range(56)]
    free = ctypes.CDLL(None).free
    free.argtypes = [ctypes.c_void_p]
    mf = bma.MemRef(f32.ctypes.data, [f32.size])
    mi = bma.MemRef(i8.ctypes.data, [i8.size], ctype=ctypes.c_int8)
    kvm = [bma.MemRef(a.ctypes.data, [1, 2, L, 128]) for a in state_kv]
    posbuf = np.zeros(1, np.int64)
    tokbuf = np.zeros((1, 1), np.int64)
    dummies = [np.zeros(1, np.int64) for _ in range(27)]
    mpos = bma.MemRef(posbuf.ctypes.data, [1], ctype=ctypes.c_longlong)
    mtok = bma.MemRef(tokbuf.ctypes.data, [1, 1], ctype=ctypes.c_longlong)
    mdum = [bma.MemRef(d.ctypes.data, [1], ctype=ctypes.c_longlong) for d in dummies]
    inv_freq = host["globals"]["inv_freq"]

    def step(tok, pos):
        tokbuf[0, 0], posbuf[0] = tok, pos
        for d in dummies:
            d[0] = pos
        res = DecodeResult()
        bh._mlir_ciface_forward_decode(*decode_args(res, mf, mi, mtok, mpos, kvm, mdum))
        assert res.logits.aligned, bh.buddy_hip_last_error()
        lg = np.ctypeslib.as_array(res.logits.aligned, shape=(shape.vocab,)).copy()
        free(ctypes.cast(res.logits.allocated, ctypes.c_void_p))
        return lg

    bh.buddy_hip_forward_reset()
    tok = 5
    for pos in range(16):
        lg = step(tok, pos)
        otok, _ = om.decode_step(tok, pos, okv)
        assert int(lg.argmax()) == otok
        tok = otok
    keep, discard, count = 4, 4, 16
    assert bh.buddy_hip_forward_discard_kv(keep, discard, count) == 0, bh.buddy_hip_last_error()
    for j in range(56):
        _, new = oracle.kv_discard(okv[j], keep, discard, count)
        if j % 2 == 0:
            new = oracle.kv_adjust_rope(new, keep, discard, count, inv_freq)
        okv[j][...] = new
    pos = count - discard
    lg = step(tok, pos)                      # the position that follows
    otok, olg = om.decode_step(tok, pos, okv)
    check_close(lg, olg)
    assert int(lg.argmax()) == otok
    other = (tok + 17) % shape.vocab
    lg = step(other, pos)                    # the same position again: a rewind
    otok, olg = om.decode_step(other, pos, okv)
    check_close(lg, olg)
    assert int(lg.argmax()) == otok
    lg = step(otok, 3)                       # and far back, inside the kept prefix
    otok2, olg = om.decode_step(otok, 3, okv)
    check_close(lg, olg)
    assert int(lg.argmax()) == otok2
    # invalidate_kv hands the truth back to the caller's (stale, unshifted) tensors
    bh.buddy_hip_forward_invalidate_kv()
    stale = [a.copy() for a in state_kv]
    lg = step(tok, pos)
    otok3, olg = om.decode_step(tok, pos, stale)
    check_close(lg, olg)
    bh.buddy_hip_forward_reset()


def test_model_level_entry_points_refuse_bad_blobs(bh):
    f32 = np.zeros(10, np.float32)
    i8 = np.zeros(10, np.int8)
    tokens = np.zeros((1, 64), np.int64)
    pres = PrefillResult()
    bh._mlir_ciface_forward_prefill(
        ctypes.byref(pres), ctypes.byref(bma.MemRef(f32.ctypes.data, [10])),
        ctypes.byref(bma.MemRef(i8.ctypes.data, [10], ctype=ctypes.c_int8)),
        ctypes.byref(bma.MemRef(tokens.ctypes.data, [1, 64], ctype=ctypes.c_longlong)))
    assert not pres.logits.aligned
    assert b"blobs hold" in bh.buddy_hip_last_error()
