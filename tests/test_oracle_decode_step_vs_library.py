"""The oracle's whole decode step (embedding, RMSNorm, f32 q/k/v + bias, RoPE,
cache write, GQA attention, int8 o_proj / gate / up / down, residuals, final norm,
int8 lm_head) against an independent implementation of the architecture: the
logits that the pip `transformers` Qwen2 model computed for the same seeded
parameters (tests/golden/make_qwen2_decode_fixture.py wrote them; the test
itself needs numpy only).  A wrong op order, RoPE convention, head mapping,
residual or norm placement in the composition fails here."""
import sys
from pathlib import Path

import numpy as np

import oracle_lib
from parity import check_close

GOLDEN = Path(__file__).resolve().parent / "golden"
sys.path.insert(0, str(GOLDEN))
import qwen2_tiny as tiny  # noqa: E402


def oracle_model(oracle):
    c = tiny.CONFIG
    w = tiny.weights()
    layers = []
    for L in w["layers"]:
        d = {"ln1": L["ln1"], "ln2": L["ln2"],
             # f32 q/k/v as [K, N], the reference's shipped w8a32 build
             "fq": np.ascontiguousarray(L["q"].T), "fk": np.ascontiguousarray(L["k"].T),
             "fv": np.ascontiguousarray(L["v"].T), "bq": L["bq"], "bk": L["bk"], "bv": L["bv"]}
        for name, key in (("o", "o"), ("g", "gate"), ("u", "up"), ("d", "down")):
            q, s = oracle.quantize_w8(np.ascontiguousarray(L[key].T))
            q2, s2 = tiny.quantize_kn(L[key])  # the fixture's own numpy recipe
            np.testing.assert_array_equal(q, q2)
            np.testing.assert_array_equal(s, s2)
            d["w" + name], d["s" + name] = q, s
        layers.append(d)
    w_lm, s_lm = oracle.quantize_w8(np.ascontiguousarray(w["lm_head"].T))
    shape = dict(layers=c["layers"], hidden=c["hidden"], heads=c["heads"],
                 kv_heads=c["kv_heads"], head_dim=c["head_dim"], inter=c["inter"],
                 vocab=c["vocab"], max_len=c["max_len"], eps=c["rms_eps"], attn_splits=4)
    return oracle_lib.OracleModel(oracle, shape, w["embed"], tiny.inv_freq(), layers,
                                  w["ln_f"], w_lm, s_lm)


def test_decode_steps_match_the_library_model(oracle):
    fx = np.load(GOLDEN / "qwen2_decode_fixture.npz")
    assert fx["tokens"].tolist() == tiny.TOKENS and int(fx["seed"]) == tiny.SEED
    c = tiny.CONFIG
    om = oracle_model(oracle)
    kv = [np.zeros((c["kv_heads"], c["max_len"], c["head_dim"]), np.float32)
          for _ in range(2 * c["layers"])]
    for pos, tok in enumerate(tiny.TOKENS):
        nxt, logits = om.decode_step(tok, pos, kv)
        want = fx["logits"][pos]
        # two f32 implementations with different summation orders and the scale
        # applied before (library: dequantised weights) or after the sum (oracle)
        check_close(logits, want, normwise=1e-4)
        assert nxt == int(want.argmax())
