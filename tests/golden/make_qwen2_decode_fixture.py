"""Writes tests/golden/qwen2_decode_fixture.npz: the logits that the pip
`transformers` Qwen2 implementation (a library the importer of the reference
itself traces, frontend use at tools/buddy-codegen/import_model.py:163-195 --
not the reference's code) computes for a tiny random-init decoder, in f32 on
the CPU.  The model is built from an in-memory config (nothing is fetched); its
parameters are replaced by the seeded ones of qwen2_tiny.py, the matrices that
the reference's w8a32 build quantizes (o_proj, gate, up, down, lm_head) by
dequant(quant(W)).

    python tests/golden/make_qwen2_decode_fixture.py

The test that reads the fixture needs numpy only.
"""
import sys
from pathlib import Path

import numpy as np
import torch
from transformers import Qwen2Config, Qwen2ForCausalLM

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE))
import qwen2_tiny as tiny  # noqa: E402


def main():
    c = tiny.CONFIG
    cfg = Qwen2Config(vocab_size=c["vocab"], hidden_size=c["hidden"],
                      intermediate_size=c["inter"], num_hidden_layers=c["layers"],
                      num_attention_heads=c["heads"], num_key_value_heads=c["kv_heads"],
                      max_position_embeddings=c["max_len"], rms_norm_eps=c["rms_eps"],
                      rope_theta=c["rope_theta"], tie_word_embeddings=False,
                      attention_dropout=0.0, use_sliding_window=False)
    cfg._attn_implementation = "eager"
    model = Qwen2ForCausalLM(cfg).eval().float()
    w = tiny.weights()

    def deq(m):
        q, s = tiny.quantize_kn(m)
        return torch.from_numpy((q.astype(np.float32) * s).T.copy())

    sd = {"model.embed_tokens.weight": torch.from_numpy(w["embed"]),
          "model.norm.weight": torch.from_numpy(w["ln_f"]),
          "lm_head.weight": deq(w["lm_head"])}
    for i, L in enumerate(w["layers"]):
        p = f"model.layers.{i}."
        sd[p + "input_layernorm.weight"] = torch.from_numpy(L["ln1"])
        sd[p + "post_attention_layernorm.weight"] = torch.from_numpy(L["ln2"])
        for n in ("q", "k", "v"):  # f32 in the reference's w8a32 build
            sd[p + f"self_attn.{n}_proj.weight"] = torch.from_numpy(L[n])
            sd[p + f"self_attn.{n}_proj.bias"] = torch.from_numpy(L["b" + n])
        sd[p + "self_attn.o_proj.weight"] = deq(L["o"])
        sd[p + "mlp.gate_proj.weight"] = deq(L["gate"])
        sd[p + "mlp.up_proj.weight"] = deq(L["up"])
        sd[p + "mlp.down_proj.weight"] = deq(L["down"])
    missing, unexpected = model.load_state_dict(sd, strict=False)
    assert not unexpected and all("rotary" in k or "inv_freq" in k for k in missing), (missing, unexpected)
    ids = torch.tensor([tiny.TOKENS], dtype=torch.long)
    with torch.no_grad():
        logits = model(input_ids=ids, use_cache=False).logits[0].float().numpy()
    np.savez(HERE / "qwen2_decode_fixture.npz", logits=logits.astype(np.float32),
             tokens=np.asarray(tiny.TOKENS, np.int64), seed=np.int64(tiny.SEED))
    print("wrote", HERE / "qwen2_decode_fixture.npz", logits.shape, "argmax", logits.argmax(axis=1))


if __name__ == "__main__":
    main()
