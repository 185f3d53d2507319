"""A tiny Qwen2-shaped decoder with parameters drawn from numpy's seeded
generator in a fixed order, shared by the script that writes the golden logits
(with the pip `transformers` implementation) and by the test that feeds the same
parameters to the CPU oracle.  Orientation is Hugging Face's: weight [out, in]."""
import numpy as np

CONFIG = dict(vocab=512, hidden=256, inter=512, layers=2, heads=2, kv_heads=1, head_dim=128,
              max_len=64, rms_eps=1e-6, rope_theta=1e6)
SEED = 20240607
TOKENS = [3, 141, 59, 265, 358, 97, 93, 238, 46, 264, 338, 327]


def weights(seed: int = SEED):
    c = CONFIG
    rng = np.random.default_rng(seed)
    H, I, V = c["hidden"], c["inter"], c["vocab"]
    QN, KVN = c["heads"] * c["head_dim"], c["kv_heads"] * c["head_dim"]

    def mat(o, i, std=0.05):
        return (rng.standard_normal((o, i)) * std).astype(np.float32)

    def vec(n, mean=0.0, std=0.1):
        return (mean + rng.standard_normal(n) * std).astype(np.float32)

    w = {"embed": mat(V, H, 0.5), "layers": []}
    for _ in range(c["layers"]):
        w["layers"].append({
            "ln1": vec(H, 1.0), "q": mat(QN, H), "bq": vec(QN), "k": mat(KVN, H), "bk": vec(KVN),
            "v": mat(KVN, H), "bv": vec(KVN), "o": mat(H, QN), "ln2": vec(H, 1.0),
            "gate": mat(I, H), "up": mat(I, H), "down": mat(H, I)})
    w["ln_f"] = vec(H, 1.0)
    w["lm_head"] = mat(V, H)
    return w


def quantize_kn(w_out_in: np.ndarray):
    """The importer's recipe on the [K, N] orientation the kernels use
    (tools/buddy-codegen/import_model.py:837-848): per output channel
    scale = max(amax / 127, 1e-10), q = clip(rint(W / scale), -128, 127)."""
    W = np.ascontiguousarray(w_out_in.T)  # [K = in, N = out]
    scale = np.maximum(np.abs(W).max(axis=0) / np.float32(127.0), np.float32(1e-10)).astype(np.float32)
    q = np.clip(np.rint(W / scale), -128, 127).astype(np.int8)
    return q, scale


def inv_freq():
    d = CONFIG["head_dim"]
    return (1.0 / (np.float32(CONFIG["rope_theta"]) **
                   (np.arange(0, d, 2, dtype=np.int64).astype(np.float32) / np.float32(d)))).astype(np.float32)
