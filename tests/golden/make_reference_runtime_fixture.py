"""Writes reference_runtime_fixture.npz: outputs of the reference's own
header-only runtime code (Sampler.h, KVCacheManager.h), as compiled into
oracle/_ref/libref_llm.so by `make -C oracle ref`, on seeded inputs that
tests/test_oracle_reference_fixture.py regenerates.  Run from the repository
root where the reference tree is present:

    make -C oracle ref && python tests/golden/make_reference_runtime_fixture.py

The fixture holds data only: token ids chosen by the reference sampler, cache
tensors after the reference's discard and key re-rotation, and its inverse
RoPE frequencies."""
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT / "tests"))
import oracle_lib  # noqa: E402

SAMPLER_CASES = [
    dict(temperature=0.0, top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=1.3, repeat_last_n=8),
    dict(temperature=0.8, top_k=40, top_p=0.95, min_p=0.05, repeat_penalty=1.1, repeat_last_n=64),
    dict(temperature=1.5, top_k=5, top_p=1.0, min_p=0.0, repeat_penalty=1.0, repeat_last_n=64),
    dict(temperature=0.7, top_k=0, top_p=0.9, min_p=0.0, repeat_penalty=1.0, repeat_last_n=64),
    dict(temperature=2.0, top_k=64, top_p=0.5, min_p=0.2, repeat_penalty=2.0, repeat_last_n=3),
]
SAMPLER_SEEDS = [1, 12345]
SAMPLER_VOCAB, SAMPLER_STEPS = 2000, 48
KV_CASES = [(2, 48, 16, 4, 12, 48), (3, 40, 8, 5, 10, 33), (1, 24, 32, 0, 1, 24),
            (2, 32, 8, 10, 0, 30), (2, 32, 8, 31, 5, 30)]


def sampler_logits(case_index, seed, step):
    rng = np.random.default_rng([case_index, seed, step])
    return (rng.standard_normal(SAMPLER_VOCAB) * 3).astype(np.float32)


def kv_input(case_index):
    heads, L, D = KV_CASES[case_index][:3]
    rng = np.random.default_rng(1000 + case_index)
    return [rng.standard_normal((heads, L, D)).astype(np.float32) for _ in range(2)]


def main():
    ref = oracle_lib.load_reference_runtime()
    if ref is None:
        raise SystemExit("oracle/_ref/libref_llm.so is missing: make -C oracle ref")
    out = {}
    for ci, cfg in enumerate(SAMPLER_CASES):
        for seed in SAMPLER_SEEDS:
            s = ref.sampler(seed=seed, **cfg)
            recent, toks = [], []
            for step in range(SAMPLER_STEPS):
                t = s.sample(sampler_logits(ci, seed, step), recent)
                toks.append(t)
                recent.append(t)
            out[f"sampler_{ci}_{seed}"] = np.array(toks, np.int32)
    for ci, (heads, L, D, keep, discard, count) in enumerate(KV_CASES):
        tensors = kv_input(ci)
        inv_freq = ref.inverse_rope_freqs(1e6, D)
        out[f"kv_{ci}_inv_freq"] = inv_freq
        ref.kv_discard(tensors, keep, discard, count)
        out[f"kv_{ci}_moved_k"], out[f"kv_{ci}_moved_v"] = tensors[0].copy(), tensors[1].copy()
        ref.kv_adjust_rope(tensors, keep, discard, count, inv_freq)
        out[f"kv_{ci}_rotated_k"] = tensors[0].copy()
        assert np.array_equal(tensors[1], out[f"kv_{ci}_moved_v"])  # values are not rotated
    for theta, D in [(1e6, 128), (1e4, 128), (1e4, 64)]:
        out[f"inv_freq_{int(theta)}_{D}"] = ref.inverse_rope_freqs(theta, D)
    path = Path(__file__).resolve().parent / "reference_runtime_fixture.npz"
    np.savez_compressed(path, **out)
    print("wrote", path, path.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
