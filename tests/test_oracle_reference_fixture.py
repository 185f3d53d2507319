"""The restated sampler and KV-cache functions against outputs of the
reference's own code kept as a fixture: tests/golden/reference_runtime_fixture.npz
was written by tests/golden/make_reference_runtime_fixture.py from
runtime/include/buddy/runtime/llm/Sampler.h and KVCacheManager.h compiled as
oracle/_ref/libref_llm.so.  Unlike tests/test_oracle_vs_reference_build.py this
needs neither the reference tree nor that library."""
import sys
from pathlib import Path

import numpy as np
import pytest

import oracle_lib

sys.path.insert(0, str(Path(__file__).resolve().parent / "golden"))
import make_reference_runtime_fixture as fx  # noqa: E402  (the seeded inputs)

FIXTURE = np.load(Path(__file__).resolve().parent / "golden" / "reference_runtime_fixture.npz")


@pytest.mark.parametrize("ci", range(len(fx.SAMPLER_CASES)))
@pytest.mark.parametrize("seed", fx.SAMPLER_SEEDS)
def test_sampler_reproduces_the_reference_tokens(oracle, ci, seed):
    s = oracle_lib.OracleSampler(oracle, seed=seed, **fx.SAMPLER_CASES[ci])
    want = FIXTURE[f"sampler_{ci}_{seed}"]
    recent = []
    for step in range(fx.SAMPLER_STEPS):
        t = s.sample(fx.sampler_logits(ci, seed, step), recent)[0]
        assert t == want[step], (ci, seed, step)
        recent.append(t)
    assert len(set(want.tolist())) > 3


@pytest.mark.parametrize("ci", range(len(fx.KV_CASES)))
def test_discard_and_rotation_reproduce_the_reference_bits(oracle, ci):
    heads, L, D, keep, discard, count = fx.KV_CASES[ci]
    k, v = fx.kv_input(ci)
    inv_freq = FIXTURE[f"kv_{ci}_inv_freq"]  # kvcache::buildInverseRopeFreqs(1e6, D)
    _, mk = oracle.kv_discard(k, keep, discard, count)
    _, mv = oracle.kv_discard(v, keep, discard, count)
    np.testing.assert_array_equal(mk.view(np.uint32), FIXTURE[f"kv_{ci}_moved_k"].view(np.uint32))
    np.testing.assert_array_equal(mv.view(np.uint32), FIXTURE[f"kv_{ci}_moved_v"].view(np.uint32))
    rk = oracle.kv_adjust_rope(mk, keep, discard, count, inv_freq)
    np.testing.assert_array_equal(rk.view(np.uint32),
                                  FIXTURE[f"kv_{ci}_rotated_k"].view(np.uint32))


def test_inverse_frequencies():
    for theta, D in [(1e6, 128), (1e4, 128), (1e4, 64)]:
        f = FIXTURE[f"inv_freq_{int(theta)}_{D}"]
        i = np.arange(D // 2, dtype=np.float64)
        np.testing.assert_allclose(f, 1.0 / theta ** (2 * i / D), rtol=3e-7)
        assert f.dtype == np.float32 and f[0] == 1.0
