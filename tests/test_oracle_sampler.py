"""Pins the oracle's restatement of the reference sampler
(runtime/include/buddy/runtime/llm/Sampler.h:62-206) against an independent
numpy re-derivation of the whole pipeline, including the draw: std::mt19937's
output sequence (numpy's MT19937 with the classic init_genrand seeding), the 53-bit
canonical double libstdc++ builds from two 32-bit outputs, and
std::discrete_distribution's normalise / partial-sum / lower_bound."""
import numpy as np
import pytest

import oracle_lib


class NumpySampler:
    def __init__(self, temperature, top_k, top_p, min_p, repeat_penalty, repeat_last_n, seed):
        self.t, self.k, self.p, self.minp = np.float32(temperature), top_k, np.float32(top_p), np.float32(min_p)
        self.rp, self.n = np.float32(repeat_penalty), repeat_last_n
        bg = np.random.MT19937()
        bg._legacy_seeding(seed)  # init_genrand(seed), what std::mt19937(seed) does
        self.bg = bg

    def canonical(self):
        r1, r2 = (int(v) for v in self.bg.random_raw(2))
        u = (float(r1) + float(r2) * 4294967296.0) / 18446744073709551616.0
        return np.nextafter(1.0, 0.0) if u >= 1.0 else u

    def sample(self, logits, recent=()):
        w = np.array(logits, np.float32)
        pen = self.rp != 1 and len(recent) > 0
        if self.t == 0 and not pen:
            return int(np.argmax(w)), 0
        if pen:
            for t in list(recent)[max(0, len(recent) - self.n):]:
                if 0 <= t < w.size:
                    w[t] = w[t] / self.rp if w[t] > 0 else w[t] * self.rp
        if self.t == 0:
            return int(np.argmax(w)), 0
        w = w * (np.float32(1.0) / self.t)
        order = np.argsort(-w, kind="stable")
        limit = self.k if 0 < self.k < w.size else w.size
        vals = w[order[:limit]]
        probs = np.exp(vals - vals[0]).astype(np.float32)
        s = np.float32(0)
        for v in probs:  # f32 running sum, in order
            s = np.float32(s + v)
        probs = (probs / s).astype(np.float32)
        if self.minp > 0:
            below = np.nonzero(probs < np.float32(self.minp * probs[0]))[0]
            if below.size and below[0] > 0:
                limit = int(below[0])
        if self.p < 1:
            cum, nl = np.float32(0), limit
            for i in range(limit):
                cum = np.float32(cum + probs[i])
                if cum >= self.p:
                    nl = i + 1
                    break
            limit = nl
        fs = np.float32(0)
        for v in probs[:limit]:
            fs = np.float32(fs + v)
        probs = (probs[:limit] / fs).astype(np.float32)
        if limit < 2:
            return int(order[0]), limit  # std::discrete_distribution draws nothing
        pd = probs.astype(np.float64)
        total = 0.0
        for v in pd:
            total += v
        cp = np.cumsum(pd / total)
        cp[-1] = 1.0
        return int(order[int(np.searchsorted(cp, self.canonical(), side="left"))]), limit


CONFIGS = [
    dict(temperature=0.0, top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=1.0, repeat_last_n=64),
    dict(temperature=0.0, top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=1.3, repeat_last_n=8),
    dict(temperature=0.8, top_k=40, top_p=0.95, min_p=0.05, repeat_penalty=1.1, repeat_last_n=64),
    dict(temperature=1.5, top_k=5, top_p=1.0, min_p=0.0, repeat_penalty=1.0, repeat_last_n=64),
    dict(temperature=0.7, top_k=0, top_p=0.9, min_p=0.0, repeat_penalty=1.0, repeat_last_n=64),
    dict(temperature=1.0, top_k=1, top_p=1.0, min_p=0.0, repeat_penalty=1.0, repeat_last_n=64),
    dict(temperature=2.0, top_k=64, top_p=0.5, min_p=0.2, repeat_penalty=2.0, repeat_last_n=3),
]


@pytest.mark.parametrize("cfg", CONFIGS)
@pytest.mark.parametrize("seed", [1, 12345])
def test_oracle_sampler_equals_numpy_rederivation(oracle, cfg, seed):
    rng = np.random.default_rng(seed + cfg["top_k"])
    a = oracle_lib.OracleSampler(oracle, seed=seed, **cfg)
    b = NumpySampler(seed=seed, **cfg)
    recent = []
    for step in range(40):
        logits = (rng.standard_normal(1000) * 3).astype(np.float32)
        ta, ka = a.sample(logits, recent)
        tb, kb = b.sample(logits, recent)
        assert (ta, ka) == (tb, kb), (step, cfg)
        recent.append(ta)


def test_greedy_is_the_first_maximum_and_penalty_counts_occurrences(oracle):
    logits = np.zeros(16, np.float32)
    logits[[3, 9]] = 5.0
    s = oracle_lib.OracleSampler(oracle, temperature=0.0)
    assert s.sample(logits)[0] == 3
    # token 3 appears twice in the window: 5 / 1.5 / 1.5 < 5 / 1.5 (token 9, once)
    s = oracle_lib.OracleSampler(oracle, temperature=0.0, repeat_penalty=1.5, repeat_last_n=3)
    w = logits.copy()
    for t in [3, 3, 9]:
        w[t] /= np.float32(1.5)
    assert s.sample(logits, [9, 9, 3, 3, 9])[0] == int(np.argmax(w)) == 9
    # negative logits are multiplied, tokens outside the vocabulary are skipped
    neg = np.full(8, -1.0, np.float32)
    neg[2] = -1.2
    s = oracle_lib.OracleSampler(oracle, temperature=0.0, repeat_penalty=2.0)
    assert s.sample(neg, [0, 1, 3, 4, 5, 6, 7, 99, -5])[0] == 2


def test_sampling_frequencies_follow_the_filtered_softmax(oracle):
    logits = np.array([2.0, 1.0, 0.5, 0.0, -1.0, -3.0], np.float32)
    s = oracle_lib.OracleSampler(oracle, temperature=1.0, top_k=4, seed=7)
    n = 20000
    counts = np.bincount([s.sample(logits)[0] for _ in range(n)], minlength=6)
    p = np.exp(logits[:4] - logits[0])
    p /= p.sum()
    assert counts[4:].sum() == 0
    assert np.abs(counts[:4] / n - p).max() < 0.012
