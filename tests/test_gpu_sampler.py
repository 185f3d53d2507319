"""The device-assisted sampler against the CPU restatement of the reference's
buddy::runtime::Sampler (runtime/include/buddy/runtime/llm/Sampler.h:62-206).

Token ids are compared exactly: both sides seed std::mt19937 with the same
value, the device side hands back the top-K (value, id) pairs bit for bit
(penalty by IEEE division/multiplication, temperature by one f32 multiply), and
the host finish is the same standard-library arithmetic.  The synthetic logits
are continuous random values, so no two of the leading candidates are equal
(the reference leaves the order of equal logits to std::sort)."""
import numpy as np
import pytest
import torch

from buddy_mlir_amd import synthetic
from buddy_mlir_amd.session import Sampler, Shape

import oracle_lib

pytestmark = pytest.mark.gpu

CONFIGS = [
    dict(temperature=0.0, top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=1.0, repeat_last_n=64),
    dict(temperature=0.0, top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=1.3, repeat_last_n=8),
    dict(temperature=0.8, top_k=40, top_p=0.95, min_p=0.05, repeat_penalty=1.1, repeat_last_n=64),
    dict(temperature=1.5, top_k=5, top_p=1.0, min_p=0.0, repeat_penalty=1.0, repeat_last_n=64),
    dict(temperature=1.0, top_k=1, top_p=1.0, min_p=0.0, repeat_penalty=1.0, repeat_last_n=64),
    dict(temperature=2.0, top_k=64, top_p=0.5, min_p=0.2, repeat_penalty=2.0, repeat_last_n=3),
    dict(temperature=1.2, top_k=128, top_p=0.99, min_p=0.0, repeat_penalty=1.05,
         repeat_last_n=1000),
    # no top-K limit, and one beyond the device selection: the host path
    dict(temperature=0.7, top_k=0, top_p=0.9, min_p=0.0, repeat_penalty=1.2, repeat_last_n=64),
    dict(temperature=0.9, top_k=500, top_p=0.97, min_p=0.0, repeat_penalty=1.0, repeat_last_n=64),
]


@pytest.mark.parametrize("cfg", CONFIGS)
@pytest.mark.parametrize("vocab", [151936, 5000, 4096, 37])
def test_sampled_tokens_equal_the_oracle(bh, oracle, cfg, vocab):
    if cfg["top_k"] > vocab:
        cfg = dict(cfg, top_k=vocab)
    seed = 1000 + vocab % 97 + cfg["top_k"]
    want = oracle_lib.OracleSampler(oracle, seed=seed, **cfg)
    got = Sampler(seed=seed, **cfg)
    g = torch.Generator(device="cuda").manual_seed(seed)
    recent = []
    for step in range(24):
        logits = torch.randn(vocab, device="cuda", generator=g) * 3
        if step % 5 == 4:  # a peaked distribution: min-P / top-P cut to one candidate
            logits[(step * 7919) % vocab] += 40.0
        torch.cuda.synchronize()
        tok = got.sample(logits, recent)
        ref, _ = want.sample(logits.cpu().numpy(), recent)
        assert tok == ref, (step, cfg, vocab)
        recent.append(tok)
        if step == 10:
            recent += [-3, vocab + 5]  # ids outside the vocabulary are skipped
    got.close()


def test_penalty_window_counts_each_occurrence(bh, oracle):
    logits = torch.zeros(9000, device="cuda")
    logits[[3, 8191, 8500]] = torch.tensor([5.0, 5.0, 4.9], device="cuda")
    recent = [3, 8191, 8191, 3, 3]
    for n_last, expect in [(2, 8191), (3, 8500), (64, 8500), (1, 8191)]:
        cfg = dict(temperature=0.0, repeat_penalty=1.5, repeat_last_n=n_last)
        tok = Sampler(**cfg).sample(logits, recent)
        assert tok == oracle_lib.OracleSampler(oracle, **cfg).sample(logits.cpu().numpy(),
                                                                      recent)[0]
        assert tok == expect
    # negative logits are multiplied by the penalty
    neg = torch.full((300,), -1.0, device="cuda")
    neg[250] = -1.2
    rec = [i for i in range(300) if i != 250]
    assert Sampler(temperature=0.0, repeat_penalty=2.0, repeat_last_n=512).sample(neg, rec) == 250


def test_equal_logits_rank_by_id(bh):
    logits = torch.ones(10000, device="cuda")
    assert Sampler(temperature=0.0, repeat_penalty=1.1).sample(logits, [0, 1]) == 2
    s = Sampler(temperature=1.0, top_k=4, seed=5)
    seen = {s.sample(logits) for _ in range(200)}
    assert seen == {0, 1, 2, 3}


def test_bad_configurations_are_refused(bh):
    from buddy_mlir_amd import BuddyHipError
    for bad in [dict(temperature=-1.0), dict(top_k=-1), dict(repeat_penalty=0.0),
                dict(repeat_last_n=-2)]:
        with pytest.raises(BuddyHipError):
            Sampler(**bad)


def test_decode_step_with_sampling(bh, oracle):
    shape = Shape(layers=2, hidden=256, heads=2, kv_heads=1, head_dim=128, inter=512,
                  vocab=3000, max_len=64)
    a, _ = synthetic.build_session(shape, context=0, ln_jitter=0.1)
    b, _ = synthetic.build_session(shape, context=0, ln_jitter=0.1)  # same seeded weights
    cfg = dict(temperature=0.9, top_k=50, top_p=0.95, min_p=0.02, repeat_penalty=1.1,
               repeat_last_n=16)
    sampler = Sampler(seed=99, **cfg)
    want = oracle_lib.OracleSampler(oracle, seed=99, **cfg)
    tok_a = tok_b = 17
    recent = []
    for pos in range(12):
        nxt = a.decode_sample(sampler, tok_a, pos, recent)
        _, logits = b.decode(tok_b, pos)
        ref, _ = want.sample(logits, recent)
        assert nxt == ref, pos
        recent.append(nxt)
        tok_a = tok_b = nxt
