"""Two sessions driven from two host threads at the same time (each on its own
stream) give what they give one after the other: the library's process-wide
state (staging buffers and workspaces keyed by stream, one-time kernel
attributes, the error string) must not couple them."""
import threading

import numpy as np
import pytest

from buddy_mlir_amd import synthetic
from buddy_mlir_amd.session import Sampler

from test_gpu_decode import SMALL

pytestmark = pytest.mark.gpu


def generate(sess, prompt, steps, sampler=None):
    nxt, _ = sess.prefill(prompt, 0)
    out = [nxt]
    if sampler is None:
        out += sess.decode_greedy(nxt, len(prompt), steps).tolist()
    else:
        for i in range(steps):
            out.append(sess.decode_sample(sampler, out[-1], len(prompt) + i, out))
    return out


def test_two_sessions_in_two_threads():
    a, _ = synthetic.build_session(SMALL, context=0, ln_jitter=0.1)
    b, _ = synthetic.build_session(SMALL, context=0, ln_jitter=0.1)
    pa = synthetic.first_tokens(SMALL, 70, seed=1).tolist()  # 70 rows: the wide matmul kernels
    pb = synthetic.first_tokens(SMALL, 23, seed=2).tolist()
    cfg = dict(temperature=0.8, top_k=30, top_p=0.95, repeat_penalty=1.1, seed=5)
    want_a = generate(a, pa, 40)
    want_b = generate(b, pb, 40, Sampler(**cfg))
    for round_ in range(3):
        got = {}
        errors = []

        def run(name, sess, prompt, sampler):
            try:
                got[name] = generate(sess, prompt, 40, sampler)
            except Exception as e:  # noqa: BLE001
                errors.append(e)

        ta = threading.Thread(target=run, args=("a", a, pa, None))
        tb = threading.Thread(target=run, args=("b", b, pb, Sampler(**cfg)))
        ta.start()
        tb.start()
        ta.join(60)
        tb.join(60)
        assert not errors, errors
        assert got["a"] == want_a and got["b"] == want_b, round_
    a.close()
    b.close()
