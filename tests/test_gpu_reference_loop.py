"""The reference's own generation loop over the GPU session.

oracle/_ref/ref_generation is the reference's runtime/llm/TextGeneration.cpp
(runGeneration), its tokenizer (TextContainer.h), its sampler and its KV-cache
helper, compiled from the reference tree where that is present, linked with
libbuddy_hip through buddy_hip::HipLLMSession (include/buddy_hip/llm_session.h),
the implementation of the reference's LLMSession interface over this library.
The test runs it on parameter files on disk and checks every generated token
against the CPU restatement driven the way the loop drives a session: prefill,
the first token from the last prompt row, one decode step per token, and when
the cache is full the discard + key re-rotation of handleKVCacheOverflow with
the loop's own hard-wired theta of 10000 (TextGeneration.cpp:164,231-237).
Skipped where the harness has not been built."""
import json
import subprocess
from pathlib import Path

import numpy as np
import pytest

import oracle_lib
from buddy_mlir_amd.session import Shape

pytestmark = pytest.mark.gpu

REF_DIR = Path(__file__).resolve().parent.parent / "oracle" / "_ref"
HARNESS = REF_DIR / "ref_generation"
EXAMPLE_MAIN = REF_DIR / "ref_w8a32_main"
PROMPT = "hello world abc"
# <bos> <bos> <user> hello Ġworld Ġ a b c <assistant> <think> \n (TextContainer.h:443-525)
PROMPT_IDS = [151646, 151646, 151644, 400, 401, 326, 300, 301, 302, 151645, 151648, 198]
SHAPE = Shape(layers=2, hidden=256, heads=2, kv_heads=1, head_dim=128, inter=512,
              vocab=151936, max_len=64)  # the tokenizer's special ids need the real vocabulary


def write_vocab(path):
    toks = [f"<{i}>" for i in range(SHAPE.vocab)]
    for j, ch in enumerate("abcdefghijklmnopqrstuvwxyz"):
        toks[300 + j] = ch
    toks[326] = "Ġ"          # the tokenizer's stand-in for a space
    toks[400], toks[401] = "hello", "Ġworld"
    path.write_text("\n".join(toks) + "\n", encoding="utf-8")


def run_harness(tmp_path, *extra):
    r = subprocess.run([str(HARNESS), "--f32", str(tmp_path / "f32.data"),
                        "--i8", str(tmp_path / "i8.data"), "--vocab", str(tmp_path / "vocab.txt"),
                        "--prompt", PROMPT, "--max-len", str(SHAPE.max_len),
                        "--layers", str(SHAPE.layers), "--hidden", str(SHAPE.hidden),
                        "--heads", str(SHAPE.heads), "--kv-heads", str(SHAPE.kv_heads),
                        "--inter", str(SHAPE.inter), "--vocab-size", str(SHAPE.vocab), *extra],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    lines = r.stdout.splitlines()
    ids_in = [int(t) for t in lines[0].split("]")[1].split()]
    events = [json.loads(l) for l in lines if l.startswith('{"event":"token"')]
    final_pos = int([l for l in lines if l.startswith("[generated]")][0].split()[-1])
    return ids_in, [e["token_id"] for e in events], final_pos


def expected(oracle, host, ids_in, sampler, total_tokens):
    """The loop of TextGeneration.cpp:157-277 over the CPU restatement."""
    om = oracle_lib.model_from_host(oracle, SHAPE, host)
    L = SHAPE.max_len
    kv = [np.zeros((SHAPE.kv_heads, L, SHAPE.head_dim), np.float32)
          for _ in range(2 * SHAPE.layers)]
    for pos, t in enumerate(ids_in):
        _, logits = om.decode_step(t, pos, kv)
    pos = len(ids_in)
    recent = []
    out = [sampler.sample(logits, recent)[0]]
    recent.append(out[0])
    i = np.arange(SHAPE.head_dim // 2, dtype=np.float32)
    inv_freq = (np.float32(1.0) / np.power(np.float32(10000.0),
                                          (np.float32(2.0) * i) / np.float32(SHAPE.head_dim))
                ).astype(np.float32)
    for _ in range(total_tokens - len(ids_in)):
        if out[-1] == 151643:
            break
        if pos >= L:  # handleKVCacheOverflow(keep = L / 4, theta = 10000)
            keep = min(max(L // 4, 0), L - 1)
            discard = max(1, (L - keep) // 2)
            for j in range(len(kv)):
                _, kv[j] = oracle.kv_discard(kv[j], keep, discard, L)
                if j % 2 == 0:
                    kv[j] = oracle.kv_adjust_rope(kv[j], keep, discard, L, inv_freq)
            pos = L - discard
        _, logits = om.decode_step(out[-1], pos, kv)
        pos += 1
        out.append(sampler.sample(logits, recent)[0])
        recent.append(out[-1])
    return out, pos


@pytest.mark.skipif(not HARNESS.exists(), reason="oracle/_ref/ref_generation not built "
                    "(needs the reference tree: make -C oracle ref)")
def test_reference_generation_loop_over_the_gpu_session(tmp_path, bh, oracle):
    from test_gpu_model_abi import make_blobs

    f32, i8, host = make_blobs(bh, SHAPE, seed=9)
    (tmp_path / "f32.data").write_bytes(f32.tobytes())
    (tmp_path / "i8.data").write_bytes(i8.tobytes())
    write_vocab(tmp_path / "vocab.txt")

    # greedy, no cache overflow
    ids_in, got, final_pos = run_harness(tmp_path, "--max-tokens", "40")
    assert ids_in == PROMPT_IDS
    want, pos = expected(oracle, host, ids_in, oracle_lib.OracleSampler(oracle), 40)
    assert got == want and final_pos == pos

    # greedy after a repetition penalty, long enough to overflow the 64-row cache
    # twice: discard + key re-rotation on the device inside the reference's loop
    opts = dict(temperature=0.0, repeat_penalty=1.3, repeat_last_n=8)
    ids_in, got, final_pos = run_harness(tmp_path, "--max-tokens", "115", "--repeat-penalty",
                                         "1.3", "--repeat-last-n", "8")
    want, pos = expected(oracle, host, ids_in, oracle_lib.OracleSampler(oracle, **opts), 115)
    assert got == want and final_pos == pos
    assert len(got) == 115 - len(ids_in) + 1 or 151643 in got
    assert final_pos < len(ids_in) + len(got) - 1  # the position went back at least once

    # sampled
    opts = dict(temperature=0.9, top_k=20, top_p=0.95, min_p=0.02, repeat_penalty=1.1,
                repeat_last_n=16)
    ids_in, got, final_pos = run_harness(
        tmp_path, "--max-tokens", "36", "--temperature", "0.9", "--top-k", "20", "--top-p",
        "0.95", "--min-p", "0.02", "--repeat-penalty", "1.1", "--repeat-last-n", "16",
        "--seed", "7")
    want, pos = expected(oracle, host, ids_in, oracle_lib.OracleSampler(oracle, seed=7, **opts), 36)
    assert got == want and final_pos == pos


@pytest.mark.skipif(not EXAMPLE_MAIN.exists(), reason="oracle/_ref/ref_w8a32_main not built "
                    "(needs the reference tree: make -C oracle ref)")
def test_reference_example_program_with_the_library_as_its_model(tmp_path, bh, oracle):
    """examples/BuddyDeepSeekR1/buddy-deepseek-r1-w8a32-main.cpp, compiled unmodified
    and linked with libbuddy_hip where the reference links the compiled model: it
    reads vocab.txt and the two parameter files, tokenizes, calls
    _mlir_ciface_forward_prefill once and _mlir_ciface_forward_decode until the
    1024-row cache is full, taking the argmax on the host.  Its tokens are
    compared with a session created in this process from the same blobs (all of
    them) and with the CPU restatement (the first ones)."""
    import ctypes

    from test_gpu_model_abi import make_blobs

    shape = Shape(max_len=1024)  # the program's MaxTokenLength
    f32, i8, host = make_blobs(bh, shape, seed=3)
    (tmp_path / "arg0-w8a32-f32.data").write_bytes(f32.tobytes())
    (tmp_path / "arg0-w8a32-i8.data").write_bytes(i8.tobytes())
    write_vocab(tmp_path / "vocab.txt")
    import os

    # the program's DecodeReturns keeps the 27 position copies together
    # (buddy-deepseek-r1-w8a32-main.cpp:163-249); the generated ModelSession's
    # DecodeABI, the library's default, interleaves them with the KV pairs
    env = dict(os.environ, BUDDY_HIP_DECODE_RESULT_LAYOUT="grouped")
    r = subprocess.run([str(EXAMPLE_MAIN)], cwd=tmp_path, input=PROMPT + "\n", env=env,
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    vocab = (tmp_path / "vocab.txt").read_text(encoding="utf-8").split("\n")
    ids = {t: i for i, t in enumerate(vocab) if t}
    got = [ids[l.split("Token: ", 1)[1].split(" | ")[0]]
           for l in r.stdout.splitlines() if "Token: " in l]
    steps = shape.max_len - len(PROMPT_IDS)
    assert len(got) == steps + 1 or got[-1] == 151643
    assert "[Decoding]" in r.stdout and "[Output]" in r.stdout

    # the same blobs through a session of this process
    cs = shape.c()
    h = bh.buddy_hip_session_create_from_w8a32_blobs(ctypes.byref(cs), f32.ctypes.data, f32.size,
                                                     i8.ctypes.data, i8.size)
    assert h, bh.buddy_hip_last_error()
    toks = np.array(PROMPT_IDS, np.int32)
    first = ctypes.c_int(-1)
    assert bh.buddy_hip_session_prefill(h, toks.ctypes.data, toks.size, 0, None,
                                        ctypes.byref(first)) == 0
    rest = np.empty(len(got) - 1, np.int32)
    assert bh.buddy_hip_session_decode_greedy(h, first.value, toks.size, rest.size,
                                              rest.ctypes.data) == 0
    bh.buddy_hip_session_destroy(h)
    assert got == [first.value] + rest.tolist()

    # the CPU restatement: prompt rows and the first eight tokens
    om = oracle_lib.model_from_host(oracle, shape, host)
    kv = [np.zeros((shape.kv_heads, shape.max_len, shape.head_dim), np.float32)
          for _ in range(2 * shape.layers)]
    for pos, t in enumerate(PROMPT_IDS):
        tok, _ = om.decode_step(t, pos, kv)
    want = [tok]
    for step in range(7):
        tok, _ = om.decode_step(tok, len(PROMPT_IDS) + step, kv)
        want.append(tok)
    assert got[:8] == want
