"""buddy_hip_run, the command-line runner for the reference's w8a32 parameter
files: argument handling without a GPU, and on the GPU a whole generation from
files on disk against the in-process session and the CPU oracle."""
import ctypes
import subprocess

import numpy as np
import pytest

import buddy_mlir_amd as bma

RUNNER = bma.library_path().parent / "buddy_hip_run"


def run(*args):
    return subprocess.run([str(RUNNER), *args], capture_output=True, text=True, timeout=300)


def test_runner_is_built_and_explains_itself():
    assert RUNNER.exists(), "run `python -m buddy_mlir_amd.build`"
    r = run("--help")
    assert r.returncode == 0 and "arg0-w8a32-f32.data" in r.stdout


@pytest.mark.parametrize("args", [
    (),                                             # nothing
    ("--f32", "a", "--i8", "b"),                    # no prompt
    ("--f32", "a", "--i8", "b", "--tokens", "1,x"),  # not a token list
    ("--f32", "a", "--i8", "b", "--tokens", "1", "--bogus", "2"),
    ("--f32", "a", "--i8", "b", "--tokens", "1,2", "--max-new", "2000"),  # beyond the cache
    ("--f32", "a", "--i8", "b", "--tokens", "999999"),                     # beyond the vocabulary
])
def test_runner_refuses_bad_arguments(args):
    r = run(*args)
    assert r.returncode == 2 and r.stderr


def test_runner_reports_missing_and_short_files(tmp_path):
    r = run("--f32", str(tmp_path / "none"), "--i8", str(tmp_path / "none"), "--tokens", "1")
    assert r.returncode == 1 and "Failed to open params file" in r.stderr
    short = tmp_path / "short.data"
    short.write_bytes(b"\0" * 100)
    r = run("--f32", str(short), "--i8", str(short), "--tokens", "1")
    assert r.returncode == 1 and "the model shape needs" in r.stderr


@pytest.mark.gpu
def test_runner_generates_what_the_session_and_the_oracle_generate(tmp_path, bh, oracle):
    import oracle_lib
    from test_gpu_decode import SMALL
    from test_gpu_model_abi import make_blobs

    f32, i8, host = make_blobs(bh, SMALL, seed=4)
    (tmp_path / "arg0-w8a32-f32.data").write_bytes(f32.tobytes())
    (tmp_path / "arg0-w8a32-i8.data").write_bytes(i8.tobytes())
    prompt = [5, 17, 300, 2, 999, 64, 31, 8]
    new = 20
    r = run("--f32", str(tmp_path / "arg0-w8a32-f32.data"),
            "--i8", str(tmp_path / "arg0-w8a32-i8.data"),
            "--tokens", ",".join(map(str, prompt)), "--max-new", str(new), "--eos", "-1",
            "--layers", str(SMALL.layers), "--hidden", str(SMALL.hidden),
            "--heads", str(SMALL.heads), "--kv-heads", str(SMALL.kv_heads),
            "--inter", str(SMALL.inter), "--vocab", str(SMALL.vocab),
            "--max-len", str(SMALL.max_len))
    assert r.returncode == 0, r.stderr
    lines = dict(l.split("]", 1) for l in r.stdout.splitlines() if l.startswith("["))
    assert [int(t) for t in lines["[Input ids"].split()] == prompt
    got = [int(t) for t in lines["[Output ids"].split()]
    assert len(got) == new
    assert float(lines["[Decoding"].split()[0]) > 0

    # the CPU oracle, token by token, on the same parameters
    om = oracle_lib.model_from_host(oracle, SMALL, host)
    kv = [np.zeros((SMALL.kv_heads, SMALL.max_len, SMALL.head_dim), np.float32)
          for _ in range(2 * SMALL.layers)]
    for pos, t in enumerate(prompt):
        tok, _ = om.decode_step(t, pos, kv)
    want = [tok]
    for step in range(new - 1):
        tok, _ = om.decode_step(tok, len(prompt) + step, kv)
        want.append(tok)
    assert got == want

    # an end-of-text id stops the generation
    r = run("--f32", str(tmp_path / "arg0-w8a32-f32.data"),
            "--i8", str(tmp_path / "arg0-w8a32-i8.data"),
            "--tokens", ",".join(map(str, prompt)), "--max-new", str(new),
            "--eos", str(want[3]),
            "--layers", str(SMALL.layers), "--hidden", str(SMALL.hidden),
            "--heads", str(SMALL.heads), "--kv-heads", str(SMALL.kv_heads),
            "--inter", str(SMALL.inter), "--vocab", str(SMALL.vocab),
            "--max-len", str(SMALL.max_len))
    assert r.returncode == 0, r.stderr
    out = [l for l in r.stdout.splitlines() if l.startswith("[Output ids]")][0]
    got = [int(t) for t in out.split("]")[1].split()]
    assert got == want[:want.index(want[3]) + 1]

    # sampled generation: the same files, the reference's sampler options
    opts = dict(temperature=0.9, top_k=20, top_p=0.95, min_p=0.02, repeat_penalty=1.15,
                repeat_last_n=8)
    r = run("--f32", str(tmp_path / "arg0-w8a32-f32.data"),
            "--i8", str(tmp_path / "arg0-w8a32-i8.data"),
            "--tokens", ",".join(map(str, prompt)), "--max-new", str(new), "--eos", "-1",
            "--layers", str(SMALL.layers), "--hidden", str(SMALL.hidden),
            "--heads", str(SMALL.heads), "--kv-heads", str(SMALL.kv_heads),
            "--inter", str(SMALL.inter), "--vocab", str(SMALL.vocab),
            "--max-len", str(SMALL.max_len), "--temperature", "0.9", "--top-k", "20",
            "--top-p", "0.95", "--min-p", "0.02", "--repeat-penalty", "1.15",
            "--repeat-last-n", "8", "--seed", "7")
    assert r.returncode == 0, r.stderr
    out = [l for l in r.stdout.splitlines() if l.startswith("[Output ids]")][0]
    got = [int(t) for t in out.split("]")[1].split()]
    sampler = oracle_lib.OracleSampler(oracle, seed=7, **opts)
    kv = [np.zeros_like(k) for k in kv]
    for pos, t in enumerate(prompt):
        _, logits = om.decode_step(t, pos, kv)
    want = [sampler.sample(logits, [])[0]]
    for step in range(new - 1):
        _, logits = om.decode_step(want[-1], len(prompt) + step, kv)
        want.append(sampler.sample(logits, want)[0])
    assert got == want
    assert len(set(got)) > 1
