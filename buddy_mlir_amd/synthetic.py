"""Seeded synthetic Qwen2-shaped int8 decoder for tests and the benchmark.

Random-init weights ~ N(0, 0.02) generated on the device with torch's seeded
generator, quantized per output channel by libbuddy_hip's own quantizer (the
reference recipe, tools/buddy-codegen/import_model.py:837-848); norm weights
are ones; the KV cache is filled with N(0,1) for the first `context` rows.
Weights are kept in the importer's orientation: W[K, N] = [in, out].
"""
from __future__ import annotations

import numpy as np
import torch

from . import ops
from .session import DecoderSession, Shape

SEED = 0x5EED


def _gen(seed):
    return torch.Generator(device="cuda").manual_seed(seed)


def quantized_linear(K: int, N: int, seed: int, std: float = 0.02):
    W = torch.randn((K, N), generator=_gen(seed), device="cuda") * std
    q, s = ops.quantize_w8(W)
    del W
    return q, s


def inv_freq(head_dim: int, theta: float = 1e6) -> torch.Tensor:
    i = torch.arange(0, head_dim, 2, dtype=torch.int64).float()
    return (1.0 / (theta ** (i / head_dim))).cuda()


def make_layer(shape: Shape, layer: int, ln_jitter: float = 0.0):
    H, QN, KVN, I = (shape.hidden, shape.heads * shape.head_dim,
                     shape.kv_heads * shape.head_dim, shape.inter)
    base = SEED + 100 * layer
    w = {}
    w["wq"], w["sq"] = quantized_linear(H, QN, base + 1)
    w["wk"], w["sk"] = quantized_linear(H, KVN, base + 2)
    w["wv"], w["sv"] = quantized_linear(H, KVN, base + 3)
    w["wo"], w["so"] = quantized_linear(QN, H, base + 4)
    w["wg"], w["sg"] = quantized_linear(H, I, base + 5)
    w["wu"], w["su"] = quantized_linear(H, I, base + 6)
    w["wd"], w["sd"] = quantized_linear(I, H, base + 7)
    ones = torch.ones(H, device="cuda")
    if ln_jitter:
        w["ln1"] = ones + ln_jitter * torch.randn(H, generator=_gen(base + 8), device="cuda")
        w["ln2"] = ones + ln_jitter * torch.randn(H, generator=_gen(base + 9), device="cuda")
    else:
        w["ln1"], w["ln2"] = ones.clone(), ones.clone()
    return w


def make_globals(shape: Shape):
    g = {}
    g["embed"] = torch.randn((shape.vocab, shape.hidden), generator=_gen(SEED - 1),
                             device="cuda") * 0.02
    g["inv_freq"] = inv_freq(shape.head_dim)
    g["ln_f"] = torch.ones(shape.hidden, device="cuda")
    g["w_lm"], g["s_lm"] = quantized_linear(shape.hidden, shape.vocab, SEED - 2)
    return g


def make_kv(shape: Shape, kv_index: int, context: int) -> torch.Tensor:
    t = torch.zeros((shape.kv_heads, shape.max_len, shape.head_dim), device="cuda")
    if context:
        t[:, :context, :] = torch.randn((shape.kv_heads, context, shape.head_dim),
                                        generator=_gen(SEED + 7000 + kv_index),
                                        device="cuda")
    return t


def build_session(shape: Shape, context: int, keep_host: bool = False,
                  ln_jitter: float = 0.0):
    """Returns (session, host) where host holds numpy copies of every tensor
    when keep_host is set (for the CPU oracle), else None."""
    sess = DecoderSession(shape)
    host = {"layers": [], "kv": []} if keep_host else None
    g = make_globals(shape)
    sess.set_globals(g["embed"], g["inv_freq"], g["ln_f"], g["w_lm"], g["s_lm"])
    if keep_host:
        host["globals"] = {k: v.cpu().numpy() for k, v in g.items()}
    sess._globals = g
    for i in range(shape.layers):
        w = make_layer(shape, i, ln_jitter)
        sess.set_layer(i, w)
        if keep_host:
            host["layers"].append({k: v.cpu().numpy() for k, v in w.items()})
        del w
    for j in range(2 * shape.layers):
        kv = make_kv(shape, j, context)
        sess.set_kv(j, kv)
        if keep_host:
            host["kv"].append(kv.cpu().numpy())
        del kv
    torch.cuda.synchronize()
    return sess, host


def first_tokens(shape: Shape, n: int, seed: int = SEED + 9999) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return rng.integers(0, shape.vocab, n).astype(np.int64)
