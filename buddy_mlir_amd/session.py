"""Host-side mirror of the reference's generated ModelSession
(tools/buddy-codegen/gen_session.py:201-256: create / loadWeights / decode /
logitsData) over libbuddy_hip's resident decoder session.

torch tensors are used as device buffers only.
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_float, c_int, c_void_p
from dataclasses import dataclass

import numpy as np
import torch

from . import BuddyHipError, check, lib


class ModelShape(Structure):
    _fields_ = [(n, c_int) for n in ("layers", "hidden", "heads", "kv_heads",
                                     "head_dim", "inter", "vocab", "max_len")] + \
               [("rms_eps", c_float)]


class LayerWeights(Structure):
    _fields_ = [(n, c_void_p) for n in
                ("ln1", "ln2", "wq", "wk", "wv", "wo", "wg", "wu", "wd",
                 "sq", "sk", "sv", "so", "sg", "su", "sd", "bq", "bk", "bv",
                 "fq", "fk", "fv")]


@dataclass
class Shape:
    layers: int = 28
    hidden: int = 1536
    heads: int = 12
    kv_heads: int = 2
    head_dim: int = 128
    inter: int = 8960
    vocab: int = 151936
    max_len: int = 1088
    rms_eps: float = 1e-6

    def c(self) -> ModelShape:
        return ModelShape(self.layers, self.hidden, self.heads, self.kv_heads,
                          self.head_dim, self.inter, self.vocab, self.max_len,
                          self.rms_eps)


QWEN2_1P5B = Shape()


def _ptr(t):
    if t is None:
        return None
    if not t.is_cuda or not t.is_contiguous():
        raise ValueError("expected a contiguous device tensor")
    return t.data_ptr()


class DecoderSession:
    """One resident decoder.  decode() mirrors ModelSession::decode(tokenId)
    with the position made explicit; the KV cache lives on the device."""

    def __init__(self, shape: Shape):
        self.shape = shape
        self._lib = lib()
        cs = shape.c()
        self._h = self._lib.buddy_hip_session_create(ctypes.byref(cs), None)
        if not self._h:
            raise BuddyHipError("session_create failed: " +
                                self._lib.buddy_hip_last_error().decode())
        self._keep = []

    def close(self):
        if self._h:
            self._lib.buddy_hip_session_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- weights (ModelSession::loadWeights) --------------------------------
    def set_globals(self, embed, inv_freq, ln_f, w_lm, s_lm):
        torch.cuda.synchronize()
        self._keep.append(embed)  # borrowed by the session
        check(self._lib.buddy_hip_session_set_globals(
            self._h, _ptr(embed), _ptr(inv_freq), _ptr(ln_f), _ptr(w_lm),
            _ptr(s_lm)), "session_set_globals")

    def set_layer(self, index: int, w: dict):
        torch.cuda.synchronize()
        lw = LayerWeights()
        for name, _ in LayerWeights._fields_:
            setattr(lw, name, _ptr(w.get(name)))
        check(self._lib.buddy_hip_session_set_layer(self._h, index, ctypes.byref(lw)),
              "session_set_layer")

    # -- KV cache -------------------------------------------------------------
    def set_kv(self, kv_index: int, t):
        if isinstance(t, np.ndarray):
            t = np.ascontiguousarray(t, np.float32)
            p = t.ctypes.data
        else:
            torch.cuda.synchronize()
            p = _ptr(t)
        check(self._lib.buddy_hip_session_set_kv(self._h, kv_index, p), "session_set_kv")

    def get_kv(self, kv_index: int) -> np.ndarray:
        s = self.shape
        out = np.empty((s.kv_heads, s.max_len, s.head_dim), np.float32)
        check(self._lib.buddy_hip_session_get_kv(self._h, kv_index, out.ctypes.data),
              "session_get_kv")
        return out

    # -- decode ---------------------------------------------------------------
    def use_graph(self, enable: bool):
        check(self._lib.buddy_hip_session_use_graph(self._h, int(enable)), "use_graph")

    def decode(self, token: int, pos: int, want_logits: bool = True):
        logits = np.empty(self.shape.vocab, np.float32) if want_logits else None
        nxt = c_int(-1)
        check(self._lib.buddy_hip_session_decode(
            self._h, token, pos, None if logits is None else logits.ctypes.data,
            ctypes.byref(nxt)), "session_decode")
        return nxt.value, logits

    def decode_greedy(self, first_token: int, start_pos: int, steps: int):
        out = np.empty(steps, np.int32)
        check(self._lib.buddy_hip_session_decode_greedy(
            self._h, first_token, start_pos, steps, out.ctypes.data), "decode_greedy")
        return out

    PREFILL_PRECISION = {"bf16": 0, "exact": 1, "digits": 2, "digits2": 3}

    def prefill(self, tokens, start_pos: int = 0, want_logits: bool = True,
                precision: str = "digits"):
        """ModelSession::prefill: the prompt as one block.  Returns (greedy next
        token, logits of the last prompt token).  precision: how the matmuls
        carry their f32 activations -- "digits" (three int8 digit planes on the
        int8 matrix cores), "digits2" (two planes), "exact" (three bf16 terms)
        or "bf16" (cast)."""
        toks = np.ascontiguousarray(tokens, np.int32)
        check(self._lib.buddy_hip_session_set_prefill_precision(
            self._h, self.PREFILL_PRECISION[precision]), "set_prefill_precision")
        logits = np.empty(self.shape.vocab, np.float32) if want_logits else None
        nxt = c_int(-1)
        check(self._lib.buddy_hip_session_prefill(
            self._h, toks.ctypes.data, toks.size, start_pos,
            None if logits is None else logits.ctypes.data, ctypes.byref(nxt)),
            "session_prefill")
        return nxt.value, logits

    def decode_sample(self, sampler: "Sampler", token: int, pos: int, recent=()):
        """One decode step, then the sampler's choice from its logits."""
        rec = np.ascontiguousarray(recent, np.int32)
        nxt = c_int(-1)
        check(self._lib.buddy_hip_session_decode_sample(
            self._h, sampler._h, token, pos, rec.ctypes.data if rec.size else None,
            rec.size, ctypes.byref(nxt)), "session_decode_sample")
        return nxt.value

    def set_state(self, token: int, pos: int):
        check(self._lib.buddy_hip_session_set_state(self._h, token, pos), "set_state")

    def discard_kv(self, keep: int, discard: int, count: int):
        """kvcache::discardKVCache + adjustKeyCacheRope on the device caches."""
        check(self._lib.buddy_hip_session_discard_kv(self._h, keep, discard, count),
              "session_discard_kv")

    def enqueue_steps(self, steps: int):
        check(self._lib.buddy_hip_session_enqueue_steps(self._h, steps), "enqueue_steps")

    @property
    def stream(self) -> int:
        return self._lib.buddy_hip_session_stream(self._h) or 0


class SamplerConfig(Structure):
    _fields_ = [("temperature", c_float), ("top_k", c_int), ("top_p", c_float),
                ("min_p", c_float), ("repeat_penalty", c_float), ("repeat_last_n", c_int),
                ("seed", ctypes.c_uint64)]


class Sampler:
    """buddy::runtime::Sampler (runtime/include/buddy/runtime/llm/Sampler.h:38-206)
    with the same defaults; logits are a device tensor."""

    def __init__(self, temperature=0.0, top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=1.0,
                 repeat_last_n=64, seed=0):
        self._lib = lib()
        cfg = SamplerConfig(temperature, top_k, top_p, min_p, repeat_penalty, repeat_last_n,
                            seed)
        self._h = self._lib.buddy_hip_sampler_create(ctypes.byref(cfg))
        if not self._h:
            raise BuddyHipError(self._lib.buddy_hip_last_error().decode())

    def sample(self, logits: torch.Tensor, recent=(), stream: int = 0) -> int:
        assert logits.dtype == torch.float32 and logits.is_contiguous()
        rec = np.ascontiguousarray(recent, np.int32)
        tok = c_int(-1)
        check(self._lib.buddy_hip_sampler_sample(
            self._h, logits.data_ptr(), logits.numel(), rec.ctypes.data if rec.size else None,
            rec.size, ctypes.byref(tok), stream or None), "sampler_sample")
        return tok.value

    def close(self):
        if getattr(self, "_h", None):
            self._lib.buddy_hip_sampler_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
