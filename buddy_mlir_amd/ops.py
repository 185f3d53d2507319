"""Helpers that call libbuddy_hip.so on torch device tensors.

torch is used for device memory and streams only; every computation here goes
through the C ABI.  Nothing falls back to torch or to the CPU.
"""
from __future__ import annotations

import ctypes

import torch

from . import check, lib

GEMV_ACCUMULATE = 1
EPI_STORE, EPI_ACCUM, EPI_SILU_MUL = 0, 1, 2


class LinearDesc(ctypes.Structure):
    """ctypes mirror of buddy_hip_linear_desc."""
    _fields_ = [("A", ctypes.c_void_p), ("lda", ctypes.c_int64),
                ("W0", ctypes.c_void_p), ("scale0", ctypes.c_void_p),
                ("W1", ctypes.c_void_p), ("scale1", ctypes.c_void_p),
                ("bias", ctypes.c_void_p), ("norm_w", ctypes.c_void_p),
                ("norm_eps", ctypes.c_float), ("C", ctypes.c_void_p),
                ("ldc", ctypes.c_int64), ("M", ctypes.c_int64),
                ("K", ctypes.c_int64), ("N", ctypes.c_int64),
                ("epilogue", ctypes.c_int), ("tile_n", ctypes.c_int)]


def linear_desc(**kw) -> LinearDesc:
    d = LinearDesc()
    for k, v in kw.items():
        setattr(d, k, v.data_ptr() if isinstance(v, torch.Tensor) else v)
    return d


def linear_w8a32(stream=None, **kw):
    """buddy_hip_linear_w8a32 with keyword fields of the descriptor."""
    d = linear_desc(**kw)
    check(lib().buddy_hip_linear_w8a32(ctypes.byref(d),
                                       _stream() if stream is None else stream),
          "linear_w8a32")


class MlpBlockDesc(ctypes.Structure):
    """ctypes mirror of buddy_hip_mlp_block_desc."""
    _fields_ = [("x", ctypes.c_void_p), ("ldx", ctypes.c_int64),
                ("norm_w", ctypes.c_void_p), ("norm_eps", ctypes.c_float),
                ("gate", ctypes.c_void_p), ("gate_scale", ctypes.c_void_p),
                ("up", ctypes.c_void_p), ("up_scale", ctypes.c_void_p),
                ("down", ctypes.c_void_p), ("down_scale", ctypes.c_void_p),
                ("y", ctypes.c_void_p), ("ldy", ctypes.c_int64),
                ("M", ctypes.c_int64), ("hidden", ctypes.c_int64), ("inter", ctypes.c_int64),
                ("flags", ctypes.c_uint), ("workspace", ctypes.c_void_p),
                ("workspace_bytes", ctypes.c_size_t)]


def mlp_block_desc(x, gate, gate_scale, up, up_scale, down, down_scale, y, hidden: int,
                   inter: int, norm_w=None, norm_eps: float = 0.0, accumulate: bool = False,
                   workspace=None):
    """Descriptor of buddy_hip_mlp_block_w8a32 over torch device tensors, plus
    the workspace tensor it points into (keep it alive)."""
    M = x.shape[0]
    if workspace is None:
        workspace = torch.empty(lib().buddy_hip_mlp_block_workspace_bytes(M, inter),
                                dtype=torch.uint8, device=x.device)
    d = MlpBlockDesc()
    d.x, d.ldx = x.data_ptr(), x.stride(0)
    d.norm_w = norm_w.data_ptr() if norm_w is not None else None
    d.norm_eps = norm_eps
    d.gate, d.gate_scale = gate.data_ptr(), gate_scale.data_ptr()
    d.up, d.up_scale = up.data_ptr(), up_scale.data_ptr()
    d.down, d.down_scale = down.data_ptr(), down_scale.data_ptr()
    d.y, d.ldy = y.data_ptr(), y.stride(0)
    d.M, d.hidden, d.inter = M, hidden, inter
    d.flags = GEMV_ACCUMULATE if accumulate else 0
    d.workspace, d.workspace_bytes = workspace.data_ptr(), workspace.numel()
    return d, workspace


def mlp_block_w8a32(x, gate, gate_scale, up, up_scale, down, down_scale, hidden: int,
                    inter: int, y=None, stream=None, **kw):
    """y (+)= (SiLU(x' . gate) * (x' . up)) . down for 1..16 rows (two launches)."""
    if y is None:
        y = torch.empty((x.shape[0], hidden), dtype=torch.float32, device=x.device)
    d, ws = mlp_block_desc(x, gate, gate_scale, up, up_scale, down, down_scale, y, hidden,
                           inter, **kw)
    check(lib().buddy_hip_mlp_block_w8a32(ctypes.byref(d),
                                          _stream() if stream is None else stream),
          "mlp_block_w8a32")
    return y


def pack_w8_tiles(q: torch.Tensor, tile_n: int) -> torch.Tensor:
    _dev(q, torch.int8)
    K, N = q.shape
    nbytes = lib().buddy_hip_w8_packed_bytes_tiles(K, N, tile_n)
    if nbytes == 0:
        raise ValueError(f"bad tile_n {tile_n}")
    out = torch.empty((nbytes,), dtype=torch.int8, device=q.device)
    check(lib().buddy_hip_pack_w8_tiles(q.data_ptr(), K, N, tile_n, out.data_ptr(),
                                        _stream()), "pack_w8_tiles")
    return out


def unpack_w8_tiles(packed: torch.Tensor, K: int, N: int, tile_n: int) -> torch.Tensor:
    _dev(packed, torch.int8)
    out = torch.empty((K, N), dtype=torch.int8, device=packed.device)
    check(lib().buddy_hip_unpack_w8_tiles(packed.data_ptr(), K, N, tile_n,
                                          out.data_ptr(), _stream()), "unpack_w8_tiles")
    return out


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor, dtype) -> torch.Tensor:
    if not t.is_cuda:
        raise ValueError("expected a device tensor")
    if t.dtype != dtype or not t.is_contiguous():
        raise ValueError(f"expected contiguous {dtype}, got {t.dtype}")
    return t


def quantize_w8(w: torch.Tensor):
    """Per-output-channel symmetric int8 quantization of W[K,N] on device."""
    _dev(w, torch.float32)
    K, N = w.shape
    q = torch.empty((K, N), dtype=torch.int8, device=w.device)
    s = torch.empty((N,), dtype=torch.float32, device=w.device)
    check(lib().buddy_hip_quantize_w8(w.data_ptr(), K, N, q.data_ptr(),
                                      s.data_ptr(), _stream()), "quantize_w8")
    return q, s


def pack_w8(q: torch.Tensor) -> torch.Tensor:
    """Row-major int8 W[K,N] -> wave-tile packed bytes."""
    _dev(q, torch.int8)
    K, N = q.shape
    nbytes = lib().buddy_hip_w8_packed_bytes(K, N)
    out = torch.empty((nbytes,), dtype=torch.int8, device=q.device)
    check(lib().buddy_hip_pack_w8(q.data_ptr(), K, N, out.data_ptr(), _stream()),
          "pack_w8")
    return out


def unpack_w8(packed: torch.Tensor, K: int, N: int) -> torch.Tensor:
    _dev(packed, torch.int8)
    out = torch.empty((K, N), dtype=torch.int8, device=packed.device)
    check(lib().buddy_hip_unpack_w8(packed.data_ptr(), K, N, out.data_ptr(),
                                    _stream()), "unpack_w8")
    return out


def gemv_w8a32(x: torch.Tensor, packed: torch.Tensor, scale: torch.Tensor,
               K: int, N: int, out: torch.Tensor | None = None,
               accumulate: bool = False):
    """out[M,N] (+)= (x[M,K] . W[K,N]) * scale[N] with W wave-tile packed."""
    _dev(x, torch.float32)
    _dev(packed, torch.int8)
    _dev(scale, torch.float32)
    M = x.shape[0]
    if x.shape != (M, K):
        raise ValueError(f"x is {tuple(x.shape)}, expected ({M},{K})")
    if out is None:
        if accumulate:
            raise ValueError("accumulate needs an output tensor")
        out = torch.empty((M, N), dtype=torch.float32, device=x.device)
    _dev(out, torch.float32)
    check(lib().buddy_hip_gemv_w8a32(
        x.data_ptr(), packed.data_ptr(), scale.data_ptr(), out.data_ptr(), M, K,
        N, GEMV_ACCUMULATE if accumulate else 0, _stream()), "gemv_w8a32")
    return out


GEMM_A_F32_EXACT = 2
GEMM_A_I8_DIGITS = 4
GEMM_SILU_PAIR = 8
GEMM_TWO_DIGITS = 16


def gemm_w8a32(x: torch.Tensor, packed: torch.Tensor, scale: torch.Tensor,
               K: int, N: int, out: torch.Tensor | None = None,
               accumulate: bool = False, exact: bool = False, digits: bool | int = False,
               silu_pair: bool = False):
    """Prefill matmul on the matrix cores: out[M,N] (+)= x[M,K] . (W * scale).
    Activations: cast to bf16 (default), three bf16 terms (exact) or three int8
    digit planes on the int8 matrix cores (digits; digits=2: two planes).  silu_pair (with digits):
    packed and scale hold two matrices of N channels one behind the other and
    out[M,N] = SiLU(x . W0) * (x . W1)."""
    _dev(x, torch.float32)
    _dev(packed, torch.int8)
    _dev(scale, torch.float32)
    M = x.shape[0]
    if out is None:
        if accumulate:
            raise ValueError("accumulate needs an output tensor")
        out = torch.empty((M, N), dtype=torch.float32, device=x.device)
    flags = ((GEMV_ACCUMULATE if accumulate else 0) | (GEMM_A_F32_EXACT if exact else 0) |
             (GEMM_A_I8_DIGITS if digits else 0) | (GEMM_SILU_PAIR if silu_pair else 0) |
             (GEMM_TWO_DIGITS if digits == 2 and digits is not True else 0))
    check(lib().buddy_hip_gemm_w8a32(x.data_ptr(), packed.data_ptr(), scale.data_ptr(),
                                     out.data_ptr(), M, K, N, flags, _stream()),
          "gemm_w8a32")
    return out
