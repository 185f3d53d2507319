"""buddy_mlir_amd -- Python face of libbuddy_hip.so.

The product is the C-ABI shared library under ``buddy_mlir_amd/lib`` (HIP
kernels for gfx950 behind buddy-mlir's ``_mlir_ciface_*`` memref convention).
This package only loads it with ctypes and offers thin helpers that pass
torch device pointers through; there is no CPU fallback: a missing library or a
failed call raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import (POINTER, Structure, c_char_p, c_float, c_int, c_int8,
                    c_int64, c_longlong, c_size_t, c_uint, c_void_p)
from pathlib import Path

__all__ = [
    "lib", "library_path", "MemRef", "memref_type", "BuddyHipError", "check",
]

_PKG = Path(__file__).resolve().parent
# BUDDY_HIP_LIBRARY: another build of the library (a measurement build), for
# the process that sets it
_LIB_PATH = Path(os.environ.get("BUDDY_HIP_LIBRARY") or _PKG / "lib" / "libbuddy_hip.so")
_lib = None


class BuddyHipError(RuntimeError):
    pass


def library_path() -> Path:
    return _LIB_PATH


def memref_type(ctype, rank: int):
    """ctypes mirror of the descriptor in include/buddy_hip/memref.h."""

    class _MemRef(Structure):
        _fields_ = [
            ("allocated", POINTER(ctype)),
            ("aligned", POINTER(ctype)),
            ("offset", ctypes.c_ssize_t),
            ("sizes", ctypes.c_ssize_t * rank),
            ("strides", ctypes.c_ssize_t * rank),
        ]

    _MemRef.__name__ = f"MemRef_{ctype.__name__}_{rank}d"
    return _MemRef


MemRefF32_1D = memref_type(c_float, 1)
MemRefF32_2D = memref_type(c_float, 2)
MemRefF32_3D = memref_type(c_float, 3)
MemRefF32_4D = memref_type(c_float, 4)
MemRefI8_1D = memref_type(c_int8, 1)
MemRefI8_2D = memref_type(c_int8, 2)
MemRefI64_1D = memref_type(c_longlong, 1)
MemRefI64_2D = memref_type(c_longlong, 2)


def MemRef(ptr: int, sizes, strides=None, ctype=c_float, offset: int = 0):
    """Builds a descriptor over raw memory at address `ptr` (host or device)."""
    rank = len(sizes)
    cls = memref_type(ctype, rank)
    if strides is None:
        strides, acc = [], 1
        for s in reversed(sizes):
            strides.insert(0, acc)
            acc *= s
    m = cls()
    p = ctypes.cast(c_void_p(ptr), POINTER(ctype))
    m.allocated = p
    m.aligned = p
    m.offset = offset
    for i in range(rank):
        m.sizes[i] = sizes[i]
        m.strides[i] = strides[i]
    return m


def _declare(lib):
    vp, i64, sz = c_void_p, c_int64, c_size_t
    sigs = {
        "buddy_hip_version": (c_char_p, []),
        "buddy_hip_last_error": (c_char_p, []),
        "buddy_hip_device_count": (c_int, []),
        "buddy_hip_variant_report": (i64, [vp, i64]),
        "buddy_hip_variant_reset": (None, []),
        "buddy_hip_w8_packed_bytes": (sz, [i64, i64]),
        "buddy_hip_pack_w8": (c_int, [vp, i64, i64, vp, vp]),
        "buddy_hip_unpack_w8": (c_int, [vp, i64, i64, vp, vp]),
        "buddy_hip_w8_packed_bytes_tiles": (sz, [i64, i64, c_int]),
        "buddy_hip_pack_w8_tiles": (c_int, [vp, i64, i64, c_int, vp, vp]),
        "buddy_hip_unpack_w8_tiles": (c_int, [vp, i64, i64, c_int, vp, vp]),
        "buddy_hip_quantize_w8": (c_int, [vp, i64, i64, vp, vp, vp]),
        "buddy_hip_gemv_w8a32": (c_int, [vp, vp, vp, vp, i64, i64, i64, c_uint,
                                         vp]),
        "buddy_hip_linear_w8a32": (c_int, [vp, vp]),
        "buddy_hip_mlp_block_workspace_bytes": (sz, [i64, i64]),
        "buddy_hip_mlp_block_w8a32": (c_int, [vp, vp]),
        "buddy_hip_gemm_w8a32": (c_int, [vp, vp, vp, vp, i64, i64, i64, c_uint, vp]),
        "buddy_hip_rmsnorm": (c_int, [vp, vp, vp, c_int, c_int, c_float, vp]),
        "buddy_hip_rope": (c_int, [vp, vp, vp, c_int, c_int, vp]),
        "buddy_hip_silu_mul": (c_int, [vp, vp, vp, i64, vp]),
        "buddy_hip_argmax_workspace_bytes": (sz, []),
        "buddy_hip_argmax": (c_int, [vp, c_int, vp, vp, vp]),
        "buddy_hip_attn_decode_workspace_bytes": (sz, [c_int, c_int]),
        "buddy_hip_gqa_decode_attention": (c_int, [vp, vp, vp, vp, vp, vp, vp, c_int,
                                                   c_int, c_int, c_int, c_float,
                                                   vp, sz, vp]),
        "buddy_hip_gqa_decode_attention_static": (c_int, [vp, vp, vp, vp, vp, vp, vp, c_int,
                                                          c_int, c_int, c_int, c_float,
                                                          vp]),
        "buddy_hip_static_scratch_init": (c_int, []),
        "buddy_hip_prefill_attention": (c_int, [vp, vp, vp, vp, vp, c_int, c_int, c_int,
                                                c_int, c_int, c_float, vp]),
        "buddy_hip_session_create": (vp, [vp, vp]),
        "buddy_hip_session_destroy": (None, [vp]),
        "buddy_hip_session_set_globals": (c_int, [vp, vp, vp, vp, vp, vp]),
        "buddy_hip_session_set_layer": (c_int, [vp, c_int, vp]),
        "buddy_hip_session_set_kv": (c_int, [vp, c_int, vp]),
        "buddy_hip_session_get_kv": (c_int, [vp, c_int, vp]),
        "buddy_hip_session_get_kv_rows": (c_int, [vp, c_int, c_int, vp]),
        "buddy_hip_session_decode_mirror": (c_int, [vp, c_int, c_int, vp, vp, vp]),
        "buddy_hip_session_use_graph": (c_int, [vp, c_int]),
        "buddy_hip_session_decode": (c_int, [vp, c_int, c_int, vp, vp]),
        "buddy_hip_session_decode_greedy": (c_int, [vp, c_int, c_int, c_int, vp]),
        "buddy_hip_session_prefill": (c_int, [vp, vp, c_int, c_int, vp, vp]),
        "buddy_hip_session_set_prefill_precision": (c_int, [vp, c_int]),
        "buddy_hip_session_prefill_all_logits": (c_int, [vp, vp, c_int, c_int, vp]),
        "buddy_hip_session_adopt": (None, [vp, vp]),
        "buddy_hip_w8a32_blob_sizes": (None, [vp, vp, vp]),
        "buddy_hip_w8a32_blob_layout": (i64, [vp, vp, i64]),
        "buddy_hip_set_gemv_batch_kernel": (c_int, [c_int]),
        "buddy_hip_gemv_w8a32_plan": (c_int, [i64, i64, i64, c_uint, vp]),
        "buddy_hip_attn_step_plan": (c_int, [c_int, c_int, c_int, vp, vp, vp]),
        "buddy_hip_session_create_from_w8a32_blobs": (vp, [vp, vp, i64, vp, i64]),
        "_mlir_ciface_forward_prefill": (None, [vp, vp, vp, vp]),
        "_mlir_ciface_forward_decode": (None, [vp] * 88),
        "buddy_hip_forward_reset": (None, []),
        "buddy_hip_forward_invalidate_kv": (None, []),
        "buddy_hip_session_set_state": (c_int, [vp, c_int, c_int]),
        "buddy_hip_session_discard_kv": (c_int, [vp, c_int, c_int, c_int]),
        "buddy_hip_session_discard_kv_freqs": (c_int, [vp, c_int, c_int, c_int, vp]),
        "buddy_hip_quantize_w4": (c_int, [vp, i64, i64, vp, vp, vp]),
        "buddy_hip_pack_int4": (c_int, [vp, i64, vp, vp]),
        "buddy_hip_gemv_w4a16": (c_int, [vp, vp, vp, vp, i64, i64, vp]),
        "buddy_hip_w4_tiles_bytes": (sz, [i64, i64]),
        "buddy_hip_pack_w4_tiles": (c_int, [vp, i64, i64, vp, vp]),
        "buddy_hip_gemv_w4a16_fast": (c_int, [vp, vp, vp, vp, i64, i64, vp]),
        "buddy_hip_kv_discard": (c_int, [vp, c_int, c_int, c_int, c_int, c_int, c_int,
                                         c_int, vp, vp]),
        "buddy_hip_forward_discard_kv": (c_int, [c_int, c_int, c_int]),
        "buddy_hip_session_enqueue_steps": (c_int, [vp, c_int]),
        "buddy_hip_session_logits": (vp, [vp]),
        "buddy_hip_session_stream": (vp, [vp]),
        "buddy_hip_session_vocab": (c_int, [vp]),
        "buddy_hip_sampler_create": (vp, [vp]),
        "buddy_hip_sampler_destroy": (None, [vp]),
        "buddy_hip_sampler_sample": (c_int, [vp, vp, c_int, vp, c_int, vp, vp]),
        "buddy_hip_session_decode_sample": (c_int, [vp, vp, c_int, c_int, vp, c_int, vp]),
        "buddy_hip_gemv_f32": (c_int, [vp, vp, vp, vp, i64, i64, c_uint, vp]),
        "buddy_hip_f32_tiles_bytes": (sz, [i64, i64]),
        "buddy_hip_tile_f32": (c_int, [vp, i64, i64, vp, vp]),
        "buddy_hip_gemv_f32_tiles": (c_int, [vp, vp, vp, vp, c_float, vp, i64, i64, c_uint,
                                             vp]),
        "buddy_hip_pack_panels_f32": (c_int, [vp, i64, i64, c_int, vp, vp]),
        "buddy_hip_unpack_panels_f32": (c_int, [vp, i64, i64, c_int, vp, vp]),
        "buddy_hip_gemv_f32_panels": (c_int, [vp, vp, vp, i64, i64, c_uint, vp]),
        "buddy_hip_w8a8_workspace_bytes": (sz, [i64, i64]),
        "buddy_hip_w8a8_matmul": (c_int, [vp, vp, vp, vp, vp, i64, i64, i64, vp, sz, vp]),
        "buddy_hip_matmul_f32": (c_int, [vp, vp, vp, i64, i64, i64, c_uint, vp]),
        "_mlir_ciface_buddy_matmul_f32": (None, [vp, vp, vp]),
        "_mlir_ciface_buddy_dequant_matmul_i8_f32": (None, [vp, vp, vp, vp]),
        "_mlir_ciface_buddy_dequant_matmul_i8_f32_acc": (None, [vp, vp, vp, vp]),
        "buddy_hip_clear_weight_cache": (None, []),
        "buddy_hip_set_weight_cache_limit": (None, [sz]),
        "buddy_hip_weight_cache_stats": (None, [vp]),
    }
    for name, (res, args) in sigs.items():
        if hasattr(lib, name):
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args


def lib():
    """Returns the loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            raise BuddyHipError(
                f"{_LIB_PATH} is missing: run `python -m buddy_mlir_amd.build`")
        _lib = ctypes.CDLL(str(_LIB_PATH), mode=os.RTLD_GLOBAL | os.RTLD_NOW)
        _declare(_lib)
    return _lib


def check(rc: int, what: str = "call"):
    if rc != 0:
        msg = lib().buddy_hip_last_error().decode()
        raise BuddyHipError(f"{what} failed with code {rc}: {msg}")
