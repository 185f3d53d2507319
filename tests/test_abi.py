"""The C-ABI library loads and exports every symbol include/buddy_hip/*.h
declares; descriptor layout matches buddy-mlir's MemRef<T,N>
(frontend/Interfaces/buddy/Core/Container.h:126-137, sizes checked against
tests/Interface/core/ContainerTest.cpp:27-60: shape {2,3} -> strides {3,1})."""
import ctypes
import re
from pathlib import Path

import buddy_mlir_amd as bma

ROOT = Path(__file__).resolve().parent.parent


def declared_symbols():
    text = (ROOT / "include" / "buddy_hip" / "buddy_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:buddy_hip_|_mlir_ciface_)\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol(bh):
    names = declared_symbols()
    assert len(names) >= 10
    missing = [n for n in names if not hasattr(bh, n)]
    assert not missing, f"declared but not exported: {missing}"


def test_version_and_error_strings(bh):
    assert b"gfx950" in bh.buddy_hip_version()
    assert isinstance(bh.buddy_hip_last_error(), bytes)


def test_memref_descriptor_layout():
    for rank in (1, 2, 3, 4):
        t = bma.memref_type(ctypes.c_float, rank)
        assert ctypes.sizeof(t) == 24 + 16 * rank
        assert t.sizes.offset == 24
        assert t.strides.offset == 24 + 8 * rank
    m = bma.MemRef(0, [2, 3])
    assert list(m.sizes) == [2, 3] and list(m.strides) == [3, 1]
    assert not m.aligned  # built over no data -> null, like the no-malloc ctor


def test_packed_bytes_is_padded_to_tiles(bh):
    assert bh.buddy_hip_w8_packed_bytes(1536, 8960) == 1536 * 8960
    assert bh.buddy_hip_w8_packed_bytes(1, 1) == 64 * 16
    assert bh.buddy_hip_w8_packed_bytes(65, 17) == 128 * 32
    assert bh.buddy_hip_w8_packed_bytes(0, 5) == 0


def test_exception_is_caught_at_the_boundary(bh):
    """A request whose host staging cannot exist (2^62 floats: std::vector
    refuses with std::length_error before anything is touched) must come back
    as an ordinary failure: result left null, message in buddy_hip_last_error(),
    the process alive -- nothing unwinds through the C ABI
    (examples/BuddyOneDNN/onednn_ops.cpp:229-241: stderr + return)."""
    import numpy as np
    a = np.zeros(4, np.float32)
    big = 1 << 31
    A = bma.MemRef(a.ctypes.data, [big, big], strides=[0, 0])
    B = bma.MemRef(a.ctypes.data, [big, 1], strides=[0, 0])
    res = bma.MemRefF32_2D()
    bh._mlir_ciface_buddy_matmul_f32(ctypes.byref(res), ctypes.byref(A), ctypes.byref(B))
    assert not res.aligned and not res.allocated
    msg = bh.buddy_hip_last_error()
    assert b"_mlir_ciface_buddy_matmul_f32" in msg, msg
