"""Compiles libbuddy_hip.so for gfx950 with hipcc, in-tree.

    python -m buddy_mlir_amd.build

hipcc cross-compiles without a GPU.  The library lands in
buddy_mlir_amd/lib/libbuddy_hip.so; objects are cached per source file under
buddy_mlir_amd/lib/obj and rebuilt when the source or a header is newer.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
LIBDIR = PKG / "lib"
OBJDIR = LIBDIR / "obj"
LIB = LIBDIR / "libbuddy_hip.so"
RUNNER_SRC = PKG / "runner" / "buddy_hip_run.cpp"
RUNNER = LIBDIR / "buddy_hip_run"

ARCH = "gfx950"
# -packed-fp32-ops off: scalar float code must not be turned into v_pk_*_f32.
COMMON = [
    "-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    f"-I{ROOT / 'include'}", f"-I{CSRC}",
]


# Kernels of these files issue global loads through inline asm and wait for them
# by hand.  The compiler believes such a load's result exists as soon as the
# load is issued: if it spilled one of those registers it would store garbage
# and hand the register to something else while the load is still in flight.
# Their kernels must therefore use no scratch at all; the build checks it.
NO_SCRATCH = {"gemm_w8_mfma.hip", "gemv_w8a32_mfma.hip", "gemv_w8a32_i8.hip", "gemm_w8_i8.hip",
              "attn_prefill.hip"}


def _check_no_scratch(src: Path, remarks: str) -> None:
    name = None
    bad = []
    for line in remarks.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in line:
            n = int(line.split("ScratchSize [bytes/lane]:")[1].split("[")[0])
            if n:
                bad.append(f"{name}: {n} bytes of scratch per lane")
    if bad:
        raise RuntimeError(
            f"{src.name}: kernels with hand-issued loads must not spill:\n  "
            + "\n  ".join(bad))


# Every kernel takes its leading scalar and pointer arguments preloaded into SGPRs by
# the command processor (up to this many argument words; arguments behind a
# struct passed by value are loaded as usual): a wavefront's first loads then do
# not wait for a scalar load of the argument block.
KERNARG_PRELOAD = 14


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def sources() -> list[Path]:
    return sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.cpp")))


def _headers_mtime() -> float:
    hs = list(CSRC.glob("*.h")) + list((ROOT / "include").rglob("*.h"))
    return max(h.stat().st_mtime for h in hs)


def _compile(src: Path, force: bool) -> Path:
    obj = OBJDIR / (src.name + ".o")
    newest = max(src.stat().st_mtime, _headers_mtime(), Path(__file__).stat().st_mtime)
    if not force and obj.exists() and obj.stat().st_mtime >= newest:
        return obj
    cmd = [_hipcc(), *COMMON, "-x", "hip", "-c", str(src), "-o", str(obj)]
    if src.name in NO_SCRATCH:
        cmd.append("-Rpass-analysis=kernel-resource-usage")
    if src.suffix == ".hip":
        cmd += ["-mllvm", f"-amdgpu-kernarg-preload-count={KERNARG_PRELOAD}"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{r.stdout}\n{r.stderr}")
    if src.name in NO_SCRATCH:
        try:
            _check_no_scratch(src, r.stderr)
        except RuntimeError:
            obj.unlink(missing_ok=True)
            raise
    return obj


def build(force: bool = False, jobs: int = 8, verbose: bool = True) -> Path:
    OBJDIR.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    cmd = [_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}",
           "-o", str(LIB), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    # the command-line runner for the reference's w8a32 parameter files: plain
    # C++ over the C interface, found next to the library at run time
    cmd = [_hipcc(), "-O2", "-std=c++17", f"-I{ROOT / 'include'}", str(RUNNER_SRC),
           f"-L{LIBDIR}", "-lbuddy_hip", "-Wl,-rpath,$ORIGIN", "-o", str(RUNNER)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"runner build failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources, and {RUNNER.name}")
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
