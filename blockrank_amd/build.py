"""Build libblockrank_hip.so in-tree with hipcc for gfx950.

Usage: ``python -m blockrank_amd.build`` (or ``blockrank_amd.build.build_library()``).  hipcc
cross-compiles without a GPU present.  The library is written next to this package so that the
loader (``blockrank_amd._lib``) finds it without any installation step.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libblockrank_hip.so"
OBJ_DIR = PKG_DIR / "csrc" / "build"

SOURCES = ["br_api.hip", "br_plan.hip", "br_prefill_mfma.hip", "br_prefill_f16.hip", "br_prefill_fp8.hip", "br_rope.hip", "br_bwd.hip", "br_norm_act.hip", "br_prefill_f32.hip", "br_scores.hip"]

# -packed-fp32-ops is switched off: the compiler must not form packed fp32 instructions on this target.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-strict-aliasing",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-inline-asm",      # the LDS-DMA asm names m0 as clobbered, which clang reports as "reserved"
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; a ROCm toolchain is required to build libblockrank_hip.so")
    return exe


def _compile(src: str, extra: list[str]) -> Path:
    obj = OBJ_DIR / (Path(src).stem + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-c", str(CSRC / src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")
    # the host pass warns that it does not know the packed-fp32 feature; anything else is shown
    noise = [l for l in res.stderr.splitlines() if l.strip() and "packed-fp32-ops" not in l]
    if noise:
        sys.stderr.write("\n".join(noise) + "\n")
    return obj


def build_library(extra_flags: list[str] | None = None, jobs: int = 6) -> Path:
    """Compile every kernel source and link the shared library.  Always recompiles."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    extra = list(extra_flags or [])
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, extra), SOURCES))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library())
