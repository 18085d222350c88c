"""Build libmaltos_hip.so (gfx950) from maltos_amd/csrc/*.hip with hipcc.

    python -m maltos_amd.build            # compile every source and link, in-tree

The library is a plain C-ABI shared object (see include/maltos_hip.h); it links only against the
HIP runtime, not against torch, so C/C++ hosts can bind it as well.
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
LIB_PATH = PKG_DIR / "libmaltos_hip.so"
OBJ_DIR = PKG_DIR / "csrc" / "build"

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-math-errno",
    # packed fp32 VALU forms are kept off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc not found; the HIP kernels cannot be built")
    return found


def _compile_one(src: Path, verbose: bool) -> Path:
    obj = OBJ_DIR / (src.stem + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{proc.stderr}")
    if verbose:
        print(f"[maltos_amd.build] compiled {src.name}", flush=True)
    return obj


def build(verbose: bool = True, jobs: int | None = None) -> Path:
    """Compile every kernel source and link the shared library; always rebuilds."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    sources = sorted(CSRC.glob("*.hip"))
    if not sources:
        raise RuntimeError(f"no .hip sources under {CSRC}")
    jobs = jobs or min(8, len(sources), os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile_one(s, verbose), sources))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[maltos_amd.build] linked {LIB_PATH}", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build(verbose=True)
    sys.exit(0)
