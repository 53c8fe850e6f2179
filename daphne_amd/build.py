"""Builds libdaphne_hip.so (gfx950 only) with hipcc. No GPU is needed to build.

    python -m daphne_amd.build          # compile every .hip under csrc/ and link

The library is placed next to this file so that it is found without installation.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
OBJ_DIR = CSRC / "build"
LIB_PATH = PKG_DIR / "libdaphne_hip.so"

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # keep hipcc from forming packed-fp32 instructions out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libdaphne_hip.so cannot be built")
    return exe


def _compile(src: Path) -> Path:
    obj = OBJ_DIR / (src.stem + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{proc.stderr}")
    return obj


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def build_all(jobs: int | None = None, verbose: bool = True) -> Path:
    """Compiles every translation unit and links the shared library. Always recompiles."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), max(1, (os.cpu_count() or 2)), 16)
    if verbose:
        print(f"[daphne_amd.build] compiling {len(srcs)} files with hipcc for gfx950 ({jobs} jobs)", flush=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, srcs))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB_PATH), *map(str, objs)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    if verbose:
        print(f"[daphne_amd.build] wrote {LIB_PATH}", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build_all()
    sys.exit(0)
