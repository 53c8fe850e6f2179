"""Builds libdaphne_hip.so (gfx950 only) with hipcc, and on top of it libHIPKernels.so, the generated
`HIP_<mnemonic>__<types>` entry points that DAPHNE's compiled programs call, with its catalog. No GPU is needed to build.

    python -m daphne_amd.build          # compile every .hip under csrc/ and link, then the kernel library

libdaphne_hip.so is placed next to this file so that it is found without installation; libHIPKernels.so and
HIPcatalog.json go to cpp/lib/ (the catalog names the library by a path relative to itself).
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
CPP_DIR = PKG_DIR / "cpp"
KERNEL_SRC_DIR = CPP_DIR / "src" / "runtime" / "local" / "kernels" / "HIP"
KERNEL_SPEC = KERNEL_SRC_DIR / "HIPkernels.json"
KERNEL_GENERATOR = KERNEL_SRC_DIR / "genHIPKernelInst.py"
KERNEL_LIB_DIR = CPP_DIR / "lib"
KERNEL_LIB_PATH = KERNEL_LIB_DIR / "libHIPKernels.so"
KERNEL_CATALOG_PATH = KERNEL_LIB_DIR / "HIPcatalog.json"
# host-side C++ of the kernel layer: DAPHNE's include paths, served here by the stand-in headers (two roots: what
# stands in for DAPHNE's MLIR-dependent context headers, and what stands in for its data structures)
HOST_CXX_FLAGS = ["-std=c++17", "-O1", "-Wall", f"-I{CPP_DIR}", f"-I{CPP_DIR / 'src'}", f"-I{CPP_DIR / 'standalone' / 'context'}",
                  f"-I{CPP_DIR / 'standalone' / 'data'}",
                  f"-I{PKG_DIR.parent / 'include'}"]

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


# The interpreting pipeline kernel rounds every operator of a body by itself, like the run-time specialised one.
EXTRA_FLAGS = {"pipeline_f32.hip": ["-ffp-contract=off"], "pipeline_f64.hip": ["-ffp-contract=off"]}
# The symmetric streaming kernel and the widest step of the double `A t(B)` kernel keep their accumulators in ordinary
# vector registers: with the matrix instructions in their accumulator-register form the compiler carries the former's
# accumulators through the loop in vector registers all the same and copies all of them over and back in every
# iteration, and parks the latter's loaded rows in accumulator registers.
for _f in ("ts_sym_f32.hip", "ts_sym_f64.hip", "ts_nt_wide_f64.hip"):
    EXTRA_FLAGS[_f] = ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]


def _compile(src: Path) -> Path:
    obj = OBJ_DIR / (src.stem + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *EXTRA_FLAGS.get(src.name, []), "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{proc.stderr}")
    return obj


JIT_PRELUDE = """// generated: sources compiled at run time (hiprtc) for fused pipeline bodies
typedef __SIZE_TYPE__ size_t;
typedef __INT32_TYPE__ int32_t;
typedef __UINT32_TYPE__ uint32_t;
typedef __INT64_TYPE__ int64_t;
typedef __UINT64_TYPE__ uint64_t;
"""


def generate_jit_sources() -> Path:
    """Embeds the public header and the device headers of the pipeline kernel as one string."""
    parts = [JIT_PRELUDE]
    for f in (PKG_DIR.parent / "include" / "daphne_hip.h", CSRC / "dev_common.h", CSRC / "ew_ops.h",
              CSRC / "pipeline_kernel.h"):
        for line in f.read_text().splitlines():
            if line.startswith("#include") or line.startswith("#pragma once"):
                continue
            parts.append(line)
    text = "\n".join(parts)
    if ')DHJIT"' in text:
        raise RuntimeError("embedded source contains the raw-string delimiter")
    # split into chunks: some compilers cap the length of a single literal
    chunks, step = [], 12000
    for i in range(0, len(text), step):
        chunks.append('R"DHJIT(' + text[i:i + step] + ')DHJIT"')
    out = OBJ_DIR / "jit_sources.inc"
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    out.write_text("static const char kJitEmbeddedSource[] =\n" + "\n".join(chunks) + ";\n")
    return out


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def build_all(jobs: int | None = None, verbose: bool = True) -> Path:
    """Compiles every translation unit and links the shared library. Always recompiles."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    generate_jit_sources()
    srcs = sources()
    jobs = jobs or min(len(srcs), max(1, (os.cpu_count() or 2)), 16)
    if verbose:
        print(f"[daphne_amd.build] compiling {len(srcs)} files with hipcc for gfx950 ({jobs} jobs)", flush=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, srcs))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB_PATH), *map(str, objs), "-lhiprtc"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    if verbose:
        print(f"[daphne_amd.build] wrote {LIB_PATH}", flush=True)
    return LIB_PATH


def generate_kernel_sources() -> Path:
    """Runs the generator: cpp/build/HIPkernels.cpp and cpp/lib/HIPcatalog.json from HIPkernels.json."""
    out_cpp = CPP_DIR / "build" / "HIPkernels.cpp"
    proc = subprocess.run([sys.executable, str(KERNEL_GENERATOR), str(KERNEL_SPEC), str(out_cpp), str(KERNEL_CATALOG_PATH), "HIP"],
                          capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"kernel generator failed:\n{proc.stdout}{proc.stderr}")
    return out_cpp


def build_kernel_library(verbose: bool = True) -> Path:
    """libHIPKernels.so: the generated entry points over the C++ kernel layer, compiled by the host compiler."""
    out_cpp = generate_kernel_sources()
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        raise RuntimeError("no host C++ compiler found; libHIPKernels.so cannot be built")
    cmd = [cxx, *HOST_CXX_FLAGS, "-fPIC", "-shared", str(out_cpp), "-o", str(KERNEL_LIB_PATH), f"-L{PKG_DIR}", "-ldaphne_hip",
           "-Wl,-rpath,$ORIGIN/../.."]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"compiling the kernel library failed:\n{proc.stderr}")
    if verbose:
        print(f"[daphne_amd.build] wrote {KERNEL_LIB_PATH} and {KERNEL_CATALOG_PATH}", flush=True)
    return KERNEL_LIB_PATH


if __name__ == "__main__":
    build_all()
    build_kernel_library()
    sys.exit(0)
