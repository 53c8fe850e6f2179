"""Builds the host-compiled test programs over the C++ kernel layer: the glue test binary and the harness library
that lets pytest make run-time objects for the generated kernel entry points. __graft_entry__.build() calls these;
tests call them only when the built files are missing."""
import subprocess
from pathlib import Path

from daphne_amd import build as b

ROOT = Path(__file__).resolve().parent.parent
OUT = ROOT / "tests" / "cpp" / "build"
GLUE_BIN = OUT / "test_glue"
HARNESS_LIB = OUT / "libglue_harness.so"
BUILDER_BIN = OUT / "test_pipeline_builder"


def _link_flags():
    return [f"-L{b.PKG_DIR}", "-ldaphne_hip", "-Wl,-rpath,$ORIGIN/../../../daphne_amd"]


def build_glue_test() -> Path:
    OUT.mkdir(parents=True, exist_ok=True)
    subprocess.run(["g++", *b.HOST_CXX_FLAGS, "-o", str(GLUE_BIN), str(ROOT / "tests" / "cpp" / "test_glue.cpp"),
                    *_link_flags(), "-ldl"], check=True)
    return GLUE_BIN


def build_harness() -> Path:
    OUT.mkdir(parents=True, exist_ok=True)
    subprocess.run(["g++", *b.HOST_CXX_FLAGS, "-fPIC", "-shared", "-o", str(HARNESS_LIB),
                    str(ROOT / "tests" / "cpp" / "glue_harness.cpp"), *_link_flags()], check=True)
    return HARNESS_LIB


def build_builder_test() -> Path:
    """Host-only: the pipeline-body lowering needs neither the device library nor a device."""
    OUT.mkdir(parents=True, exist_ok=True)
    subprocess.run(["g++", *b.HOST_CXX_FLAGS, "-o", str(BUILDER_BIN), str(ROOT / "tests" / "cpp" / "test_pipeline_builder.cpp")],
                   check=True)
    return BUILDER_BIN
