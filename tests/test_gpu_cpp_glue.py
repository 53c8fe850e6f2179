"""GPU: the C++ kernel layer (daphne_amd/cpp: namespace HIP with the reference's Kernel<...>::apply signatures, the
device context, the allocation descriptor, the vectorized-pipeline task) run as a plain host-compiled program over
the reference's own test vectors, plus the generated entry points of libHIPKernels.so called through dlsym.
The binary is built by __graft_entry__.build(); it is only compiled here if missing."""
import subprocess

import pytest

import cpp_build
from daphne_amd import build as b


@pytest.mark.gpu
def test_cpp_kernel_layer_on_reference_vectors():
    if not cpp_build.GLUE_BIN.exists():
        cpp_build.build_glue_test()
    if not b.KERNEL_LIB_PATH.exists():
        b.build_kernel_library(verbose=False)
    p = subprocess.run([str(cpp_build.GLUE_BIN), str(b.KERNEL_LIB_PATH)], capture_output=True, text=True, timeout=300)
    print(p.stdout, p.stderr)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "PASSED" in p.stdout


def test_cpp_kernel_layer_compiles_with_a_host_compiler():
    """No HIP header is needed above the C ABI: g++ alone compiles the kernel layer, its test and the harness."""
    for src in ("test_glue.cpp", "glue_harness.cpp"):
        subprocess.run(["g++", *b.HOST_CXX_FLAGS, "-fsyntax-only", "-Werror", str(cpp_build.ROOT / "tests" / "cpp" / src)], check=True)
