"""GPU: the C++ kernel interface (daphne_amd/cpp/daphne_hip_kernels.h, namespace HIP, the reference's
Kernel<...>::apply signatures) run as a plain host-compiled program over the reference's own test
vectors. The binary is built by __graft_entry__.build(); it is only compiled here if missing."""
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
BIN = ROOT / "tests" / "cpp" / "build" / "test_glue"


def build_glue_test():
    BIN.parent.mkdir(parents=True, exist_ok=True)
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-o", str(BIN), str(ROOT / "tests" / "cpp" / "test_glue.cpp"),
                    f"-L{ROOT / 'daphne_amd'}", "-ldaphne_hip", "-Wl,-rpath,$ORIGIN/../../../daphne_amd"], check=True)


@pytest.mark.gpu
def test_cpp_kernel_interface_on_reference_vectors():
    if not BIN.exists():
        build_glue_test()
    p = subprocess.run([str(BIN)], capture_output=True, text=True, timeout=300)
    print(p.stdout, p.stderr)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "PASSED" in p.stdout


def test_cpp_kernel_interface_compiles_with_a_host_compiler(tmp_path):
    """No HIP header is needed above the C ABI: g++ alone compiles the interface and its test."""
    out = tmp_path / "glue.o"
    subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-Werror", str(ROOT / "tests" / "cpp" / "test_glue.cpp")],
                   check=True)
    assert not out.exists()
