"""CPU, build container only: the C++ kernel layer against the reference's REAL data structures.

tests/cpp/test_glue_reference.cpp (the placement and vectorized-pipeline tests that `test_glue` runs on the GPU over the
stand-in data structures) is compiled here against the reference's own datastructures/{DenseMatrix, MetaDataObject,
DataPlacement, Structure}.cpp - copied to a temporary directory with patches/0011-dense-matrix-device-views.patch
applied - and linked with tests/cpp/mock_daphne_hip.cpp, a host-memory implementation of the C ABI. Headers of the
reference that need MLIR or libraries this image lacks are shadowed: the context side by the stand-in
(daphne_amd/cpp/standalone/context), spdlog / fmt / DaphneSerializer by the three files of tests/cpp/reference_shim.
This is a type-and-semantics check of product glue, not an oracle. Skipped where /root/reference is absent.
"""
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
CPP = ROOT / "daphne_amd" / "cpp"
REF = Path("/root/reference")
DS = "src/runtime/local/datastructures"
pytestmark = pytest.mark.skipif(not (REF / DS).is_dir(), reason="the reference tree is not present")

SOURCES = ["DenseMatrix.cpp", "MetaDataObject.cpp", "DataPlacement.cpp", "Structure.cpp", "ValueTypeUtils.cpp"]


def _includes(patched_src: Path):
    return [f"-I{ROOT / 'tests' / 'cpp' / 'reference_shim'}", f"-I{CPP / 'standalone' / 'context'}", f"-I{patched_src}",
            f"-I{REF / 'src'}", f"-I{CPP / 'src'}", f"-I{ROOT / 'include'}", f"-I{ROOT / 'tests' / 'cpp'}"]


def _patched_copy(tmp_path: Path, apply_patch: bool) -> Path:
    """A src/ tree holding the reference's data-structure directory (its files include each other by relative paths, so
    the whole directory travels), with or without the patch."""
    patch = CPP / "patches" / "0011-dense-matrix-device-views.patch"
    shutil.copytree(REF / DS, tmp_path / DS)
    if apply_patch:
        r = subprocess.run(["patch", "-p1", "--fuzz=0", "-s", "-i", str(patch)], cwd=tmp_path, capture_output=True, text=True)
        assert r.returncode == 0, r.stdout + r.stderr
    return tmp_path / "src"


def _build_and_run(tmp_path: Path, src: Path):
    flags = ["-std=c++20", "-O1", "-Wall", "-Wno-unused-parameter", *_includes(src)]
    objs = []
    for name in SOURCES:
        patched = src / "runtime/local/datastructures" / name
        source = patched if patched.exists() else REF / DS / name
        obj = tmp_path / (name + ".o")
        r = subprocess.run(["g++", *flags, "-c", str(source), "-o", str(obj)], capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-4000:]
        objs.append(str(obj))
    exe = tmp_path / "test_glue_reference"
    r = subprocess.run(["g++", *flags, "-o", str(exe), str(ROOT / "tests/cpp/test_glue_reference.cpp"),
                        str(ROOT / "tests/cpp/mock_daphne_hip.cpp"), *objs], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-6000:]
    return subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)


def test_kernel_layer_on_the_reference_data_structures(tmp_path):
    r = _build_and_run(tmp_path, _patched_copy(tmp_path, True))
    assert r.returncode == 0 and "PASSED" in r.stdout, r.stdout[-4000:] + r.stderr[-2000:]


def test_the_checks_notice_views_that_yield_their_parents_base(tmp_path):
    """The unpatched reference hands out the allocation's base for an inherited placement (DenseMatrix.cpp:176-182).
    Taking the offset back out of the patched sources must make the share / batch and view checks fail: the test
    above is only worth something if it does."""
    src = _patched_copy(tmp_path, True)
    cpp = src / "runtime/local/datastructures/DenseMatrix.cpp"
    text = cpp.read_text()
    assert text.count(" + offsetIn(placement->dp_id);") == 1
    cpp.write_text(text.replace(" + offsetIn(placement->dp_id);", ";"))
    r = _build_and_run(tmp_path, src)
    assert r.returncode != 0 and "FAILED" in r.stdout
    assert "placement_and_tasks.h" in r.stdout


def test_tasks_refuse_to_compile_on_unpatched_views(tmp_path):
    """Without the patch every view yields its parent's device base (DenseMatrix.cpp:176-182): the task header must not build."""
    src = _patched_copy(tmp_path, False)
    flags = ["-std=c++20", "-fsyntax-only", *_includes(src)]
    probe = tmp_path / "probe.cpp"
    probe.write_text("#include <runtime/local/vectorized/TasksHIP.h>\nint main() { return 0; }\n")
    r = subprocess.run(["g++", *flags, str(probe)], capture_output=True, text=True)
    assert r.returncode != 0
    assert "0011-dense-matrix-device-views.patch" in r.stderr
