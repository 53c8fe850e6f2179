"""CPU: the DAPHNE-side sources that cannot be compiled here are at least consistent with the reference tree, where
that tree is present (it is not on the GPU box): every patch applies, and the members of DAPHNE's data objects that
the kernel layer calls exist there under the same names as in the stand-in headers."""
import re
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
CPP = ROOT / "daphne_amd" / "cpp"
REF = Path("/root/reference")
needs_reference = pytest.mark.skipif(not (REF / "src").is_dir(), reason="the reference tree is not present")


@needs_reference
def test_patches_apply_to_the_reference_tree(tmp_path):
    patches = sorted((CPP / "patches").glob("*.patch"))
    assert len(patches) >= 11
    for p in patches:
        for line in p.read_text().splitlines():
            if line.startswith("--- a/"):
                rel = line[len("--- a/"):]
                (tmp_path / rel).parent.mkdir(parents=True, exist_ok=True)
                if not (tmp_path / rel).exists():
                    shutil.copy(REF / rel, tmp_path / rel)
    for p in patches:
        r = subprocess.run(["patch", "-p1", "--fuzz=0", "-s", "-i", str(p)], cwd=tmp_path, capture_output=True, text=True)
        assert r.returncode == 0, f"{p.name}: {r.stdout}{r.stderr}"
    assert 'backend = "HIP"' in (tmp_path / "src/compiler/lowering/RewriteToCallKernelOpPass.cpp").read_text()
    assert "hip_contexts" in (tmp_path / "src/runtime/local/context/DaphneContext.h").read_text()


@needs_reference
def test_standins_use_the_reference_member_names():
    ds = REF / "src/runtime/local/datastructures"
    dense = (ds / "DenseMatrix.h").read_text() + (ds / "Structure.h").read_text()
    for member in ("getNumRows", "getNumCols", "getRowSkip", "getNumItems", "getBufferSize", "getValues", "sliceRow", "sliceCol",
                   "slice", "increaseRefCounter", "getMetaDataObject"):
        assert re.search(rf"\b{member}\s*\(", dense), member
    alloc = (ds / "IAllocationDescriptor.h").read_text()
    for member in ("getType", "createAllocation", "getLocation", "getData", "transferTo", "transferFrom", "clone", "GPU_HIP"):
        assert member in alloc, member
    mdo = (ds / "MetaDataObject.h").read_text()
    for member in ("addDataPlacement", "findDataPlacementByType", "getDataPlacementByID", "isLatestVersion", "addLatest", "setLatest",
                   "getLatest"):
        assert member in mdo, member
    tasks = (REF / "src/runtime/local/vectorized/Tasks.h").read_text()
    for member in ("_funcs", "_isScalar", "_inputs", "_numInputs", "_numOutputs", "_outRows", "_outCols", "_splits", "_combines",
                   "_rl", "_ru", "_offset", "_ctx", "createFuncInputs"):
        assert member in tasks, member
    ctx = (REF / "src/runtime/local/context/DaphneContext.h").read_text()
    for member in ("getUserConfig", "dispatchMapping", "startKernelTimer", "stopKernelTimer", "cuda_contexts"):
        assert member in ctx, member


def test_overlay_holds_the_files_the_readme_names():
    src = CPP / "src"
    for rel in ("runtime/local/context/HIPContext.h", "runtime/local/datastructures/AllocationDescriptorHIP.h",
                "runtime/local/vectorized/TasksHIP.h", "runtime/local/kernels/HIP/VectorizedPipeline.h",
                "runtime/local/kernels/HIP/HIPkernels.json", "runtime/local/kernels/HIP/genHIPKernelInst.py",
                "compiler/lowering/MarkHIPOpsPass.cpp"):
        assert (src / rel).is_file(), rel
    # every header the specification names exists
    import json

    for k in json.loads((src / "runtime/local/kernels/HIP/HIPkernels.json").read_text()):
        assert (src / "runtime/local/kernels/HIP" / k["kernelTemplate"]["header"]).is_file(), k["kernelTemplate"]["header"]
