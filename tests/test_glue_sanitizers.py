"""CPU: the C++ kernel layer's placement, task and shared-pipeline tests (tests/cpp/placement_and_tasks.h) over the
stand-in data structures and tests/cpp/mock_daphne_hip.cpp, a host-memory implementation of the C ABI, built with the
host compiler's thread sanitizer and with its address / undefined-behaviour sanitizers. The pipeline shared between a
device worker and CPU workers (MTWrapperHIP.h, WorkerHIP.h) is the part with threads in it: its workers, queues and the
placement records they touch must come through without a report. Skipped where the sanitizer run-times are missing."""
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
CPP = ROOT / "daphne_amd" / "cpp"
INCLUDES = [f"-I{CPP}", f"-I{CPP / 'src'}", f"-I{CPP / 'standalone' / 'context'}", f"-I{CPP / 'standalone' / 'data'}",
            f"-I{ROOT / 'include'}", f"-I{ROOT / 'tests' / 'cpp'}"]
SOURCES = [str(ROOT / "tests" / "cpp" / "test_glue_reference.cpp"), str(ROOT / "tests" / "cpp" / "mock_daphne_hip.cpp")]


@pytest.mark.parametrize("sanitizer", ["thread", "address,undefined"])
def test_kernel_layer_under_sanitizers(tmp_path, sanitizer):
    exe = tmp_path / "glue_sanitized"
    build = subprocess.run(["g++", "-std=c++17", "-O1", "-g", f"-fsanitize={sanitizer}", "-fno-sanitize-recover=all", *INCLUDES,
                            "-o", str(exe), *SOURCES], capture_output=True, text=True)
    if build.returncode != 0 and ("sanitizer" in build.stderr.lower() or "cannot find -l" in build.stderr):
        pytest.skip("the host compiler has no run-time for -fsanitize=" + sanitizer)
    assert build.returncode == 0, build.stderr[-4000:]
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=600)
    assert run.returncode == 0 and "PASSED" in run.stdout, run.stdout[-3000:] + run.stderr[-3000:]
    assert "WARNING: ThreadSanitizer" not in run.stderr and "ERROR: AddressSanitizer" not in run.stderr, run.stderr[-4000:]
