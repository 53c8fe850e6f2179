"""CPU: HIP::PipelineProgramBuilder lowers the operator list of a pipeline's device body (text, DaphneIR mnemonics) to the
instruction list of the fused pipeline kernel, or says why a body does not fit. The checks are in
tests/cpp/test_pipeline_builder.cpp (host compiler only, no device library)."""
import subprocess

import cpp_build


def test_pipeline_program_builder():
    exe = cpp_build.BUILDER_BIN
    if not exe.exists():
        cpp_build.build_builder_test()
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0 and "PASSED" in r.stdout, r.stdout + r.stderr
