"""CPU: the oracle reproduces every known-answer vector of the reference's own kernel unit tests."""
import numpy as np
import pytest

import golden_cases as gc
from backends import OracleBackend

CHECKS = list(gc.all_checks())


@pytest.mark.parametrize("dt", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("cid,f,c,k", CHECKS, ids=[c[0] for c in CHECKS])
def test_oracle_matches_reference_vectors(cid, f, c, k, dt):
    try:
        gc.run(OracleBackend(), f, c, k, dt)
    except gc.Skip as e:
        pytest.skip(str(e))


def test_golden_file_covers_the_kernel_set():
    ran = {}
    for cid, f, c, k in CHECKS:
        try:
            gc.run(OracleBackend(), f, c, k, np.float64)
            ran[f["file"]] = ran.get(f["file"], 0) + 1
        except gc.Skip:
            pass
    for must in ("EwBinaryMatTest.cpp", "EwBinaryObjScaTest.cpp", "EwUnaryMatTest.cpp", "AggAllTest.cpp",
                 "AggRowTest.cpp", "AggColTest.cpp", "MatMulTest.cpp", "CUDA/MatMulTest.cpp", "SyrkTest.cpp",
                 "SolveTest.cpp", "SoftmaxTest.cpp", "DNNConv2DForwardTest.cpp", "DNNPoolingTestForward.cpp",
                 "DNNBiasAddForwardTest.cpp", "DNNBatchNorm2DForwardTest.cpp", "CUDA/DNNAffineTest.cpp",
                 "CUDA/BiasAddTest.cpp", "CUDA/DNNBatchNormTest.cpp", "CUDA/DNNConvolutionTest.cpp",
                 "CUDA/DNNSoftmaxTest.cpp", "CUDA/DNNActivationTest.cpp", "TransposeTest.cpp", "ColBindTest.cpp",
                 "ExtractColTest.cpp"):
        assert ran.get(must, 0) > 0, f"no vector of {must} was replayed"


@pytest.mark.parametrize("dt", [np.int64, np.uint64, np.int32, np.uint32], ids=["si64", "ui64", "si32", "ui32"])
@pytest.mark.parametrize("cid,f,c,k", CHECKS, ids=[c[0] for c in CHECKS])
def test_oracle_matches_reference_vectors_for_integers(cid, f, c, k, dt):
    """The reference runs these tests with integer value types too (VALUE_TYPES in EwBinaryMatTest.cpp:34,
    AggAllTest.cpp:32, AggRowTest.cpp:33 ...): literals that are integers of the type are replayed with it."""
    try:
        gc.run(OracleBackend(), f, c, k, dt)
    except gc.Skip as e:
        pytest.skip(str(e))
