"""GPU: the HIP kernels reproduce every known-answer vector of the reference's own kernel unit tests."""
import numpy as np
import pytest

import golden_cases as gc
from backends import HipBackend

pytestmark = pytest.mark.gpu
CHECKS = list(gc.all_checks())


@pytest.mark.parametrize("dt", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("cid,f,c,k", CHECKS, ids=[c[0] for c in CHECKS])
def test_hip_matches_reference_vectors(ctx, cid, f, c, k, dt):
    try:
        gc.run(HipBackend(ctx), f, c, k, dt)
    except gc.Skip as e:
        pytest.skip(str(e))


@pytest.mark.parametrize("dt", [np.int64, np.uint64, np.int32, np.uint32], ids=["si64", "ui64", "si32", "ui32"])
@pytest.mark.parametrize("cid,f,c,k", CHECKS, ids=[c[0] for c in CHECKS])
def test_hip_matches_reference_vectors_for_integers(ctx, cid, f, c, k, dt):
    """The reference runs these tests with integer value types too (VALUE_TYPES in EwBinaryMatTest.cpp:34,
    AggAllTest.cpp:32, AggRowTest.cpp:33 ...): literals that are integers of the type are replayed with it."""
    try:
        gc.run(HipBackend(ctx), f, c, k, dt)
    except gc.Skip as e:
        pytest.skip(str(e))
