"""Device context and allocator (the counterpart of CUDAContext, src/runtime/local/context/CUDAContext.cpp:41-135):
budget, registry, zero-initialisation, block reuse, and that reuse in stream order never corrupts results."""
import numpy as np
import pytest

from daphne_amd import capi
from daphne_amd.capi import DaphneHipError
from daphne_amd.kernels import BinaryOpCode, DenseMatrix, HIPContext, ewBinaryObjSca

pytestmark = pytest.mark.gpu


def test_budget_is_ninety_percent_of_device_memory():
    c = HIPContext(0)
    total = c.props()["total_mem"]
    assert c.getMemBudget() == int(total * 0.9) or abs(c.getMemBudget() - total * 0.9) < 2  # CUDAContext.cpp:49-50
    assert c.memInUse() == 0
    c.destroy()


def test_malloc_zero_registry_and_reuse():
    c = HIPContext(0)
    p = c.malloc(1 << 20, zero=True)
    assert c.memInUse() == 1 << 20
    host = np.ones(1 << 20, dtype=np.uint8)
    capi.check(capi.lib().dh_d2h(c._h, host.ctypes.data, p, 1 << 20))
    assert not host.any()
    c.free(p)
    assert c.memInUse() == 0 and c.memCached() >= 1 << 20
    q = c.malloc((1 << 20) - 100)  # same size class: the cached block comes back
    assert q == p and c.memCached() == 0
    c.free(q)
    c.releaseCached()
    assert c.memCached() == 0
    with pytest.raises(DaphneHipError):
        c.free(12345)  # not a pointer of this context
    with pytest.raises(DaphneHipError):
        c.malloc(c.getMemBudget() + 1)
    z = c.malloc(0)  # distinct non-null key for an empty object
    assert z != 0
    c.free(z)
    c.destroy()


def test_reused_blocks_keep_results_intact():
    """A chain of temporaries that are freed while the kernels reading them may still be queued."""
    c = HIPContext(0)
    x = np.arange(1 << 18, dtype=np.float32).reshape(512, 512)
    cur = DenseMatrix.from_numpy(c, x)
    for i in range(50):
        nxt = ewBinaryObjSca(BinaryOpCode.ADD, None, cur, 1.0, c)
        del cur  # its block returns to the cache at once and is handed out again two steps later
        cur = nxt
    np.testing.assert_array_equal(cur.to_numpy(), x + 50.0)
    c.destroy()
