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


def test_two_host_threads_share_one_context():
    """The reference calls device kernels from its main thread, its CPU workers and its device worker
    (src/runtime/local/vectorized/MTWrapper.h:94-98). Two threads on ONE context each allocate, run a checked unary
    operator (domain flag), a column and a full aggregation (workspace, scalar slot) of their own data and free
    again, many times over; every result must be the thread's own, compared with the CPU oracle."""
    import threading

    import oracle_binding as orc
    from daphne_amd.kernels import AggOpCode, UnaryOpCode, aggAll, aggCol, ewUnaryMat
    from parity import assert_close

    c = HIPContext(0)
    errors = []

    def worker(seed, rows, cols, poison):
        try:
            rng = np.random.default_rng(seed)
            x = (rng.random((rows, cols)) * (seed + 1) + 0.5).astype(np.float32)
            _, sq_e = orc.ew_unary(UnaryOpCode.SQRT, x)
            _, col_e = orc.agg_col(AggOpCode.SUM, x)
            _, all_e = orc.agg_all(AggOpCode.MAX, x)
            bad = x.copy()
            bad[rows // 2, cols // 3] = -1.0
            for it in range(40):
                X = DenseMatrix.from_numpy(c, x)
                np.testing.assert_array_equal(ewUnaryMat(UnaryOpCode.SQRT, None, X, c).to_numpy(), sq_e)
                assert_close(aggCol(AggOpCode.SUM, None, X, c).to_numpy(), col_e)
                assert aggAll(AggOpCode.MAX, X, c) == all_e
                if poison and it % 4 == 0:
                    # this thread's domain error must never surface in the other thread's call
                    with pytest.raises(capi.DaphneHipDomainError):
                        ewUnaryMat(UnaryOpCode.SQRT, None, DenseMatrix.from_numpy(c, bad), c)
                del X
        except BaseException as e:  # noqa: BLE001 - reported by the main thread
            errors.append((seed, repr(e)))

    ts = [threading.Thread(target=worker, args=(1, 3000, 64, True)), threading.Thread(target=worker, args=(2, 50001, 7, False))]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    assert not errors, errors
    c.sync()
    assert c.memInUse() == 0
    c.destroy()


def test_pitched_copies_between_device_and_host():
    """dh_d2d_2d and dh_d2h_2d move `rows` pieces of `width` bytes between buffers with their own row pitches: a
    pipeline's row or column share on its way into the whole result (TasksCUDA.cpp:73-100, MTWrapper_dense.cpp:339-373)."""
    c = HIPContext(0)
    lib = capi.lib()
    rows, width, sp, dp, hp = 37, 24, 40, 56, 64
    src = np.arange(rows * sp, dtype=np.uint8)
    d_src, d_dst = c.malloc(src.nbytes), c.malloc(rows * dp, zero=True)
    capi.check(lib.dh_h2d(c._h, d_src, src.ctypes.data, src.nbytes))
    capi.check(lib.dh_d2d_2d(c._h, d_dst, dp, d_src, sp, width, rows))
    host = np.full(rows * hp, 255, dtype=np.uint8)
    capi.check(lib.dh_d2h_2d(c._h, host.ctypes.data, hp, d_dst, dp, width, rows))
    want = np.full((rows, hp), 255, dtype=np.uint8)
    want[:, :width] = src.reshape(rows, sp)[:, :width]
    np.testing.assert_array_equal(host.reshape(rows, hp), want)
    tight = np.empty(rows * width, dtype=np.uint8)  # both pitches equal to the width: one plain copy
    packed = c.malloc(rows * width)
    capi.check(lib.dh_d2d_2d(c._h, packed, width, d_src, sp, width, rows))
    capi.check(lib.dh_d2h_2d(c._h, tight.ctypes.data, width, packed, width, width, rows))
    np.testing.assert_array_equal(tight.reshape(rows, width), want[:, :width])
    with pytest.raises(DaphneHipError):
        capi.check(lib.dh_d2h_2d(c._h, host.ctypes.data, width - 1, d_dst, dp, width, rows))
    for p in (d_src, d_dst, packed):
        c.free(p)
    c.destroy()
