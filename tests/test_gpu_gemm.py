"""GPU parity: MatMul / Syrk / Solve / Affine (through the C ABI) against the CPU oracle.

Tolerance: norm-wise relative error max|got - exp| / max|exp| <= 1e-4 (float) / 1e-10 (double):
the reference's BLAS and the MFMA kernels sum in different orders, so single entries that are
sums with heavy cancellation cannot be compared relative to themselves. Integer-valued inputs
(every partial sum exactly representable) must match bit for bit in any order.
"""
import numpy as np
import pytest

import oracle_binding as orc
from parity import assert_close, assert_exact

pytestmark = pytest.mark.gpu

from daphne_amd import capi
from daphne_amd.kernels import (AggOpCode, BinaryOpCode, DenseMatrix, affineForward, affineForwardFused, aggRow, ewBinaryMat,
                                ewBinaryObjSca, kmeansAssign, kmeansStep, kmeansUpdate, matMul, reluForward, solve, syrk)

DTYPES = [np.float32, np.float64]

SHAPES = [  # (m, n, k)
    (1, 1, 1), (3, 5, 7), (16, 16, 16), (33, 17, 65), (128, 128, 128), (129, 127, 130), (200, 300, 50),
    (256, 32, 64), (1000, 16, 64), (16, 64, 3000), (20, 300, 40), (5, 5, 20000), (260, 7, 9), (384, 512, 640),
    (64, 800, 5000), (40, 513, 300), (800, 64, 5000), (513, 33, 100),  # 64 x 256 and 256 x 64 tiles, with and without split-K
]


def _stored(rng, r, c, dt, trans):
    a = (rng.random((c, r) if trans else (r, c)) * 2 - 1).astype(dt)
    return a


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("m,n,k", SHAPES)
def test_matmul_random(ctx, dt, ta, tb, m, n, k):
    rng = np.random.default_rng(m * 1000003 + n * 1009 + k)
    a, b = _stored(rng, m, k, dt, ta), _stored(rng, k, n, dt, tb)
    st, exp = orc.matmul(a, b, ta, tb)
    assert st == 0
    truth = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
    got = matMul(None, DenseMatrix.from_numpy(ctx, a), DenseMatrix.from_numpy(ctx, b), ta, tb, ctx).to_numpy()
    assert got.shape == (m, n)
    assert_close(got, exp, elementwise=False)
    assert_close(got, truth.astype(dt), elementwise=False)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_matmul_integer_valued_exact(ctx, dt, ta, tb):
    rng = np.random.default_rng(1)
    for (m, n, k) in [(37, 41, 53), (130, 140, 300), (8, 8, 5000), (300, 20, 64)]:
        a = rng.integers(-4, 5, (k, m) if ta else (m, k)).astype(dt)
        b = rng.integers(-4, 5, (n, k) if tb else (k, n)).astype(dt)
        exp = ((a.T if ta else a).astype(np.int64) @ (b.T if tb else b).astype(np.int64)).astype(dt)
        got = matMul(None, DenseMatrix.from_numpy(ctx, a), DenseMatrix.from_numpy(ctx, b), ta, tb, ctx).to_numpy()
        assert_exact(got, exp)
        assert_exact(orc.matmul(a, b, ta, tb)[1], exp)


@pytest.mark.parametrize("dt", DTYPES)
def test_matmul_views(ctx, dt):
    """rowSkip > numCols on lhs, rhs and res (kernels/MatMul.cpp:269-271 passes rowSkip as ld)."""
    rng = np.random.default_rng(2)
    A = (rng.random((90, 77)) - 0.5).astype(dt)
    B = (rng.random((80, 66)) - 0.5).astype(dt)
    dA, dB = DenseMatrix.from_numpy(ctx, A), DenseMatrix.from_numpy(ctx, B)
    va, vb = A[5:70, 3:60], B[10:67, 1:50]  # 65x57 @ 57x49
    res = DenseMatrix(ctx, 100, 60, dt, zero=True)
    matMul(res.slice(7, 72, 2, 51), dA.slice(5, 70, 3, 60), dB.slice(10, 67, 1, 50), False, False, ctx)
    full = res.to_numpy()
    assert_close(full[7:72, 2:51], orc.matmul(va, vb)[1], elementwise=False)
    full[7:72, 2:51] = 0
    assert (full == 0).all(), "wrote outside the result view"
    # unaligned leading dimensions / odd offsets with transposes
    got = matMul(None, dA.slice(5, 62, 3, 68), dB.slice(10, 67, 1, 50), True, False, ctx).to_numpy()
    assert_close(got, orc.matmul(A[5:62, 3:68], vb, True, False)[1], elementwise=False)


@pytest.mark.parametrize("dt", DTYPES)
def test_matmul_vectors(ctx, dt):
    """matrix-vector and vector-vector shapes (kernels/MatMul.cpp:277-283)."""
    rng = np.random.default_rng(3)
    A = (rng.random((500, 70)) - 0.5).astype(dt)
    x = (rng.random((70, 1)) - 0.5).astype(dt)
    y = (rng.random((500, 1)) - 0.5).astype(dt)
    dA = DenseMatrix.from_numpy(ctx, A)
    assert_close(matMul(None, dA, DenseMatrix.from_numpy(ctx, x), False, False, ctx).to_numpy(), orc.matmul(A, x)[1],
                 elementwise=False)
    assert_close(matMul(None, dA, DenseMatrix.from_numpy(ctx, y), True, False, ctx).to_numpy(),
                 orc.matmul(A, y, True, False)[1], elementwise=False)
    xr = np.ascontiguousarray(x.T)
    assert_close(matMul(None, dA, DenseMatrix.from_numpy(ctx, xr), False, True, ctx).to_numpy(),
                 orc.matmul(A, xr, False, True)[1], elementwise=False)
    # dot products
    u = (rng.random((1, 3000)) - 0.5).astype(dt)
    v = (rng.random((3000, 1)) - 0.5).astype(dt)
    got = matMul(None, DenseMatrix.from_numpy(ctx, u), DenseMatrix.from_numpy(ctx, v), False, False, ctx).to_numpy()
    assert got.shape == (1, 1)
    assert_close(got, (u.astype(np.float64) @ v.astype(np.float64)).astype(dt), rtol=1e-4 if dt == np.float32 else 1e-10,
                 elementwise=False)
    got = matMul(None, DenseMatrix.from_numpy(ctx, v), DenseMatrix.from_numpy(ctx, v), True, False, ctx).to_numpy()
    assert_close(got, (v.T.astype(np.float64) @ v.astype(np.float64)).astype(dt), elementwise=False)


@pytest.mark.parametrize("dt", DTYPES)
def test_matmul_shape_error(ctx, dt):
    a = DenseMatrix.from_numpy(ctx, np.ones((4, 5), dt))
    b = DenseMatrix.from_numpy(ctx, np.ones((4, 5), dt))
    with pytest.raises(capi.DaphneHipError, match="#cols of lhs and #rows of rhs must be the same"):
        matMul(None, a, b, False, False, ctx)
    matMul(None, a, b, True, False, ctx)
    matMul(None, a, b, False, True, ctx)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("trans_left", [True, False])
@pytest.mark.parametrize("rows,cols", [(7, 3), (100, 100), (1000, 100), (5000, 130), (64, 257), (20000, 16)])
def test_syrk(ctx, dt, trans_left, rows, cols):
    rng = np.random.default_rng(rows + cols)
    if not trans_left:
        rows, cols = cols, rows
    x = (rng.random((rows, cols)) * 2 - 1).astype(dt)
    st, exp = orc.syrk(x, trans_left)
    got = syrk(None, DenseMatrix.from_numpy(ctx, x), trans_left, ctx).to_numpy()
    assert_close(got, exp, elementwise=False)
    assert_exact(got, got.T)  # the lower triangle is a copy of the upper one (Syrk.h:65-69)
    # syrk(X) == matMul(t(X), X) (test/runtime/local/kernels/SyrkTest.cpp:32-58)
    X = DenseMatrix.from_numpy(ctx, x)
    mm = matMul(None, X, X, trans_left, not trans_left, ctx).to_numpy()
    assert_close(got, mm, elementwise=False)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("trans_left", [True, False])
@pytest.mark.parametrize("n,k", [(1300, 300), (2100, 70), (4100, 520)])
def test_syrk_many_tiles(ctx, dt, trans_left, n, k):
    """Results of 11, 17 and 33 tiles a side: the triangular tile order walks several groups of 8 x 8 tiles, and at
    33 a side (561 tiles, more than the device holds at once) the last tiles run as a launch of their own that
    splits K. Integer-valued inputs: every order of summation gives the same bits; the expectation is numpy's."""
    rng = np.random.default_rng(n + k)
    x = rng.integers(-3, 4, (k, n) if trans_left else (n, k)).astype(dt)
    xi = x.astype(np.int64)
    exp = ((xi.T @ xi) if trans_left else (xi @ xi.T)).astype(dt)
    got = syrk(None, DenseMatrix.from_numpy(ctx, x), trans_left, ctx).to_numpy()
    assert_exact(got, exp)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("ta,tb", [(False, False), (True, True)])
@pytest.mark.parametrize("m,n,k", [(4224, 2048, 512), (4200, 2040, 520)])
def test_matmul_leftover_tiles(ctx, dt, ta, tb, m, n, k):
    """33 x 16 = 528 tiles of 128 x 128: 512 run as one launch, the other 16 as a second launch that splits K
    (with and without partial tiles). Integer-valued inputs, exact; then a random case with a bias row through
    Affine, norm-wise against numpy in double."""
    rng = np.random.default_rng(m + n + k)
    a = rng.integers(-3, 4, (k, m) if ta else (m, k)).astype(dt)
    b = rng.integers(-3, 4, (n, k) if tb else (k, n)).astype(dt)
    exp = ((a.T if ta else a).astype(np.int64) @ (b.T if tb else b).astype(np.int64)).astype(dt)
    got = matMul(None, DenseMatrix.from_numpy(ctx, a), DenseMatrix.from_numpy(ctx, b), ta, tb, ctx).to_numpy()
    assert_exact(got, exp)
    if not ta and not tb:
        x = (rng.random((m, k)) - 0.5).astype(dt)
        w = (rng.standard_normal((k, n)) * np.sqrt(2.0 / k)).astype(dt)
        bias = (rng.standard_normal((1, n)) * 0.1).astype(dt)
        truth = (x.astype(np.float64) @ w.astype(np.float64) + bias.astype(np.float64)).astype(dt)
        got = affineForward(None, DenseMatrix.from_numpy(ctx, x), DenseMatrix.from_numpy(ctx, w),
                            DenseMatrix.from_numpy(ctx, bias), ctx).to_numpy()
        assert_close(got, truth, elementwise=False)


@pytest.mark.parametrize("dt", DTYPES)
def test_syrk_integer_valued_exact(ctx, dt):
    rng = np.random.default_rng(9)
    x = rng.integers(-3, 4, (3000, 150)).astype(dt)
    exp = (x.T.astype(np.int64) @ x.astype(np.int64)).astype(dt)
    assert_exact(syrk(None, DenseMatrix.from_numpy(ctx, x), True, ctx).to_numpy(), exp)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("n", [1, 3, 10, 63, 64, 65, 100, 128, 135, 136, 150, 190, 192, 193, 257])
def test_solve(ctx, dt, n):
    rng = np.random.default_rng(n)
    A = (rng.random((n, n)) - 0.5).astype(dt) + np.eye(n, dtype=dt) * dt(0.1)
    b = (rng.random((n, 1)) - 0.5).astype(dt)
    st, exp = orc.solve(A, b)
    assert st == 0
    got = solve(None, DenseMatrix.from_numpy(ctx, A), DenseMatrix.from_numpy(ctx, b), ctx).to_numpy()
    tol = (1e-3 if dt == np.float32 else 1e-9) if n > 50 else (1e-4 if dt == np.float32 else 1e-10)
    assert_close(got, exp, rtol=tol, elementwise=False)
    # residual against the definition
    r = A.astype(np.float64) @ got.astype(np.float64) - b
    assert np.abs(r).max() <= (5e-4 if dt == np.float32 else 1e-11) * max(1.0, np.abs(got).max()) * n


@pytest.mark.parametrize("dt", DTYPES)
def test_solve_pivoting_and_late_singularity(ctx, dt):
    rng = np.random.default_rng(77)
    for n in (4, 70, 130, 200):
        # zero diagonal: every column needs a row exchange; integer entries make ties in the pivot search
        A = rng.integers(-3, 4, (n, n)).astype(dt)
        np.fill_diagonal(A, 0)
        A += np.roll(np.eye(n, dtype=dt), 1, axis=0) * dt(9)
        b = rng.integers(-5, 6, (n, 1)).astype(dt)
        st, exp = orc.solve(A, b)
        assert st == 0
        got = solve(None, DenseMatrix.from_numpy(ctx, A), DenseMatrix.from_numpy(ctx, b), ctx).to_numpy()
        assert_close(got, exp, rtol=2e-3 if dt == np.float32 else 1e-9, elementwise=False)
        # rank deficiency that only shows in the last column
        S = rng.random((n, n)).astype(dt)
        S[:, -1] = S[:, 0]
        if n <= 4:  # exact zero pivot only when the elimination is exact
            S = np.array([[1, 2, 3, 1], [0, 1, 4, 0], [0, 0, 1, 0], [1, 2, 3, 1]], dt)
            with pytest.raises(capi.DaphneHipError, match="exactly singular"):
                solve(None, DenseMatrix.from_numpy(ctx, S), DenseMatrix.from_numpy(ctx, b), ctx)
            assert orc.solve(S, b)[0] != 0


@pytest.mark.parametrize("dt", DTYPES)
def test_solve_errors(ctx, dt):
    A = DenseMatrix.from_numpy(ctx, np.zeros((3, 3), dt))
    b = DenseMatrix.from_numpy(ctx, np.ones((3, 1), dt))
    with pytest.raises(capi.DaphneHipError, match="exactly singular"):
        solve(None, A, b, ctx)
    with pytest.raises(capi.DaphneHipError, match="#rows and #cols of lhs must be the same"):
        solve(None, DenseMatrix.from_numpy(ctx, np.ones((3, 2), dt)), b, ctx)


@pytest.mark.parametrize("dt", DTYPES)
def test_solve_with_deferred_verdicts(ctx, dt):
    """Inside a deferred block solves do not wait for their verdict: good systems give the bits of the direct call,
    and a singular one among them is reported when the block ends, with the direct call's error."""
    rng = np.random.default_rng(5)
    systems = []
    for n in (3, 100, 150):  # LDS-resident (one and two rows a lane) and the global-memory kernel's sizes
        A = rng.random((n, n)).astype(dt) + np.eye(n, dtype=dt) * dt(n)
        b = rng.random((n, 1)).astype(dt)
        systems.append((DenseMatrix.from_numpy(ctx, A), DenseMatrix.from_numpy(ctx, b)))
    direct = [solve(None, A, b, ctx).to_numpy() for A, b in systems]
    with ctx.deferred_checks():
        inside = [solve(None, A, b, ctx) for A, b in systems]
    for d, i in zip(direct, inside):
        assert np.array_equal(d, i.to_numpy())
    Z = DenseMatrix.from_numpy(ctx, np.zeros((3, 3), dt))
    with pytest.raises(capi.DaphneHipError, match="exactly singular"):
        with ctx.deferred_checks():
            solve(None, *systems[1], ctx)
            solve(None, Z, systems[0][1], ctx)
            solve(None, *systems[0], ctx)  # a good one after the failure does not clear it
    ctx.check_deferred()  # reported once
    assert np.array_equal(solve(None, *systems[1], ctx).to_numpy(), direct[1])


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m,k,n", [(1, 9, 2), (64, 100, 10), (300, 3136, 512), (257, 512, 10)])
def test_affine(ctx, dt, m, k, n):
    """Affine = MatMul then row-vector add (the reference has no CPU affine kernel)."""
    rng = np.random.default_rng(m + k + n)
    x = (rng.random((m, k)) - 0.5).astype(dt)
    w = (rng.standard_normal((k, n)) * np.sqrt(2.0 / k)).astype(dt)
    b = (rng.standard_normal((1, n)) * 0.1).astype(dt)
    st, mm = orc.matmul(x, w)
    st, exp = orc.ew_binary(0, mm, b)
    got = affineForward(None, DenseMatrix.from_numpy(ctx, x), DenseMatrix.from_numpy(ctx, w),
                        DenseMatrix.from_numpy(ctx, b), ctx).to_numpy()
    assert_close(got, exp, elementwise=False)
    got = affineForward(None, DenseMatrix.from_numpy(ctx, x), DenseMatrix.from_numpy(ctx, w), None, ctx).to_numpy()
    assert_close(got, mm, elementwise=False)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m,k,n", [(1, 9, 2), (64, 100, 10), (300, 3136, 512), (257, 512, 10), (4096, 3136, 512), (700, 64, 130),
                                   (2304, 256, 1280)])
def test_affine_with_relu_equals_affine_then_relu(ctx, dt, m, k, n):
    """The rectifier in the epilogue (direct store, split-K reduction, leftover tiles, no bias) against the two kernels."""
    rng = np.random.default_rng(m + k + n + 1)
    x = DenseMatrix.from_numpy(ctx, (rng.random((m, k)) - 0.5).astype(dt))
    w = DenseMatrix.from_numpy(ctx, (rng.standard_normal((k, n)) * np.sqrt(2.0 / k)).astype(dt))
    for bias in (DenseMatrix.from_numpy(ctx, (rng.standard_normal((1, n)) * 0.1).astype(dt)),
                 DenseMatrix.from_numpy(ctx, np.full((1, 1), 0.05, dt)), None):
        exp = reluForward(None, affineForward(None, x, w, bias, ctx), ctx).to_numpy()
        got = affineForwardFused(None, x, w, bias, ctx).to_numpy()
        assert_exact(got, exp)
        assert m * n < 100 or ((exp == 0).any() and (exp > 0).any())
        assert_exact(affineForwardFused(None, x, w, bias, ctx, relu=False).to_numpy(), affineForward(None, x, w, bias, ctx).to_numpy())


@pytest.mark.parametrize("dt", DTYPES)
def test_affine_errors(ctx, dt):
    x = DenseMatrix.from_numpy(ctx, np.ones((4, 5), dt))
    w = DenseMatrix.from_numpy(ctx, np.ones((6, 3), dt))
    with pytest.raises(capi.DaphneHipError, match="#cols of lhs and #rows of rhs must be the same"):
        affineForward(None, x, w, None, ctx)
    w = DenseMatrix.from_numpy(ctx, np.ones((5, 3), dt))
    with pytest.raises(capi.DaphneHipError, match="bias dimensions not matching"):
        affineForward(None, x, w, DenseMatrix.from_numpy(ctx, np.ones((3, 1), dt)), ctx)


# ---------------------------------------------------------------------------------------------------
# tall-and-skinny shapes (the streaming kernels): t(A) B with a long contraction, A t(B) with many rows
# ---------------------------------------------------------------------------------------------------
TS_TN = [  # (K, m, n): every side class (<=16, <=64, <=128) on both sides, ragged K
    (4096, 1, 1), (5000, 16, 64), (4097, 16, 16), (7001, 64, 16), (6000, 40, 40), (9999, 64, 64), (4500, 100, 100),
    (4100, 128, 128), (8191, 100, 1), (5003, 128, 60), (5003, 30, 120), (4099, 13, 7), (20000, 18, 66),
]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("K,m,n", TS_TN)
def test_matmul_tall_tn(ctx, dt, K, m, n):
    rng = np.random.default_rng(K + 31 * m + n)
    a = (rng.random((K, m)) * 2 - 1).astype(dt)
    b = (rng.random((K, n)) * 2 - 1).astype(dt)
    truth = (a.T.astype(np.float64) @ b.astype(np.float64)).astype(dt)
    got = matMul(None, DenseMatrix.from_numpy(ctx, a), DenseMatrix.from_numpy(ctx, b), True, False, ctx).to_numpy()
    assert got.shape == (m, n)
    assert_close(got, truth, elementwise=False)
    if K * m * n <= 5000 * 64 * 64:
        assert_close(got, orc.matmul(a, b, True, False)[1], elementwise=False)


@pytest.mark.parametrize("dt", DTYPES)
def test_matmul_tall_tn_integer_exact_and_views(ctx, dt):
    rng = np.random.default_rng(5)
    K = 6007
    A = rng.integers(-3, 4, (K, 72)).astype(dt)
    B = rng.integers(-3, 4, (K, 136)).astype(dt)
    dA, dB = DenseMatrix.from_numpy(ctx, A), DenseMatrix.from_numpy(ctx, B)
    # whole matrices, column slices at aligned and unaligned offsets (leading dimension > columns)
    for (a0, a1, b0, b1) in [(0, 72, 0, 128), (8, 40, 16, 80), (3, 19, 5, 69), (0, 16, 4, 68), (1, 2, 0, 1)]:
        exp = (A[:, a0:a1].T.astype(np.int64) @ B[:, b0:b1].astype(np.int64)).astype(dt)
        got = matMul(None, dA.slice(0, K, a0, a1), dB.slice(0, K, b0, b1), True, False, ctx).to_numpy()
        assert_exact(got, exp)
    # into a view of a larger result
    res = DenseMatrix(ctx, 80, 140, dt, zero=True)
    matMul(res.slice(2, 74, 3, 131), dA, dB.slice(0, K, 0, 128), True, False, ctx)
    full = res.to_numpy()
    assert_exact(full[2:74, 3:131], (A.T.astype(np.int64) @ B[:, :128].astype(np.int64)).astype(dt))
    full[2:74, 3:131] = 0
    assert (full == 0).all()


@pytest.mark.parametrize("dt", DTYPES)
def test_syrk_and_gemv_tall(ctx, dt):
    rng = np.random.default_rng(6)
    X = (rng.random((50000, 100)) * 2 - 1).astype(dt)
    y = (rng.random((50000, 1)) * 2 - 1).astype(dt)
    dX, dy = DenseMatrix.from_numpy(ctx, X), DenseMatrix.from_numpy(ctx, y)
    got = syrk(None, dX, True, ctx).to_numpy()
    truth = X.T.astype(np.float64) @ X.astype(np.float64)
    assert_close(got, truth.astype(dt), elementwise=False)
    assert_exact(got, got.T)  # both triangles come from the same products in the same order
    gv = matMul(None, dX, dy, True, False, ctx).to_numpy()
    assert gv.shape == (100, 1)
    assert_close(gv, (X.T.astype(np.float64) @ y.astype(np.float64)).astype(dt), elementwise=False)
    # the vector given as a row (transposed rhs) and as a strided column of a wider matrix
    yr = np.ascontiguousarray(y.T)
    assert_close(matMul(None, dX, DenseMatrix.from_numpy(ctx, yr), True, True, ctx).to_numpy(), gv, elementwise=False)
    Y3 = np.repeat(y, 3, axis=1).copy()
    assert_exact(matMul(None, dX, DenseMatrix.from_numpy(ctx, Y3).slice(0, 50000, 1, 2), True, False, ctx).to_numpy(), gv)


TS_NT = [  # (M, n, K)
    (65536, 16, 64), (70001, 16, 64), (65537, 1, 4), (66000, 7, 20), (65536, 32, 128), (80000, 17, 72), (65536, 16, 512),
    (100003, 10, 100),
]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("M,n,K", TS_NT)
def test_matmul_tall_nt(ctx, dt, M, n, K):
    rng = np.random.default_rng(M + 7 * n + K)
    a = (rng.random((M, K)) * 2 - 1).astype(dt)
    b = (rng.random((n, K)) * 2 - 1).astype(dt)
    truth = (a.astype(np.float64) @ b.T.astype(np.float64)).astype(dt)
    got = matMul(None, DenseMatrix.from_numpy(ctx, a), DenseMatrix.from_numpy(ctx, b), False, True, ctx).to_numpy()
    assert got.shape == (M, n)
    assert_close(got, truth, elementwise=False)
    ai = rng.integers(-3, 4, (M, K)).astype(dt)
    bi = rng.integers(-3, 4, (n, K)).astype(dt)
    goti = matMul(None, DenseMatrix.from_numpy(ctx, ai), DenseMatrix.from_numpy(ctx, bi), False, True, ctx).to_numpy()
    assert_exact(goti, (ai.astype(np.int64) @ bi.T.astype(np.int64)).astype(dt))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("cols,ld", [(65, 72), (80, 80), (81, 88), (96, 96), (100, 100), (111, 112), (112, 120), (113, 128),
                                      (128, 128)])
@pytest.mark.parametrize("rows", [4096, 10_007])
def test_syrk_and_normal_equations_of_65_to_128_columns(ctx, dt, cols, ld, rows):
    """The triangle-only kernel for 65..128 columns (every tile count and tail shape, rows that do not fill the last
    step, a view with a row stride): syrk, and the normal equations with t(X) y from the same pass, against the
    oracle's Syrk / MatMul and against float64 numpy."""
    from daphne_amd.kernels import normalEquations

    if (ld * np.dtype(dt).itemsize) % 16:
        pytest.skip("rows of this stride are not 16-byte aligned for this value type: the general kernels take it")
    rng = np.random.default_rng(rows + cols)
    base = np.full((rows, ld), np.nan, dt)  # what lies beyond the columns must never reach a result
    base[:, :cols] = (rng.random((rows, cols)) * 2 - 1).astype(dt)
    x = base[:, :cols]
    y = (rng.random((rows, 1)) * 2 - 1).astype(dt)
    X = DenseMatrix.from_numpy(ctx, base).slice(0, rows, 0, cols)
    Y = DenseMatrix.from_numpy(ctx, y)
    S = syrk(None, X, True, ctx).to_numpy()
    assert_exact(S, S.T)
    assert_close(S, orc.syrk(np.ascontiguousarray(x), True)[1], elementwise=False)
    lam = 0.25
    A, b = normalEquations(X, Y, lam, ctx)
    x64 = x.astype(np.float64)
    assert_close(A.to_numpy(), (x64.T @ x64 + lam * np.eye(cols)).astype(dt), elementwise=False)
    assert_close(b.to_numpy(), (x64.T @ y.astype(np.float64)).astype(dt), elementwise=False)
    assert_exact(A.to_numpy() - np.diag(np.diag(A.to_numpy())), S - np.diag(np.diag(S)))  # the same kernel, with and without y


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("rows,cols", [(5000, 20), (300, 100), (7000, 64), (4096, 200)])
def test_normal_equations_of_other_shapes(ctx, dt, rows, cols):
    """Shapes the fused kernel does not take run the operator sequence; same results."""
    from daphne_amd.kernels import normalEquations

    rng = np.random.default_rng(cols)
    x = (rng.random((rows, cols)) * 2 - 1).astype(dt)
    y = (rng.random((rows, 1)) * 2 - 1).astype(dt)
    A, b = normalEquations(DenseMatrix.from_numpy(ctx, x), DenseMatrix.from_numpy(ctx, y), 1e-3, ctx)
    x64 = x.astype(np.float64)
    assert_close(A.to_numpy(), (x64.T @ x64 + 1e-3 * np.eye(cols)).astype(dt), elementwise=False)
    assert_close(b.to_numpy(), (x64.T @ y.astype(np.float64)).astype(dt), elementwise=False)


KMEANS_SHAPES = [  # rows, cols, k
    (1, 4, 1), (7, 8, 3), (100, 64, 16), (513, 64, 16), (70_000, 64, 16), (66_000, 32, 32), (65_600, 12, 17), (3000, 200, 5),
    (2049, 128, 20), (131_072, 4, 2), (33, 52, 2), (300_001, 60, 30), (1_000_000, 64, 7), (70_001, 40, 9), (65_537, 36, 20),
    (70_003, 16, 5), (66_001, 24, 12), (67_000, 28, 16),  # two, three and four chunks of doubles in one step
]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,cols,k", KMEANS_SHAPES)
def test_kmeans_assign_and_update(ctx, dt, rows, cols, k):
    """The two passes against the operator sequence on the device (bit for bit where the product takes the streaming
    kernel: 65536 rows or more) and against the oracle (away from near-ties)."""
    rng = np.random.default_rng(rows + cols + k)
    centres = rng.standard_normal((k, cols)) * 3
    x = (centres[rng.integers(0, k, rows)] + rng.standard_normal((rows, cols))).astype(dt)
    c = (centres + 0.3 * rng.standard_normal((k, cols))).astype(dt)
    if k > 2:
        c[k - 1] = c[1]  # two equal centroids: the lower position wins
    X, C = DenseMatrix.from_numpy(ctx, x), DenseMatrix.from_numpy(ctx, c)
    xx = aggRow(AggOpCode.SUM, None, ewBinaryMat(BinaryOpCode.MUL, None, X, X, ctx), ctx)
    cc = aggRow(AggOpCode.SUM, None, ewBinaryMat(BinaryOpCode.MUL, None, C, C, ctx), ctx)
    idx = kmeansAssign(None, X, C, xx, cc, ctx).to_numpy()
    # the operator sequence
    XC = matMul(None, X, C, False, True, ctx)
    D = ewBinaryObjSca(BinaryOpCode.MUL, None, XC, -2.0, ctx)
    D = ewBinaryMat(BinaryOpCode.ADD, None, D, xx, ctx)
    cc_row = DenseMatrix.from_numpy(ctx, np.ascontiguousarray(cc.to_numpy().T))
    D = ewBinaryMat(BinaryOpCode.ADD, None, D, cc_row, ctx)
    idx_seq = aggRow(AggOpCode.IDXMIN, None, D, ctx).to_numpy()
    d = D.to_numpy().astype(np.float64)
    if rows >= 65536:
        assert_exact(idx, idx_seq)
    else:
        part = np.partition(d, 1, axis=1) if k > 1 else np.concatenate([d, d + 1], axis=1)
        clear = (part[:, 1] - part[:, 0]) > 1e-3 * np.abs(part[:, 0]) if k > 1 else np.ones(rows, bool)
        if k > 2:
            clear &= ~np.isin(idx_seq[:, 0], (1, k - 1))
        assert_exact(idx[clear], idx_seq[clear])
    assert idx.dtype == np.uint64 and (idx < k).all()
    if k > 2:
        assert not (idx == k - 1).any()
    st, idx_o = orc.agg_row(AggOpCode.IDXMIN, d.astype(dt))
    same = (idx == idx_o).mean()
    assert same > 0.999
    # update: per-cluster means and sizes from idx
    if cols > (256 if dt == np.float32 else 128):
        with pytest.raises(capi.DaphneHipError, match="features are supported"):
            kmeansUpdate(None, X, DenseMatrix.from_numpy(ctx, idx), k, ctx)
        return
    Cn, counts = kmeansUpdate(None, X, DenseMatrix.from_numpy(ctx, idx), k, ctx)
    # both passes as one call (one pass over X for up to 64 features): the same assignment and sizes bit for bit
    idx1, Cn1, counts1 = kmeansStep(None, None, X, C, xx, cc, ctx)
    assert_exact(idx1.to_numpy(), idx)
    assert_exact(counts1.to_numpy(), counts.to_numpy())
    assert_close(Cn1.to_numpy(), Cn.to_numpy(), rtol=2e-5 if dt == np.float32 else 1e-12, elementwise=False)
    cnt = np.bincount(idx[:, 0].astype(np.int64), minlength=k).astype(np.float64)
    assert_exact(counts.to_numpy()[0].astype(np.float64), cnt)
    sums = np.zeros((k, cols))
    np.add.at(sums, idx[:, 0].astype(np.int64), x.astype(np.float64))
    with np.errstate(invalid="ignore", divide="ignore"):
        exp = (sums / cnt[:, None]).astype(dt)
    assert_close(Cn.to_numpy(), exp, rtol=2e-5 if dt == np.float32 else 1e-12, elementwise=False)
    assert np.isnan(Cn.to_numpy()[cnt == 0]).all()


@pytest.mark.parametrize("dt", DTYPES)
def test_kmeans_assign_nan_semantics_and_errors(ctx, dt):
    """IDXMIN's rules on the fused distances: NaN is never better, a row that starts with NaN or holds only NaN gives 0."""
    rows, cols, k = 64, 8, 6
    rng = np.random.default_rng(0)
    x = rng.standard_normal((rows, cols)).astype(dt)
    c = rng.standard_normal((k, cols)).astype(dt)
    X, C = DenseMatrix.from_numpy(ctx, x), DenseMatrix.from_numpy(ctx, c)
    xx = DenseMatrix.from_numpy(ctx, (x * x).sum(1, keepdims=True).astype(dt))
    cc_h = (c * c).sum(1, keepdims=True).astype(dt)
    cc_h[0] = np.nan   # distance to centroid 0 is NaN in every row: position 0 by the first-value rule
    idx = kmeansAssign(None, X, C, xx, DenseMatrix.from_numpy(ctx, cc_h), ctx).to_numpy()
    assert (idx == 0).all()
    cc_h[0], cc_h[3] = (c[0] * c[0]).sum(), np.nan  # a NaN elsewhere is skipped
    idx = kmeansAssign(None, X, C, xx, DenseMatrix.from_numpy(ctx, cc_h), ctx).to_numpy()
    d = (x @ c.T) * -2 + (x * x).sum(1, keepdims=True) + cc_h.T
    assert_exact(idx[:, 0], np.nanargmin(d, axis=1).astype(np.uint64))
    with pytest.raises(capi.DaphneHipError, match="1..32 centroids"):
        kmeansAssign(None, X, DenseMatrix.from_numpy(ctx, np.zeros((33, cols), dt)), xx, DenseMatrix.from_numpy(ctx, np.zeros((33, 1), dt)), ctx)
    with pytest.raises(capi.DaphneHipError, match="16-byte"):
        x3 = DenseMatrix.from_numpy(ctx, np.zeros((4, 3), dt))
        kmeansAssign(None, x3, DenseMatrix.from_numpy(ctx, np.zeros((2, 3), dt)), DenseMatrix.from_numpy(ctx, np.zeros((4, 1), dt)),
                     DenseMatrix.from_numpy(ctx, np.zeros((2, 1), dt)), ctx)
    with pytest.raises(capi.DaphneHipError, match="features are supported"):
        wide = DenseMatrix.from_numpy(ctx, np.zeros((4, 600), dt))
        kmeansUpdate(None, wide, DenseMatrix.from_numpy(ctx, np.zeros((4, 1), np.uint64)), 2, ctx)
    # a null pointer is refused on the host (the kernels read and write all of these unconditionally); only
    # `counts` may be left out
    suf = "f32" if dt == np.float32 else "f64"
    lib = capi.lib()
    idx_ok = DenseMatrix(ctx, X.rows, 1, np.uint64)
    cc = DenseMatrix.from_numpy(ctx, cc_h)
    cn = DenseMatrix(ctx, k, cols, dt)
    good = dict(idx=idx_ok.ptr, X=X.ptr, C=C.ptr, xx=xx.ptr, cc=cc.ptr)
    for missing in good:
        a = dict(good, **{missing: None})
        st = getattr(lib, f"dh_kmeans_assign_{suf}")(ctx._h, a["idx"], a["X"], X.rows, cols, X.row_skip, a["C"], k, C.row_skip, a["xx"], a["cc"])
        assert st == 2 and b"must not be null" in lib.dh_last_error(), missing   # DH_ERR_INVALID_ARG
        st = getattr(lib, f"dh_kmeans_step_{suf}")(ctx._h, a["idx"], cn.ptr, cn.row_skip, None, a["X"], X.rows, cols, X.row_skip, a["C"], k,
                                                   C.row_skip, a["xx"], a["cc"])
        assert st == 2 and b"must not be null" in lib.dh_last_error(), missing
    st = getattr(lib, f"dh_kmeans_step_{suf}")(ctx._h, idx_ok.ptr, None, cols, None, X.ptr, X.rows, cols, X.row_skip, C.ptr, k, C.row_skip,
                                               xx.ptr, cc.ptr)
    assert st == 2
    for a_cn, a_x, a_idx in ((None, X.ptr, idx_ok.ptr), (cn.ptr, None, idx_ok.ptr), (cn.ptr, X.ptr, None)):
        st = getattr(lib, f"dh_kmeans_update_{suf}")(ctx._h, a_cn, cols, None, a_x, X.rows, cols, X.row_skip, a_idx, k)
        assert st == 2 and b"must not be null" in lib.dh_last_error()
    capi.check(getattr(lib, f"dh_kmeans_update_{suf}")(ctx._h, cn.ptr, cn.row_skip, None, X.ptr, X.rows, cols, X.row_skip, idx_ok.ptr, k))
