"""GPU parity of the remaining device kernels of the reference's kernel library - Fill, ColBind, ExtractCol,
Transpose, Gemv, ReLU activation, average pooling - against the CPU oracle, through the C ABI. Data movement and
ReLU are bit-exact; Gemv and average pooling within 1e-4 (float) / 1e-10 (double) relative."""
import numpy as np
import pytest

import oracle_binding as orc
from parity import assert_close, assert_exact

pytestmark = pytest.mark.gpu

from daphne_amd import capi
from daphne_amd.kernels import (DenseMatrix, avgPoolForward, colBind, extractCol, fill, gemv, reluForward, transpose)

DTYPES = [np.float32, np.float64]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("shape", [(0, 0), (0, 5), (5, 0), (1, 1), (1, 5), (1, 1000), (1000, 1), (3, 4), (123, 456),
                                   (1000, 1000), (70000, 3)])  # the shapes of FillTest.cpp and CUDA/FillTest.cpp
@pytest.mark.parametrize("value", [0.0, 2.5, 123.45])
def test_fill(ctx, dt, shape, value):
    got = fill(None, value, shape[0], shape[1], ctx, dtype=dt).to_numpy()
    st, exp = orc.fill(value, shape[0], shape[1], dt)
    assert st == 0 and got.shape == shape
    assert_exact(got, exp)


@pytest.mark.parametrize("dt", DTYPES)
def test_fill_into_view(ctx, dt):
    big = DenseMatrix(ctx, 40, 37, dt, zero=True)
    fill(big.slice(3, 30, 5, 22), -7.0, 27, 17, ctx)
    full = big.to_numpy()
    assert (full[3:30, 5:22] == -7).all()
    full[3:30, 5:22] = 0
    assert (full == 0).all()


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,lc,rc", [(3, 2, 3), (1, 1, 1), (100, 64, 16), (1000, 7, 9), (65, 128, 4), (20000, 16, 1),
                                        (5, 0, 3), (5, 3, 0), (0, 3, 2)])
def test_col_bind(ctx, dt, rows, lc, rc):
    rng = np.random.default_rng(rows + lc + rc)
    a, b = rng.standard_normal((rows, lc)).astype(dt), rng.standard_normal((rows, rc)).astype(dt)
    st, exp = orc.col_bind(a, b)
    assert st == 0
    assert_exact(exp, np.hstack([a, b]))
    got = colBind(None, DenseMatrix.from_numpy(ctx, a), DenseMatrix.from_numpy(ctx, b), ctx).to_numpy()
    assert_exact(got, exp)


@pytest.mark.parametrize("dt", DTYPES)
def test_col_bind_views_and_errors(ctx, dt):
    rng = np.random.default_rng(3)
    A, B = rng.standard_normal((50, 40)).astype(dt), rng.standard_normal((60, 30)).astype(dt)
    dA, dB = DenseMatrix.from_numpy(ctx, A), DenseMatrix.from_numpy(ctx, B)
    res = DenseMatrix(ctx, 60, 70, dt, zero=True)
    colBind(res.slice(5, 45, 3, 3 + 21 + 13), dA.slice(2, 42, 7, 28), dB.slice(11, 51, 1, 14), ctx)
    full = res.to_numpy()
    assert_exact(full[5:45, 3:37], np.hstack([A[2:42, 7:28], B[11:51, 1:14]]))
    full[5:45, 3:37] = 0
    assert (full == 0).all()
    with pytest.raises(capi.DaphneHipError, match="same number of rows"):
        colBind(None, dA, dB, ctx)
    assert orc.col_bind(A, B)[0] == orc.ST_RUNTIME


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,cols,sel", [(3, 3, [0, 2]), (3, 3, [2, 0, 1]), (3, 3, [1, 2, 2, 0, 1, 0, 1, 2]), (5, 7, [-1, -7, 3]),
                                           (100000, 64, [63, 0, 17, 17]), (1, 1, [0]), (40, 300, list(range(299, -1, -3))),
                                           # selections that take the kernel which streams whole rows (4096 rows or more,
                                           # rows of 1, 4, 16, 64 vectors), with a last wavefront that is not full
                                           (50001, 64, [5, -1, 33, 33, 0, -64, 47, 18]), (8193, 16, [3, -1, 0]),
                                           (20000, 256, list(range(0, 256, 3))), (5003, 4, [1]), (4100, 64, list(range(63, -1, -1)))])
def test_extract_col(ctx, dt, rows, cols, sel):
    rng = np.random.default_rng(rows + cols)
    a = rng.standard_normal((rows, cols)).astype(dt)
    s = np.asarray(sel, dtype=np.int64).reshape(-1, 1)
    st, exp = orc.extract_col(a, s)
    assert st == 0
    assert_exact(exp, a[:, [v % cols for v in sel]])
    got = extractCol(None, DenseMatrix.from_numpy(ctx, a), DenseMatrix.from_numpy(ctx, s), ctx).to_numpy()
    assert_exact(got, exp)


@pytest.mark.parametrize("dt", DTYPES)
def test_extract_col_errors_and_views(ctx, dt):
    a = np.arange(1, 10, dtype=dt).reshape(3, 3)
    dA = DenseMatrix.from_numpy(ctx, a)
    for bad in ([-4, -3], [1, 3]):  # ExtractColTest.cpp:190-197
        s = np.asarray(bad, dtype=np.int64).reshape(-1, 1)
        with pytest.raises(capi.DaphneHipOutOfRange, match="out of bounds"):
            extractCol(None, dA, DenseMatrix.from_numpy(ctx, s), ctx)
        assert orc.extract_col(a, s)[0] == 6
    two = DenseMatrix.from_numpy(ctx, np.zeros((2, 2), np.int64))
    with pytest.raises(capi.DaphneHipError, match="column matrix"):
        extractCol(None, dA, two, ctx)
    # the same on views of a matrix with enough rows for the kernel that streams whole rows
    rngv = np.random.default_rng(18)
    wide = rngv.standard_normal((6000, 80)).astype(dt)
    sv = np.asarray([63, 1, -2, 40, 7, 7, 22, 0], dtype=np.int64).reshape(-1, 1)
    resv = DenseMatrix(ctx, 6000, 12, dt, zero=True)
    extractCol(resv.slice(0, 6000, 2, 10), DenseMatrix.from_numpy(ctx, wide).slice(0, 6000, 8, 72), DenseMatrix.from_numpy(ctx, sv), ctx)
    fullv = resv.to_numpy()
    assert_exact(fullv[:, 2:10], wide[:, 8:72][:, [63, 1, 62, 40, 7, 7, 22, 0]])
    assert (fullv[:, :2] == 0).all() and (fullv[:, 10:] == 0).all()
    # argument and result views
    rng = np.random.default_rng(8)
    big = rng.standard_normal((30, 20)).astype(dt)
    s = np.asarray([4, 0, -1], dtype=np.int64).reshape(-1, 1)
    res = DenseMatrix(ctx, 30, 10, dt, zero=True)
    extractCol(res.slice(3, 23, 2, 5), DenseMatrix.from_numpy(ctx, big).slice(5, 25, 6, 16), DenseMatrix.from_numpy(ctx, s), ctx)
    full = res.to_numpy()
    assert_exact(full[3:23, 2:5], big[5:25, 6:16][:, [4, 0, 9]])
    full[3:23, 2:5] = 0
    assert (full == 0).all()


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("shape", [(3, 4), (5, 6), (1, 1), (1, 700), (700, 1), (64, 64), (65, 63), (1000, 37), (37, 1000),
                                   (4096, 512), (0, 4), (100000, 16)])
def test_transpose(ctx, dt, shape):
    rng = np.random.default_rng(shape[0] * 7 + shape[1])
    a = rng.standard_normal(shape).astype(dt)
    st, exp = orc.transpose(a)
    assert st == 0
    assert_exact(exp, a.T)
    got = transpose(None, DenseMatrix.from_numpy(ctx, a), ctx).to_numpy()
    assert got.shape == (shape[1], shape[0])
    assert_exact(got, exp)


@pytest.mark.parametrize("dt", DTYPES)
def test_transpose_views(ctx, dt):
    rng = np.random.default_rng(4)
    big = rng.standard_normal((200, 150)).astype(dt)
    res = DenseMatrix(ctx, 160, 210, dt, zero=True)
    transpose(res.slice(7, 7 + 131, 9, 9 + 177), DenseMatrix.from_numpy(ctx, big).slice(11, 188, 5, 136), ctx)
    full = res.to_numpy()
    assert_exact(full[7:138, 9:186], big[11:188, 5:136].T)
    full[7:138, 9:186] = 0
    assert (full == 0).all()


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,cols", [(7, 3), (1, 1), (300, 100), (5000, 100), (100000, 100), (4099, 13), (64, 2000)])
def test_gemv(ctx, dt, rows, cols):
    rng = np.random.default_rng(rows + cols)
    m = (rng.random((rows, cols)) * 2 - 1).astype(dt)
    v = (rng.random((rows, 1)) * 2 - 1).astype(dt)
    truth = (m.T.astype(np.float64) @ v.astype(np.float64)).astype(dt)
    got = gemv(None, DenseMatrix.from_numpy(ctx, m), DenseMatrix.from_numpy(ctx, v), ctx).to_numpy()
    assert got.shape == (cols, 1)
    assert_close(got, truth, elementwise=False)
    if rows * cols <= 500000:
        st, exp = orc.gemv(m, v)
        assert st == 0
        assert_close(got, exp, elementwise=False)
    mi, vi = rng.integers(-3, 4, (rows, cols)).astype(dt), rng.integers(-3, 4, (rows, 1)).astype(dt)
    assert_exact(gemv(None, DenseMatrix.from_numpy(ctx, mi), DenseMatrix.from_numpy(ctx, vi), ctx).to_numpy(),
                 (mi.T.astype(np.int64) @ vi.astype(np.int64)).astype(dt))
    with pytest.raises(capi.DaphneHipError, match="#rows of mat and #rows of vec"):
        gemv(None, DenseMatrix.from_numpy(ctx, m), DenseMatrix.from_numpy(ctx, np.ones((rows + 1, 1), dt)), ctx)


@pytest.mark.parametrize("dt", DTYPES)
def test_relu(ctx, dt):
    x = np.array([[-3, -2, -1, 0, 1, 2, 3, 4, 5]], dtype=dt)  # CUDA/DNNActivationTest.cpp:34-40
    assert_exact(reluForward(None, DenseMatrix.from_numpy(ctx, x), ctx).to_numpy(), np.array([[0, 0, 0, 0, 1, 2, 3, 4, 5]], dt))
    rng = np.random.default_rng(1)
    a = rng.standard_normal((777, 333)).astype(dt)
    a[0, :5] = [np.nan, -np.inf, np.inf, -0.0, 0.0]
    st, exp = orc.relu(a)
    assert st == 0
    d = DenseMatrix.from_numpy(ctx, a)
    assert_exact(reluForward(None, d, ctx).to_numpy(), exp)
    reluForward(d, d, ctx)  # in place
    assert_exact(d.to_numpy(), exp)


POOL = [  # N, C, H, W, ph, pw, sh, sw, padh, padw
    (2, 3, 5, 5, 2, 2, 2, 2, 1, 1),    # DNNPoolingTestForward.cpp:36-38
    (2, 3, 5, 5, 2, 2, 1, 1, 0, 0), (3, 2, 8, 8, 2, 2, 2, 2, 0, 0), (2, 2, 9, 7, 3, 2, 2, 3, 1, 0), (1, 1, 6, 6, 3, 3, 3, 3, 0, 0),
    (2, 4, 7, 1, 7, 1, 1, 1, 0, 0),    # one output per plane of a one-column image (the quick path)
    (2, 2, 5, 1, 3, 1, 1, 1, 0, 0), (4, 3, 12, 10, 4, 5, 1, 1, 2, 2), (64, 8, 28, 28, 2, 2, 2, 2, 0, 0),
    (333, 64, 14, 14, 3, 3, 2, 2, 1, 1),   # several planes per workgroup staged in LDS, short last workgroup
    (301, 33, 7, 7, 3, 3, 1, 1, 1, 1),     # planes of 49 values: a multiple of four planes per workgroup
    (2, 2, 80, 80, 4, 4, 2, 2, 1, 1),      # planes too large for the LDS kernel
    (7, 11887, 14, 14, 3, 2, 2, 2, 1, 0),  # thousands of workgroups, short last one
]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("p", POOL)
def test_avgpool(ctx, dt, p):
    N, C_, H, W = p[:4]
    rng = np.random.default_rng(sum(p))
    x = (rng.standard_normal((N, C_ * H * W)) * 3).astype(dt)
    st, exp, eh, ew = orc.avgpool(x, *p)
    assert st == 0
    got, gh, gw = avgPoolForward(None, DenseMatrix.from_numpy(ctx, x), *p, ctx)
    assert (gh, gw) == (eh, ew)
    assert_close(got.to_numpy(), exp)
    xi = rng.integers(-8, 9, (N, C_ * H * W)).astype(dt) * 4.0  # window sums and their scaling are exact for 2^k windows
    if (p[4] * p[5]) & (p[4] * p[5] - 1) == 0:
        assert_exact(avgPoolForward(None, DenseMatrix.from_numpy(ctx, xi.astype(dt)), *p, ctx)[0].to_numpy(),
                     orc.avgpool(xi.astype(dt), *p)[1])
