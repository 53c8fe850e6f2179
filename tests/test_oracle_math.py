"""CPU: pins the oracle by what the mathematics fixes, independently of its own formulas: numpy /
scipy library routines, closed forms, brute force on small inputs. Each check is chosen so that a
plausible slip (dropped term, wrong sign or index, transposed operand, wrong divisor) fails it."""
import numpy as np
import pytest
import scipy.special

import oracle_binding as orc

DT = [np.float32, np.float64]


def tol(dt):
    return 2e-6 if dt == np.float32 else 1e-13


@pytest.mark.parametrize("dt", DT)
def test_ew_single_ieee_ops_equal_numpy_bitwise(dt):
    rng = np.random.default_rng(0)
    a, b = rng.standard_normal((31, 17)).astype(dt), rng.standard_normal((31, 17)).astype(dt)
    with np.errstate(all="ignore"):
        for op, f in {0: np.add, 1: np.subtract, 2: np.multiply, 3: np.divide, 5: np.fmod}.items():
            assert np.array_equal(orc.ew_binary(op, a, b)[1], f(a, b))
        for op, f in {7: np.equal, 8: np.not_equal, 9: np.less, 10: np.less_equal, 11: np.greater, 12: np.greater_equal}.items():
            assert np.array_equal(orc.ew_binary(op, a, b)[1], f(a, b).astype(dt))
        assert np.array_equal(orc.ew_binary(13, a, b)[1], np.minimum(a, b))
        assert np.array_equal(orc.ew_binary(14, a, b)[1], np.maximum(a, b))
        assert np.allclose(orc.ew_binary(4, np.abs(a), b)[1], np.power(np.abs(a), b), rtol=tol(dt) * 10)
        assert np.allclose(orc.ew_binary(6, np.abs(a) + 1, np.abs(b) + 2)[1], np.log(np.abs(a) + 1) / np.log(np.abs(b) + 2), rtol=tol(dt) * 10)
    # broadcasting: result has lhs' shape, row vector over rows, column vector over columns
    rv, cv = b[:1], b[:, :1]
    assert np.array_equal(orc.ew_binary(1, a, rv)[1], a - rv)
    assert np.array_equal(orc.ew_binary(1, a, cv)[1], a - cv)
    assert orc.ew_binary(0, a, b[:5])[0] == orc.ST_RUNTIME
    # std::min / std::max NaN rule: NaN on the right is ignored, NaN on the left stays
    x, y = np.array([[np.nan, 1.0]], dt), np.array([[1.0, np.nan]], dt)
    r = orc.ew_binary(13, x, y)[1]
    assert np.isnan(r[0, 0]) and r[0, 1] == 1.0


@pytest.mark.parametrize("dt", DT)
def test_unary_against_numpy(dt):
    rng = np.random.default_rng(1)
    a = rng.standard_normal((9, 13)).astype(dt) * 2
    fns = {0: np.negative, 1: np.abs, 2: np.sign, 4: np.exp, 6: np.sin, 7: np.cos, 8: np.tan, 11: np.arctan, 12: np.sinh,
           13: np.cosh, 14: np.tanh, 15: np.floor, 16: np.ceil}
    for op, f in fns.items():
        assert np.allclose(orc.ew_unary(op, a)[1], f(a), rtol=tol(dt) * 20, atol=0), op
    assert np.array_equal(orc.ew_unary(3, np.abs(a))[1], np.sqrt(np.abs(a)))
    # round: half away from zero (C round), unlike numpy's half-to-even
    h = np.array([[0.5, 1.5, 2.5, -0.5, -1.5, -2.5]], dt)
    assert np.array_equal(orc.ew_unary(17, h)[1], np.array([[1, 2, 3, -1, -2, -3]], dt))
    assert np.array_equal(orc.ew_unary(18, np.array([[np.nan, 1.0]], dt))[1], np.array([[1, 0]], dt))
    for op, bad in ((3, -1.0), (5, -1.0), (9, 1.01), (10, -1.01)):
        assert orc.ew_unary(op, np.array([[0.5, bad]], dt))[0] == orc.ST_DOMAIN
        assert orc.ew_unary(op, np.array([[0.5, 0.25]], dt))[0] == 0
    assert orc.ew_unary(3, np.array([[-0.0, np.nan]], dt))[0] == 0  # -0 and NaN are inside the domain check


@pytest.mark.parametrize("dt", DT)
def test_aggregations_against_numpy(dt):
    rng = np.random.default_rng(2)
    a = (rng.standard_normal((57, 23)) * 3 + 1).astype(dt)
    a64 = a.astype(np.float64)
    rt = 1e-5 if dt == np.float32 else 1e-12
    at = rt * np.abs(a64).sum(axis=1).max()  # sums with cancellation: error relative to the summed magnitudes
    for op, f in {0: np.sum, 2: np.min, 3: np.max, 6: np.mean, 7: np.std, 8: np.var}.items():
        assert np.allclose(orc.agg_all(op, a)[1], f(a64), rtol=rt, atol=at)
        assert np.allclose(orc.agg_row(op, a)[1][:, 0], f(a64, axis=1), rtol=rt, atol=at)
        assert np.allclose(orc.agg_col(op, a)[1][0], f(a64, axis=0), rtol=rt, atol=at)
    p = (1 + 0.01 * rng.standard_normal((11, 7))).astype(dt)
    assert np.allclose(orc.agg_all(1, p)[1], np.prod(p.astype(np.float64)), rtol=rt)
    # index of the first strict extremum == numpy argmin / argmax (ties: first)
    t = rng.integers(0, 4, (40, 9)).astype(dt)
    assert np.array_equal(orc.agg_row(4, t)[1][:, 0], np.argmin(t, axis=1).astype(np.uint64))
    assert np.array_equal(orc.agg_row(5, t)[1][:, 0], np.argmax(t, axis=1).astype(np.uint64))
    assert np.array_equal(orc.agg_col(4, t)[1][0], np.argmin(t, axis=0).astype(np.uint64))
    assert np.array_equal(orc.agg_col(5, t)[1][0], np.argmax(t, axis=0).astype(np.uint64))
    # views: leading dimension larger than the column count
    big = rng.standard_normal((20, 30)).astype(dt)
    v = big[3:17, 4:21]
    assert np.allclose(orc.agg_all(0, v)[1], v.astype(np.float64).sum(), rtol=rt)
    assert np.allclose(orc.agg_col(8, v)[1][0], v.astype(np.float64).var(axis=0), rtol=rt)


@pytest.mark.parametrize("dt", DT)
def test_contractions_against_numpy(dt):
    rng = np.random.default_rng(3)
    rt = 1e-5 if dt == np.float32 else 1e-12
    A, B = rng.standard_normal((13, 29)).astype(dt), rng.standard_normal((29, 7)).astype(dt)
    ref = A.astype(np.float64) @ B.astype(np.float64)
    for ta, tb in ((0, 0), (1, 0), (0, 1), (1, 1)):
        a = np.ascontiguousarray(A.T) if ta else A
        b = np.ascontiguousarray(B.T) if tb else B
        st, got = orc.matmul(a, b, ta, tb)
        assert st == 0 and np.allclose(got, ref, rtol=rt, atol=rt * np.abs(ref).max())
    assert orc.matmul(A, A)[0] == orc.ST_RUNTIME
    X = rng.standard_normal((50, 6)).astype(dt)
    for tl in (True, False):
        st, S = orc.syrk(X, tl)
        refS = X.astype(np.float64).T @ X.astype(np.float64) if tl else X.astype(np.float64) @ X.astype(np.float64).T
        assert np.allclose(S, refS, rtol=rt, atol=rt * np.abs(refS).max()) and np.array_equal(S, S.T)
    M = rng.standard_normal((12, 12)).astype(dt) + 4 * np.eye(12, dtype=dt)
    b = rng.standard_normal((12, 1)).astype(dt)
    st, x = orc.solve(M, b)
    assert st == 0 and np.allclose(x, np.linalg.solve(M.astype(np.float64), b.astype(np.float64)), rtol=1e-3 if dt == np.float32 else 1e-10)
    assert orc.solve(np.zeros((3, 3), dt), np.ones((3, 1), dt))[0] == orc.ST_RUNTIME
    # a system that needs the row exchange (zero leading pivot)
    P = np.array([[0, 2, 1], [1, 1, 1], [2, 0, 3]], dt)
    assert np.allclose(orc.solve(P, np.array([[3], [3], [5]], dt))[1], np.linalg.solve(P.astype(np.float64), [[3], [3], [5]]), rtol=1e-5)


def _conv_brute(x, w, bias, N, C, H, W, F, Hf, Wf, sh, sw, ph, pw):
    xp = np.zeros((N, C, H + 2 * ph, W + 2 * pw))
    xp[:, :, ph:ph + H, pw:pw + W] = x.reshape(N, C, H, W)
    P, Q = (H + 2 * ph - Hf) // sh + 1, (W + 2 * pw - Wf) // sw + 1
    win = np.lib.stride_tricks.sliding_window_view(xp, (Hf, Wf), axis=(2, 3))[:, :, ::sh, ::sw][:, :, :P, :Q]
    out = np.einsum("ncpqhw,fchw->nfpq", win, w.reshape(F, C, Hf, Wf).astype(np.float64))
    if bias is not None:
        out += bias.reshape(1, F, 1, 1)
    return out.reshape(N, F * P * Q), P, Q


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("case", [(2, 3, 7, 6, 4, 3, 2, 1, 1, 1, 0), (1, 2, 9, 9, 5, 3, 3, 2, 2, 1, 1), (3, 1, 5, 5, 2, 5, 5, 1, 1, 2, 2),
                                  (2, 4, 6, 8, 3, 1, 1, 1, 2, 0, 0)])
def test_conv_against_brute_force(dt, case):
    N, C, H, W, F, Hf, Wf, sh, sw, ph, pw = case
    rng = np.random.default_rng(sum(case))
    x = rng.standard_normal((N, C * H * W)).astype(dt)
    w = rng.standard_normal((F, C * Hf * Wf)).astype(dt)
    b = rng.standard_normal((F, 1)).astype(dt)
    st, got, oh, ow = orc.conv2d(x, w, b, N, C, H, W, Hf, Wf, sh, sw, ph, pw)
    exp, P, Q = _conv_brute(x.astype(np.float64), w, b.astype(np.float64), N, C, H, W, F, Hf, Wf, sh, sw, ph, pw)
    assert st == 0 and (oh, ow) == (P, Q)
    assert np.allclose(got, exp, rtol=1e-4 if dt == np.float32 else 1e-11, atol=1e-4 if dt == np.float32 else 1e-11)


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("case", [(2, 3, 6, 6, 2, 2, 2, 2, 0, 0), (1, 2, 7, 5, 3, 3, 1, 1, 1, 1), (2, 1, 8, 8, 3, 2, 2, 2, 1, 1)])
def test_maxpool_against_brute_force(dt, case):
    N, C, H, W, ph, pw, sh, sw, padh, padw = case
    rng = np.random.default_rng(sum(case))
    x = rng.standard_normal((N, C * H * W)).astype(dt)
    st, got, oh, ow = orc.maxpool(x, N, C, H, W, ph, pw, sh, sw, padh, padw)
    xp = np.zeros((N, C, H + 2 * padh, W + 2 * padw), dt)  # zero padding takes part, and the fold starts at 0
    xp[:, :, padh:padh + H, padw:padw + W] = x.reshape(N, C, H, W)
    P, Q = (H + 2 * padh - ph) // sw + 1, (W + 2 * padw - pw) // sh + 1  # the reference's swapped strides
    exp = np.zeros((N, C, P, Q), dt)
    for p in range(P):
        for q in range(Q):
            win = xp[:, :, p * sh:p * sh + ph, q * sw:q * sw + pw]
            exp[:, :, p, q] = np.maximum(0, win.max(axis=(2, 3)))
    assert st == 0 and (oh, ow) == (P, Q) and np.array_equal(got, exp.reshape(N, -1))


@pytest.mark.parametrize("dt", DT)
def test_channel_ops_and_softmax_closed_forms(dt):
    rng = np.random.default_rng(5)
    N, C, HW = 4, 3, 10
    x = rng.standard_normal((N, C * HW)).astype(dt)
    b = rng.standard_normal((C, 1)).astype(dt)
    assert np.array_equal(orc.bias_add(x, b)[1], (x.reshape(N, C, HW) + b.reshape(1, C, 1)).reshape(N, -1))
    g, be, mu, var = (rng.random((C, 1)).astype(dt) + 0.5 for _ in range(4))
    exp = (g.reshape(1, C, 1) * (x.reshape(N, C, HW) - mu.reshape(1, C, 1)) / np.sqrt(var.reshape(1, C, 1) + dt(1e-5))
           + be.reshape(1, C, 1)).reshape(N, -1)
    assert np.allclose(orc.batchnorm(x, g, be, mu, var, 1e-5, 0)[1], exp, rtol=1e-5 if dt == np.float32 else 1e-13)
    gi, bi, mi, vi = (rng.random((N, 1)).astype(dt) + 0.5 for _ in range(4))
    exp = gi * (x - mi) / np.sqrt(vi + dt(1e-5)) + bi  # statistics per row, the reference's CPU loop
    assert np.allclose(orc.batchnorm(x, gi, bi, mi, vi, 1e-5, 1)[1], exp, rtol=1e-5 if dt == np.float32 else 1e-13)
    s = orc.softmax(x * 5)[1]
    assert np.allclose(s, scipy.special.softmax(x.astype(np.float64) * 5, axis=1), rtol=1e-5 if dt == np.float32 else 1e-13)
    assert np.allclose(s.sum(axis=1), 1.0, rtol=1e-5)


def test_vectorized_engine_equals_plain_kernels():
    """The multithreaded row-split engine gives what the plain kernels give on the whole matrix
    (reference: test/runtime/local/vectorized/MultiThreadedKernelTest.cpp:41-154)."""
    rng = np.random.default_rng(6)
    x = (rng.standard_normal((5000, 64)) * 2 + 5).astype(np.float32)
    st, mu, sd, r, s, _ = orc.zscore_pipeline(x, threads=5, thr=64.0)
    mu1 = orc.agg_col(6, x)[1]
    sd1 = orc.ew_unary(3, orc.agg_col(8, x)[1])[1]
    z = orc.ew_binary(3, orc.ew_binary(1, x, mu1)[1], sd1)[1]
    r1 = orc.agg_row(0, orc.ew_binary(2, z, z)[1])[1]
    assert np.array_equal(mu, mu1) and np.array_equal(sd, sd1) and np.array_equal(r, r1)
    assert s == float((r1 > 64.0).sum())
    for threads in (1, 2, 7):
        assert np.array_equal(orc.zscore_pipeline(x, threads=threads, thr=64.0)[3], r1)


# ---------------------------------------------------------------------------------------------------
# data reorganisation, ReLU and average pooling: numpy definitions and brute force
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_reorg_kernels_against_numpy(dt):
    rng = np.random.default_rng(11)
    a, b = rng.standard_normal((13, 7)).astype(dt), rng.standard_normal((13, 4)).astype(dt)
    assert np.array_equal(orc.transpose(a)[1], a.T)
    assert np.array_equal(orc.col_bind(a, b)[1], np.hstack([a, b]))
    assert orc.col_bind(a, b[:5])[0] == orc.ST_RUNTIME
    sel = np.array([[6], [-7], [0], [3], [3]], dtype=np.int64)
    assert np.array_equal(orc.extract_col(a, sel)[1], a[:, [6, 0, 0, 3, 3]])
    assert orc.extract_col(a, np.array([[7]], dtype=np.int64))[0] == 6
    assert orc.extract_col(a, np.array([[-8]], dtype=np.int64))[0] == 6
    assert orc.extract_col(a, np.zeros((2, 2), np.int64))[0] == orc.ST_RUNTIME
    assert np.array_equal(orc.fill(2.5, 4, 3, dt)[1], np.full((4, 3), 2.5, dt))
    assert orc.fill(1.0, 0, 3, dt)[1].shape == (0, 3)
    x = a.copy()
    x[0, :3] = [np.nan, -0.0, -np.inf]
    r = orc.relu(x)[1]
    assert np.isnan(r[0, 0]) and r[0, 2] == 0 and np.array_equal(r[1:], np.maximum(x[1:], 0))
    v = rng.standard_normal((13, 1)).astype(dt)
    np.testing.assert_allclose(orc.gemv(a, v)[1], a.T.astype(np.float64) @ v.astype(np.float64), rtol=1e-5 if dt == np.float32 else 1e-12,
                               atol=1e-5 if dt == np.float32 else 1e-12)


@pytest.mark.parametrize("p", [(2, 3, 5, 5, 2, 2, 2, 2, 1, 1), (1, 2, 6, 7, 3, 2, 1, 1, 0, 0), (2, 1, 9, 8, 2, 3, 3, 2, 1, 2),
                               (2, 2, 4, 1, 3, 1, 1, 1, 0, 0)])
def test_avgpool_brute_force(p):
    """Mean over the window of the zero-padded image with the FULL window as divisor (Pooling.cpp:50); output extents
    with the swapped strides of Pooling.cpp:38-39; the one-column quick path sums the first min(pool_h, H) values."""
    N, C_, H, W, ph, pw, sh, sw, padh, padw = p
    rng = np.random.default_rng(sum(p))
    x = rng.standard_normal((N, C_ * H * W))
    st, got, oh, ow = orc.avgpool(x, *p)
    P, Q = (H + 2 * padh - ph) // sw + 1, (W + 2 * padw - pw) // sh + 1
    assert st == 0 and (oh, ow) == (P, Q)
    img = np.pad(x.reshape(N, C_, H, W), ((0, 0), (0, 0), (padh, padh), (padw, padw)))
    exp = np.zeros((N, C_, P, Q))
    if P == 1 and Q == 1 and W == 1:
        exp[:, :, 0, 0] = x.reshape(N, C_, H)[:, :, :min(ph, H)].sum(axis=2) / (ph * pw)
    else:
        for i in range(P):
            for j in range(Q):
                exp[:, :, i, j] = img[:, :, i * sh:i * sh + ph, j * sw:j * sw + pw].sum(axis=(2, 3)) / (ph * pw)
    np.testing.assert_allclose(got, exp.reshape(N, -1), rtol=1e-12, atol=1e-12)


INT_TYPES = [np.int64, np.uint64, np.int32, np.uint32]


@pytest.mark.parametrize("dt", INT_TYPES, ids=["si64", "ui64", "si32", "ui32"])
def test_integer_elementwise_against_exact_python_arithmetic(dt):
    """The integer instantiations are pinned by Python's exact integers: + - * wrap modulo 2^bits, / truncates toward
    zero, MOD keeps the sign of the dividend (fmod), POW is the exact power where it fits, comparisons give 0 / 1."""
    rng = np.random.default_rng(5)
    info = np.iinfo(dt)
    signed = info.min < 0
    bits = info.bits
    lo = -50 if signed else 0
    a = rng.integers(lo, 50, (7, 9)).astype(dt)
    b = rng.integers(lo, 50, (7, 9)).astype(dt)
    b[b == 0] = 3
    big = rng.integers(info.max // 2, info.max, (7, 9), dtype=np.uint64 if not signed else np.int64).astype(dt)

    def wrap(v):
        v &= (1 << bits) - 1
        return v - (1 << bits) if signed and v >= 1 << (bits - 1) else v

    def table(f, x, y):
        return np.array([[f(int(p), int(q)) for p, q in zip(r, s)] for r, s in zip(x, y)], dtype=object)

    def tdiv(p, q):
        return abs(p) // abs(q) * (1 if (p < 0) == (q < 0) else -1)

    cases = {0: lambda p, q: wrap(p + q), 1: lambda p, q: wrap(p - q), 2: lambda p, q: wrap(p * q), 3: tdiv,
             5: lambda p, q: p - q * tdiv(p, q), 7: lambda p, q: int(p == q), 8: lambda p, q: int(p != q),
             9: lambda p, q: int(p < q), 10: lambda p, q: int(p <= q), 11: lambda p, q: int(p > q),
             12: lambda p, q: int(p >= q), 13: min, 14: max, 15: lambda p, q: int(bool(p) and bool(q)),
             16: lambda p, q: int(bool(p) or bool(q))}
    for op, f in cases.items():
        for x, y in ((a, b), (big, b)) if op in (0, 1, 2, 13, 14) else ((a, b),):
            st, got = orc.ew_binary(op, x, y)
            assert st == orc.ST_OK
            want = table(f, x, y)
            assert np.array_equal(got.astype(object), want), (op, dt)
        s = 7
        st, got = orc.ew_binary_sca(op, a, s)
        assert st == orc.ST_OK and np.array_equal(got.astype(object), table(f, a, np.full(a.shape, s, dtype=dt)))
    # POW: exact where it fits 53 bits; a negative exponent truncates to 0 (or +-1 for bases +-1)
    base = rng.integers(lo // 10, 6, (5, 5)).astype(dt)
    ex = rng.integers(0, 9, (5, 5)).astype(dt)
    st, got = orc.ew_binary(4, base, ex)
    assert st == orc.ST_OK and np.array_equal(got.astype(object), table(lambda p, q: wrap(p ** q), base, ex))
    # row- and column-vector broadcasts take the same scalar path
    st, got = orc.ew_binary(0, a, b[:1])
    assert np.array_equal(got, a + b[:1])
    st, got = orc.ew_binary(2, a, b[:, :1])
    assert np.array_equal(got, a * b[:, :1])
    # what would trap in the reference's process is a domain error here: x / 0, x mod 0, and INT_MIN / -1
    z = b.copy()
    z[2, 3] = 0
    assert orc.ew_binary(3, a, z)[0] == orc.ST_DOMAIN and orc.ew_binary(5, a, z)[0] == orc.ST_DOMAIN
    assert orc.ew_binary_sca(3, a, 0)[0] == orc.ST_DOMAIN
    if signed:
        m = a.copy()
        m[0, 0] = info.min
        assert orc.ew_binary_sca(3, m, -1)[0] == orc.ST_DOMAIN
        assert orc.ew_binary_sca(5, m, -1)[0] == orc.ST_OK  # fmod is defined there


def test_si64_aggregations_against_numpy():
    rng = np.random.default_rng(6)
    x = rng.integers(-1000, 1000, (37, 23)).astype(np.int64)
    x[5, 7] = np.iinfo(np.int64).max
    x[9, 2] = np.iinfo(np.int64).min
    for op, f in ((0, np.sum), (2, np.min), (3, np.max)):
        with np.errstate(over="ignore"):
            assert orc.agg_all(op, x) == (orc.ST_OK, f(x))
            st, r = orc.agg_row(op, x)
            assert st == orc.ST_OK and np.array_equal(r[:, 0], f(x, axis=1))
            st, c = orc.agg_col(op, x)
            assert st == orc.ST_OK and np.array_equal(c[0], f(x, axis=0))
    small = rng.integers(-3, 4, (6, 5)).astype(np.int64)
    assert orc.agg_all(1, small)[1] == np.prod(small)
    ties = rng.integers(0, 4, (50, 12)).astype(np.int64)  # many ties: the first one wins
    assert np.array_equal(orc.agg_row(4, ties)[1][:, 0], np.argmin(ties, axis=1))
    assert np.array_equal(orc.agg_row(5, ties)[1][:, 0], np.argmax(ties, axis=1))
    assert np.array_equal(orc.agg_col(4, ties)[1][0], np.argmin(ties, axis=0))
    assert np.array_equal(orc.agg_col(5, ties)[1][0], np.argmax(ties, axis=0))
    v = x[3:30, 4:20]  # a view: row stride larger than the width
    assert orc.agg_all(0, v)[1] == v.sum() and np.array_equal(orc.agg_col(3, v)[1][0], v.max(axis=0))
    # data reorganisation of 64-bit integers
    assert np.array_equal(orc.transpose(x)[1], x.T)
    assert np.array_equal(orc.col_bind(x, ties[:37])[1], np.hstack([x, ties[:37]]))
    assert np.array_equal(orc.extract_col(x, np.array([[3], [0], [-1]]))[1], x[:, [3, 0, -1]])
    assert np.array_equal(orc.fill(-5, 3, 4, np.int64)[1], np.full((3, 4), -5, np.int64))
    assert np.array_equal(orc.fill(2 ** 63 + 1, 2, 2, np.uint64)[1], np.full((2, 2), 2 ** 63 + 1, np.uint64))


# -- DNN training kernels: pinned by calculus and linear algebra, independent of the restated loops ----------
def _conv_fwd(x, w, N, C, H, W, F, Hf, Wf, sh, sw, ph, pw):
    st, out, P, Q = orc.conv2d(x, w, np.zeros((F, 1), x.dtype), N, C, H, W, Hf, Wf, sh, sw, ph, pw)
    assert st == orc.ST_OK
    return out, P, Q


@pytest.mark.parametrize("case", [(2, 3, 7, 6, 4, 3, 3, 1, 1, 1, 1), (1, 2, 9, 8, 3, 2, 3, 2, 1, 0, 1), (3, 1, 5, 5, 2, 5, 5, 1, 1, 2, 2),
                                  (2, 2, 8, 8, 2, 3, 2, 2, 3, 1, 0), (1, 3, 3, 3, 2, 2, 2, 2, 2, 1, 1)])
def test_conv_backward_is_the_adjoint_of_the_forward_convolution(case):
    """<conv(x, w), dy> = <x, backward_data(w, dy)> = <w, backward_filter(x, dy)>: the convolution is bilinear, so both
    gradients are fixed by the forward kernel (itself pinned by the reference's vectors and brute force)."""
    N, C, H, W, F, Hf, Wf, sh, sw, ph, pw = case
    rng = np.random.default_rng(sum(case))
    x = rng.standard_normal((N, C * H * W))
    w = rng.standard_normal((F, C * Hf * Wf))
    y, P, Q = _conv_fwd(x, w, *case)
    dy = rng.standard_normal(y.shape)
    st, dx = orc.conv2d_backward_data(w, dy, *case)
    assert st == orc.ST_OK
    st, dw = orc.conv2d_backward_filter(x, dy, *case)
    assert st == orc.ST_OK
    lhs = float((y * dy).sum())
    assert abs(lhs - float((x * dx).sum())) <= 1e-10 * max(1.0, abs(lhs))
    assert abs(lhs - float((w * dw).sum())) <= 1e-10 * max(1.0, abs(lhs))
    # and each single gradient entry is the forward result of a unit impulse
    e = np.zeros_like(x)
    e[0, 5] = 1.0
    ye, _, _ = _conv_fwd(e, w, *case)
    assert abs(float((ye * dy).sum()) - dx[0, 5]) <= 1e-12 * max(1.0, abs(dx[0, 5]))


@pytest.mark.parametrize("p", [(2, 3, 6, 6, 2, 2, 2, 2, 0, 0), (1, 2, 7, 5, 3, 3, 1, 1, 1, 1), (2, 1, 8, 8, 3, 2, 2, 2, 1, 0),
                               (1, 1, 5, 5, 2, 2, 1, 1, 0, 0)])
def test_pooling_backward_against_adjoint_and_brute_force(p):
    N, C, H, W, ph, pw, sh, sw, padh, padw = p
    rng = np.random.default_rng(sum(p))
    x = rng.permutation(N * C * H * W).astype(np.float64).reshape(N, C * H * W) + 1.0  # distinct, positive: unique maxima
    st, y, P, Q = orc.avgpool(x, *p)
    assert st == orc.ST_OK
    dy = rng.standard_normal(y.shape)
    # average pooling is linear: its backward pass is the adjoint
    st, dx = orc.avgpool_backward(x, dy, *p)
    assert st == orc.ST_OK
    assert abs(float((y * dy).sum()) - float((x * dx).sum())) <= 1e-10 * max(1.0, abs(float((y * dy).sum())))
    # max pooling: every window sends its gradient to the position of its maximum (brute force on the padded image)
    st, dxm = orc.maxpool_backward(x, dy, *p)
    assert st == orc.ST_OK
    want = np.zeros((N, C, H + 2 * padh, W + 2 * padw))
    xp = np.zeros_like(want)
    xp[:, :, padh:padh + H, padw:padw + W] = x.reshape(N, C, H, W)
    d4 = dy.reshape(N, C, P, Q)
    for n in range(N):
        for c in range(C):
            for a in range(P):
                for b in range(Q):
                    win = xp[n, c, a * sh:a * sh + ph, b * sw:b * sw + pw]
                    if win.shape != (ph, pw):
                        continue
                    i, j = np.unravel_index(np.argmax(win), win.shape)  # first maximum in row-major order
                    want[n, c, a * sh + i, b * sw + j] += d4[n, c, a, b]
    np.testing.assert_allclose(dxm.reshape(N, C, H, W), want[:, :, padh:padh + H, padw:padw + W], rtol=0, atol=1e-12)


def test_batchnorm_training_against_numpy_and_finite_differences():
    rng = np.random.default_rng(8)
    N, C, HW = 5, 3, 7
    x = rng.standard_normal((N, C * HW)) * 2 + 1
    gamma, beta = rng.random((C, 1)) + 0.5, rng.standard_normal((C, 1))
    em, ev = rng.standard_normal((C, 1)), rng.random((C, 1)) + 0.5
    eps, mu = 1e-5, 0.3
    st, res, nm, nv, mean, iv = orc.batchnorm_train_forward(x, gamma, beta, em, ev, eps, mu)
    assert st == orc.ST_OK
    xc = x.reshape(N, C, HW).transpose(1, 0, 2).reshape(C, -1)
    m, v = xc.mean(axis=1, keepdims=True), xc.var(axis=1, keepdims=True)
    np.testing.assert_allclose(mean, m, rtol=1e-12)
    np.testing.assert_allclose(iv, 1 / np.sqrt(v + eps), rtol=1e-12)
    np.testing.assert_allclose(nm, (1 - mu) * em + mu * m, rtol=1e-12)
    np.testing.assert_allclose(nv, (1 - mu) * ev + mu * v, rtol=1e-12)
    want = (gamma * (xc - m) / np.sqrt(v + eps) + beta).reshape(C, N, HW).transpose(1, 0, 2).reshape(N, C * HW)
    np.testing.assert_allclose(res, want, rtol=1e-11, atol=1e-12)

    # backward: gradient of L = <dout, BN(x)> by central differences, through the forward kernel itself
    dout = rng.standard_normal(x.shape)
    st, dX, dG, dB = orc.batchnorm_backward(mean, iv, x, dout, gamma)
    assert st == orc.ST_OK

    def loss(xx, gg, bb):
        return float((orc.batchnorm_train_forward(xx, gg, bb, em, ev, eps, mu)[1] * dout).sum())

    h = 1e-6
    for (i, j) in ((0, 0), (2, 9), (4, 20), (1, 13)):
        xp, xm = x.copy(), x.copy()
        xp[i, j] += h
        xm[i, j] -= h
        assert abs((loss(xp, gamma, beta) - loss(xm, gamma, beta)) / (2 * h) - dX[i, j]) <= 1e-6 * max(1.0, abs(dX[i, j]))
    for c in range(C):
        gp, gm = gamma.copy(), gamma.copy()
        gp[c] += h
        gm[c] -= h
        assert abs((loss(x, gp, beta) - loss(x, gm, beta)) / (2 * h) - dG[c, 0]) <= 1e-6 * max(1.0, abs(dG[c, 0]))
        bp, bm = beta.copy(), beta.copy()
        bp[c] += h
        bm[c] -= h
        assert abs((loss(x, gamma, bp) - loss(x, gamma, bm)) / (2 * h) - dB[c, 0]) <= 1e-6 * max(1.0, abs(dB[c, 0]))
