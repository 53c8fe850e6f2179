"""GPU parity: elementwise and aggregation kernels (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest

import oracle_binding as orc
from parity import assert_close, assert_exact, variance_floor

pytestmark = pytest.mark.gpu

from daphne_amd import capi
from daphne_amd.kernels import (AggOpCode, BinaryOpCode, DenseMatrix, UnaryOpCode, aggAll, aggCol, aggRow,
                                ewBinaryMat, ewBinaryObjSca, ewUnaryMat)

DTYPES = [np.float32, np.float64]
EXACT_BIN = {BinaryOpCode.ADD, BinaryOpCode.SUB, BinaryOpCode.MUL, BinaryOpCode.DIV, BinaryOpCode.EQ,
             BinaryOpCode.NEQ, BinaryOpCode.LT, BinaryOpCode.LE, BinaryOpCode.GT, BinaryOpCode.GE, BinaryOpCode.MIN,
             BinaryOpCode.MAX, BinaryOpCode.AND, BinaryOpCode.OR, BinaryOpCode.MOD}
FP_BIN = [BinaryOpCode(i) for i in range(17)]
EXACT_UN = {UnaryOpCode.MINUS, UnaryOpCode.ABS, UnaryOpCode.SIGN, UnaryOpCode.SQRT, UnaryOpCode.FLOOR,
            UnaryOpCode.CEIL, UnaryOpCode.ROUND, UnaryOpCode.ISNAN}


def _rand(rng, shape, dt, special=True):
    a = rng.standard_normal(shape).astype(dt) * 3
    if special and a.size >= 16:
        flat = a.reshape(-1)
        flat[1] = np.nan
        flat[3] = np.inf
        flat[5] = -np.inf
        flat[7] = 0.0
        flat[9] = -0.0
        flat[11] = flat[10]
    return a


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op", FP_BIN)
@pytest.mark.parametrize("shape", [(37, 64), (5, 7), (1, 1000), (1000, 1), (130, 3)])
def test_ew_binary_same_shape(ctx, dt, op, shape):
    rng = np.random.default_rng(hash((int(op), shape)) % 2**32)
    a, b = _rand(rng, shape, dt), _rand(rng, shape, dt)
    if op in (BinaryOpCode.POW, BinaryOpCode.LOG):
        a = np.abs(a) + dt(0.5)
    st, exp = orc.ew_binary(op, a, b)
    assert st == 0
    got = ewBinaryMat(op, None, DenseMatrix.from_numpy(ctx, a), DenseMatrix.from_numpy(ctx, b), ctx).to_numpy()
    (assert_exact if op in EXACT_BIN else assert_close)(got, exp)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op", [BinaryOpCode.ADD, BinaryOpCode.SUB, BinaryOpCode.DIV, BinaryOpCode.MIN,
                                BinaryOpCode.GE, BinaryOpCode.POW])
@pytest.mark.parametrize("shape", [(1000, 64), (33, 5), (2, 1026), (4097, 16)])
def test_ew_binary_broadcast(ctx, dt, op, shape):
    rng = np.random.default_rng(7)
    a = _rand(rng, shape, dt)
    if op == BinaryOpCode.POW:
        a = np.abs(a) + dt(0.5)
    rowv = _rand(rng, (1, shape[1]), dt, special=False)
    colv = _rand(rng, (shape[0], 1), dt, special=False)
    A = DenseMatrix.from_numpy(ctx, a)
    for v in (rowv, colv):
        st, exp = orc.ew_binary(op, a, v)
        assert st == 0
        got = ewBinaryMat(op, None, A, DenseMatrix.from_numpy(ctx, v), ctx).to_numpy()
        (assert_exact if op in EXACT_BIN else assert_close)(got, exp)


@pytest.mark.parametrize("dt", DTYPES)
def test_ew_binary_views_and_inplace(ctx, dt):
    """rowSkip > numCols on every operand (views), and res aliasing lhs."""
    rng = np.random.default_rng(3)
    big_a, big_b = _rand(rng, (50, 40), dt), _rand(rng, (50, 40), dt)
    A, B = DenseMatrix.from_numpy(ctx, big_a), DenseMatrix.from_numpy(ctx, big_b)
    for (r0, r1, c0, c1) in [(3, 47, 4, 36), (0, 50, 1, 2), (10, 11, 0, 40), (5, 25, 3, 30)]:
        va, vb = big_a[r0:r1, c0:c1], big_b[r0:r1, c0:c1]
        st, exp = orc.ew_binary(BinaryOpCode.MUL, va, vb)
        got = ewBinaryMat(BinaryOpCode.MUL, None, A.slice(r0, r1, c0, c1), B.slice(r0, r1, c0, c1), ctx).to_numpy()
        assert_exact(got, exp)
    # in place: res == lhs, on a view
    C = DenseMatrix.from_numpy(ctx, big_a)
    v = C.slice(2, 40, 4, 36)
    ewBinaryMat(BinaryOpCode.ADD, v, v, B.slice(2, 40, 4, 36), ctx)
    exp = big_a.copy()
    exp[2:40, 4:36] = big_a[2:40, 4:36] + big_b[2:40, 4:36]
    assert_exact(C.to_numpy(), exp)


@pytest.mark.parametrize("dt", DTYPES)
def test_ew_binary_errors(ctx, dt):
    a = DenseMatrix.from_numpy(ctx, np.ones((4, 5), dt))
    b = DenseMatrix.from_numpy(ctx, np.ones((3, 5), dt))
    with pytest.raises(capi.DaphneHipError, match="lhs and rhs must either have the same dimensions"):
        ewBinaryMat(BinaryOpCode.ADD, None, a, b, ctx)
    with pytest.raises(capi.DaphneHipError, match="unknown BinaryOpCode"):
        ewBinaryMat(999, None, a, a, ctx)
    with pytest.raises(capi.DaphneHipError, match="not supported on the value types"):
        ewBinaryMat(BinaryOpCode.BITWISE_AND, None, a, a, ctx)
    with pytest.raises(capi.DaphneHipError, match="unknown UnaryOpCode"):
        ewUnaryMat(999, None, a, ctx)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op", FP_BIN)
def test_ew_binary_scalar(ctx, dt, op):
    rng = np.random.default_rng(11)
    for shape in [(513, 16), (1, 1), (77, 3)]:
        a = _rand(rng, shape, dt)
        s = 1.75
        if op in (BinaryOpCode.POW, BinaryOpCode.LOG):
            a = np.abs(a) + dt(0.5)
        st, exp = orc.ew_binary_sca(op, a, s)
        got = ewBinaryObjSca(op, None, DenseMatrix.from_numpy(ctx, a), s, ctx).to_numpy()
        (assert_exact if op in EXACT_BIN else assert_close)(got, exp)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op", [UnaryOpCode(i) for i in range(19)])
def test_ew_unary(ctx, dt, op):
    rng = np.random.default_rng(int(op))
    for shape in [(64, 64), (3, 1000), (1, 7)]:
        a = rng.standard_normal(shape).astype(dt)
        if op in (UnaryOpCode.SQRT, UnaryOpCode.LN):
            a = np.abs(a)
            a.reshape(-1)[0] = 0.0
            a.reshape(-1)[1] = -0.0
            a.reshape(-1)[2] = np.nan
        elif op in (UnaryOpCode.ASIN, UnaryOpCode.ACOS):
            a = np.clip(a, -1, 1)
        else:
            a.reshape(-1)[:6] = [np.nan, np.inf, -np.inf, 0.0, -0.0, 2.5]
        if op in (UnaryOpCode.SIN, UnaryOpCode.COS, UnaryOpCode.TAN):
            a[np.isinf(a)] = 1.0
        st, exp = orc.ew_unary(op, a)
        assert st == 0
        got = ewUnaryMat(op, None, DenseMatrix.from_numpy(ctx, a), ctx).to_numpy()
        if op in EXACT_UN:
            assert_exact(got, exp)
        elif op == UnaryOpCode.TAN:
            assert_close(got, exp, rtol=1e-4 if dt == np.float32 else 1e-9)
        else:
            assert_close(got, exp)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op,bad", [(UnaryOpCode.SQRT, -1.0), (UnaryOpCode.LN, -1e-30), (UnaryOpCode.ASIN, 1.5),
                                    (UnaryOpCode.ACOS, -1.0001)])
@pytest.mark.parametrize("shape", [(100, 33), (300, 40), (1, 64)])  # one workgroup that also sets the flag; the large kernel
def test_ew_unary_domain_error(ctx, dt, op, bad, shape):
    a = np.full(shape, 0.5, dt)
    a[shape[0] * 3 // 4, 20] = bad
    st, _ = orc.ew_unary(op, a)
    assert st == orc.ST_DOMAIN
    with pytest.raises(capi.DaphneHipDomainError, match="invalid argument"):
        ewUnaryMat(op, None, DenseMatrix.from_numpy(ctx, a), ctx)
    # the flag is cleared again for the next call
    a[shape[0] * 3 // 4, 20] = 0.25
    d = DenseMatrix.from_numpy(ctx, a)
    assert_close(ewUnaryMat(op, d, d, ctx).to_numpy(), orc.ew_unary(op, a)[1])  # in place


AGG_VALUE_OPS = [AggOpCode.SUM, AggOpCode.PROD, AggOpCode.MIN, AggOpCode.MAX, AggOpCode.MEAN, AggOpCode.STDDEV,
                 AggOpCode.VAR]
AGG_SHAPES = [(1000, 64), (7, 5), (1, 300), (300, 1), (4100, 16), (3, 1030), (50000, 4), (33, 6), (100, 12), (64, 22), (257, 66)]


def _agg_input(rng, shape, dt, op):
    if op == AggOpCode.PROD:
        return (1.0 + 0.01 * rng.standard_normal(shape)).astype(dt)
    return (rng.standard_normal(shape) * 2 + 5).astype(dt)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op", AGG_VALUE_OPS)
@pytest.mark.parametrize("shape", AGG_SHAPES)
def test_agg_row_col_all(ctx, dt, op, shape):
    rng = np.random.default_rng(shape[0] * 31 + shape[1])
    a = _agg_input(rng, shape, dt, op)
    A = DenseMatrix.from_numpy(ctx, a)
    exact = op in (AggOpCode.MIN, AggOpCode.MAX)
    cmp = assert_exact if exact else assert_close
    # item by item at the stated relative tolerance; a variance that is (nearly) zero - one value per row or
    # column - is compared against the rounding noise of its own computation instead of against itself
    kw = {}
    if op in (AggOpCode.VAR, AggOpCode.STDDEV):
        kw = {"atol": variance_floor(a, op == AggOpCode.STDDEV)}
    st, exp = orc.agg_row(op, a)
    cmp(aggRow(op, None, A, ctx).to_numpy(), exp, **kw)
    st, exp = orc.agg_col(op, a)
    cmp(aggCol(op, None, A, ctx).to_numpy(), exp, **kw)
    st, exp = orc.agg_all(op, a)
    got = aggAll(op, A, ctx)
    cmp(np.array([got]), np.array([exp]))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op", [o for o in AGG_VALUE_OPS if o != AggOpCode.PROD])  # 300000 float factors: rounding alone exceeds 1e-4
@pytest.mark.parametrize("shape,ld", [((1, 300_000), 300_000), ((3, 70_001), 70_016), ((16, 65_536), 65_536)])
def test_agg_row_of_a_few_very_wide_rows(ctx, dt, op, shape, ld):
    """A 1 x N vector and other few-row, very wide matrices: every row is spread over the device (for SUM, PROD and
    the moments), also through a view with a row stride; the result must be the row aggregate all the same."""
    rng = np.random.default_rng(shape[1])
    base = np.zeros((shape[0], ld), dt)
    base[:, :shape[1]] = _agg_input(rng, shape, dt, op)
    a = base[:, :shape[1]]
    A = DenseMatrix.from_numpy(ctx, base).slice(0, shape[0], 0, shape[1])
    kw = {"atol": variance_floor(a, op == AggOpCode.STDDEV)} if op in (AggOpCode.VAR, AggOpCode.STDDEV) else {}
    st, exp = orc.agg_row(op, np.ascontiguousarray(a))
    (assert_exact if op in (AggOpCode.MIN, AggOpCode.MAX) else assert_close)(aggRow(op, None, A, ctx).to_numpy(), exp, **kw)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op", [AggOpCode.IDXMIN, AggOpCode.IDXMAX])
@pytest.mark.parametrize("shape", [(2000, 16), (7, 5), (1, 300), (300, 1), (513, 64), (3, 1030), (9, 130), (33, 6), (100, 12),
                                   (64, 22), (257, 66)])
def test_agg_idx_bit_exact(ctx, dt, op, shape):
    rng = np.random.default_rng(shape[0] + 7 * shape[1])
    # few distinct values -> many ties; plus NaN / inf rows
    a = rng.integers(0, 6, shape).astype(dt)
    if shape[0] >= 7 and shape[1] >= 5:
        a[0, :] = np.nan
        a[1, 0] = np.nan
        a[2, 1:] = np.nan
        a[3, :] = np.inf
        a[4, :] = -np.inf
        a[5, 2] = np.nan
        a[6, :] = 3.0
    A = DenseMatrix.from_numpy(ctx, a)
    st, exp = orc.agg_row(op, a)
    got = aggRow(op, None, A, ctx).to_numpy()
    assert got.dtype == np.uint64
    assert_exact(got, exp)
    st, exp = orc.agg_col(op, a)
    assert_exact(aggCol(op, None, A, ctx).to_numpy(), exp)


@pytest.mark.parametrize("dt", DTYPES)
def test_agg_minmax_nan_rules(ctx, dt):
    """NaN in the first element is the result of row/col MIN/MAX; elsewhere it is ignored; AggAll
    ignores NaN altogether (the reference builds these on std::min / std::max)."""
    a = np.arange(40, dtype=dt).reshape(5, 8) + 1
    a[0, 0] = np.nan
    a[1, 3] = np.nan
    a[3, 0] = np.nan
    A = DenseMatrix.from_numpy(ctx, a)
    for op in (AggOpCode.MIN, AggOpCode.MAX):
        assert_exact(aggRow(op, None, A, ctx).to_numpy(), orc.agg_row(op, a)[1])
        assert_exact(aggCol(op, None, A, ctx).to_numpy(), orc.agg_col(op, a)[1])
        assert_exact(np.array([aggAll(op, A, ctx)]), np.array([orc.agg_all(op, a)[1]]))


@pytest.mark.parametrize("dt", DTYPES)
def test_agg_on_views(ctx, dt):
    rng = np.random.default_rng(5)
    big = (rng.standard_normal((300, 70)) + 2).astype(dt)
    B = DenseMatrix.from_numpy(ctx, big)
    for (r0, r1, c0, c1) in [(3, 290, 4, 68), (0, 300, 1, 2), (10, 11, 0, 70), (5, 250, 3, 35)]:
        v, V = big[r0:r1, c0:c1], B.slice(r0, r1, c0, c1)
        for op in (AggOpCode.SUM, AggOpCode.MAX, AggOpCode.MEAN, AggOpCode.VAR):
            cmp = assert_exact if op == AggOpCode.MAX else assert_close
            kw = {"atol": variance_floor(v)} if op == AggOpCode.VAR else {}
            cmp(aggRow(op, None, V, ctx).to_numpy(), orc.agg_row(op, v)[1], **kw)
            cmp(aggCol(op, None, V, ctx).to_numpy(), orc.agg_col(op, v)[1], **kw)
            cmp(np.array([aggAll(op, V, ctx)]), np.array([orc.agg_all(op, v)[1]]))
        assert_exact(aggRow(AggOpCode.IDXMIN, None, V, ctx).to_numpy(), orc.agg_row(AggOpCode.IDXMIN, v)[1])


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("shape", AGG_SHAPES + [(200000, 64)])
def test_agg_col_moments_one_pass(ctx, dt, shape):
    """Column means and variances from one pass equal the two separate aggregations (oracle: AggCol MEAN / VAR / STDDEV)."""
    from daphne_amd.kernels import aggColMoments
    rng = np.random.default_rng(shape[0] + 3 * shape[1])
    a = (rng.standard_normal(shape) * 2 + 5).astype(dt)
    A = DenseMatrix.from_numpy(ctx, a)
    mean, var = aggColMoments(A, ctx)
    _, sd = aggColMoments(A, ctx, stddev=True)
    truth_mean, truth_var = a.astype(np.float64).mean(axis=0, keepdims=True), a.astype(np.float64).var(axis=0, keepdims=True)
    assert_close(mean.to_numpy(), truth_mean.astype(dt))
    assert_close(var.to_numpy(), truth_var.astype(dt), atol=variance_floor(a))
    assert_close(sd.to_numpy(), np.sqrt(truth_var).astype(dt), atol=variance_floor(a, True))
    if shape[0] <= 50000:
        assert_close(mean.to_numpy(), orc.agg_col(AggOpCode.MEAN, a)[1])
        assert_close(var.to_numpy(), orc.agg_col(AggOpCode.VAR, a)[1], atol=variance_floor(a))
    # the same numbers as the separate device kernels
    assert_close(mean.to_numpy(), aggCol(AggOpCode.MEAN, None, A, ctx).to_numpy())
    assert_exact(var.to_numpy(), aggCol(AggOpCode.VAR, None, A, ctx).to_numpy())
    # a view
    if shape[0] > 10 and shape[1] > 4:
        v, V = a[3:-2, 1:-1], A.slice(3, shape[0] - 2, 1, shape[1] - 1)
        m2, v2 = aggColMoments(V, ctx)
        assert_close(m2.to_numpy(), v.astype(np.float64).mean(axis=0, keepdims=True).astype(dt))
        assert_close(v2.to_numpy(), v.astype(np.float64).var(axis=0, keepdims=True).astype(dt), atol=variance_floor(v))
