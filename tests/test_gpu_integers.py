"""GPU parity, bit-exact: the integer instantiations (elementwise binary for si64 / ui64 / si32 / ui32, aggregations and
data reorganisation for si64) through the C ABI against the CPU oracle."""
import numpy as np
import pytest

import oracle_binding as orc
from parity import assert_exact

pytestmark = pytest.mark.gpu

from daphne_amd import capi
from daphne_amd.kernels import (AggOpCode, BinaryOpCode, DenseMatrix, aggAll, aggCol, aggRow, colBind, ewBinaryMat,
                                ewBinaryObjSca, ewUnaryMat, extractCol, fill, matMul, transpose)

INT_TYPES = [np.int64, np.uint64, np.int32, np.uint32]
IDS = ["si64", "ui64", "si32", "ui32"]
OPS = [BinaryOpCode(i) for i in range(17)]


def _ints(rng, shape, dt, wide=False):
    info = np.iinfo(dt)
    if wide:  # the whole range of the type: sums, products and differences wrap
        return rng.integers(info.min, info.max, shape, dtype=dt, endpoint=True)
    return rng.integers(-40 if info.min < 0 else 0, 40, shape).astype(dt)


def _operands(rng, op, shape, dt, rshape=None):
    rshape = rshape or shape
    wide = op in (BinaryOpCode.ADD, BinaryOpCode.SUB, BinaryOpCode.MUL, BinaryOpCode.MIN, BinaryOpCode.MAX,
                  BinaryOpCode.EQ, BinaryOpCode.LT, BinaryOpCode.GE)
    a, b = _ints(rng, shape, dt, wide), _ints(rng, rshape, dt, wide)
    if op in (BinaryOpCode.DIV, BinaryOpCode.MOD):
        b[b == 0] = 7
    if op == BinaryOpCode.POW:  # exact powers that fit 53 bits
        a = rng.integers(-6 if np.iinfo(dt).min < 0 else 0, 7, shape).astype(dt)
        b = rng.integers(0, 11, rshape).astype(dt)
    if op == BinaryOpCode.LOG:  # quotients of logarithms well away from an integer (the truncation is then unambiguous)
        a = rng.choice(np.array([3, 5, 6, 7, 10, 11, 30, 100, 1000], dtype=dt), shape)
        b = rng.choice(np.array([2, 4, 8], dtype=dt), rshape)
    return a, b


@pytest.mark.parametrize("dt", INT_TYPES, ids=IDS)
@pytest.mark.parametrize("op", OPS)
@pytest.mark.parametrize("shape", [(37, 64), (5, 7), (1, 1000), (1000, 1), (513, 24)])
def test_integer_ew_binary_same_shape(ctx, dt, op, shape):
    rng = np.random.default_rng(int(op) * 131 + shape[0])
    a, b = _operands(rng, op, shape, dt)
    st, exp = orc.ew_binary(op, a, b)
    assert st == 0
    got = ewBinaryMat(op, None, DenseMatrix.from_numpy(ctx, a), DenseMatrix.from_numpy(ctx, b), ctx).to_numpy()
    assert got.dtype == np.dtype(dt)
    assert_exact(got, exp)


@pytest.mark.parametrize("dt", INT_TYPES, ids=IDS)
@pytest.mark.parametrize("op", [BinaryOpCode.ADD, BinaryOpCode.MUL, BinaryOpCode.DIV, BinaryOpCode.MOD, BinaryOpCode.MAX,
                                BinaryOpCode.NEQ, BinaryOpCode.POW])
@pytest.mark.parametrize("shape", [(1000, 64), (33, 5), (2, 1026), (4097, 16)])
def test_integer_ew_binary_broadcast_and_scalar(ctx, dt, op, shape):
    rng = np.random.default_rng(11)
    a, rowv = _operands(rng, op, shape, dt, (1, shape[1]))
    _, colv = _operands(rng, op, shape, dt, (shape[0], 1))
    A = DenseMatrix.from_numpy(ctx, a)
    for v in (rowv, colv):
        st, exp = orc.ew_binary(op, a, v)
        assert st == 0
        assert_exact(ewBinaryMat(op, None, A, DenseMatrix.from_numpy(ctx, v), ctx).to_numpy(), exp)
    s = int(rowv[0, 0])
    st, exp = orc.ew_binary_sca(op, a, s)
    assert st == 0
    assert_exact(ewBinaryObjSca(op, None, A, s, ctx).to_numpy(), exp)


@pytest.mark.parametrize("dt", INT_TYPES, ids=IDS)
def test_integer_ew_views_and_inplace(ctx, dt):
    rng = np.random.default_rng(3)
    big_a, big_b = _ints(rng, (50, 40), dt, True), _ints(rng, (50, 40), dt, True)
    A, B = DenseMatrix.from_numpy(ctx, big_a), DenseMatrix.from_numpy(ctx, big_b)
    for (r0, r1, c0, c1) in [(3, 47, 4, 36), (0, 50, 1, 2), (10, 11, 0, 40), (5, 25, 3, 30)]:
        va, vb = big_a[r0:r1, c0:c1], big_b[r0:r1, c0:c1]
        st, exp = orc.ew_binary(BinaryOpCode.SUB, np.ascontiguousarray(va), np.ascontiguousarray(vb))
        got = ewBinaryMat(BinaryOpCode.SUB, None, A.slice(r0, r1, c0, c1), B.slice(r0, r1, c0, c1), ctx).to_numpy()
        assert_exact(got, exp)
    C = DenseMatrix.from_numpy(ctx, big_a)
    ewBinaryMat(BinaryOpCode.MUL, C, C, B, ctx)  # res aliases lhs
    with np.errstate(over="ignore"):
        assert_exact(C.to_numpy(), big_a * big_b)


@pytest.mark.parametrize("dt", INT_TYPES, ids=IDS)
def test_integer_division_by_zero_is_a_domain_error(ctx, dt):
    """Where the reference's process would stop with a hardware trap, the call reports a domain error."""
    rng = np.random.default_rng(4)
    a, b = _ints(rng, (300, 64), dt), _ints(rng, (300, 64), dt)
    b[b == 0] = 5
    A = DenseMatrix.from_numpy(ctx, a)
    ewBinaryMat(BinaryOpCode.DIV, None, A, DenseMatrix.from_numpy(ctx, b), ctx)  # fine
    z = b.copy()
    z[123, 45] = 0
    Z = DenseMatrix.from_numpy(ctx, z)
    for op in (BinaryOpCode.DIV, BinaryOpCode.MOD):
        assert orc.ew_binary(op, a, z)[0] == orc.ST_DOMAIN
        with pytest.raises(capi.DaphneHipDomainError):
            ewBinaryMat(op, None, A, Z, ctx)
        with pytest.raises(capi.DaphneHipDomainError):
            ewBinaryObjSca(op, None, A, 0, ctx)
    if np.iinfo(dt).min < 0:
        m = a.copy()
        m[7, 7] = np.iinfo(dt).min
        M = DenseMatrix.from_numpy(ctx, m)
        with pytest.raises(capi.DaphneHipDomainError):
            ewBinaryObjSca(BinaryOpCode.DIV, None, M, -1, ctx)
        st, exp = orc.ew_binary_sca(BinaryOpCode.MOD, m, -1)
        assert st == 0
        assert_exact(ewBinaryObjSca(BinaryOpCode.MOD, None, M, -1, ctx).to_numpy(), exp)
    # the context keeps working after the error
    assert_exact(ewBinaryObjSca(BinaryOpCode.ADD, None, A, 1, ctx).to_numpy(), a + np.array(1, dt))


def test_kernels_without_integer_instantiation_refuse(ctx):
    a = DenseMatrix.from_numpy(ctx, np.arange(12, dtype=np.int64).reshape(3, 4))
    with pytest.raises(capi.DaphneHipError):
        ewUnaryMat(0, None, a, ctx)
    with pytest.raises(capi.DaphneHipError):
        matMul(None, a, a, False, True, ctx)
    with pytest.raises(capi.DaphneHipError):
        ewBinaryMat(BinaryOpCode.ADD, None, a, DenseMatrix.from_numpy(ctx, np.ones((3, 4), np.int32)), ctx)
    for op in (AggOpCode.MEAN, AggOpCode.VAR, AggOpCode.STDDEV):
        with pytest.raises(capi.DaphneHipError):
            aggAll(op, a, ctx)
        with pytest.raises(capi.DaphneHipError):
            aggRow(op, None, a, ctx)
        with pytest.raises(capi.DaphneHipError):
            aggCol(op, None, a, ctx)


@pytest.mark.parametrize("shape", [(1000, 64), (4099, 16), (37, 5), (3, 1000), (20000, 3), (1, 1), (64, 130)])
def test_si64_aggregations(ctx, shape):
    rng = np.random.default_rng(shape[0] + shape[1])
    x = rng.integers(-10 ** 12, 10 ** 12, shape).astype(np.int64)
    x.reshape(-1)[rng.integers(0, x.size)] = np.iinfo(np.int64).max
    x.reshape(-1)[rng.integers(0, x.size)] = np.iinfo(np.int64).min
    X = DenseMatrix.from_numpy(ctx, x)
    for op in (AggOpCode.SUM, AggOpCode.MIN, AggOpCode.MAX):
        st, e = orc.agg_all(op, x)
        assert aggAll(op, X, ctx) == e
        assert_exact(aggRow(op, None, X, ctx).to_numpy(), orc.agg_row(op, x)[1])
        assert_exact(aggCol(op, None, X, ctx).to_numpy(), orc.agg_col(op, x)[1])
    t = rng.integers(0, 5, shape).astype(np.int64)  # many ties
    T = DenseMatrix.from_numpy(ctx, t)
    for op in (AggOpCode.IDXMIN, AggOpCode.IDXMAX):
        assert_exact(aggRow(op, None, T, ctx).to_numpy(), orc.agg_row(op, t)[1])
        assert_exact(aggCol(op, None, T, ctx).to_numpy(), orc.agg_col(op, t)[1])
    p = rng.integers(-2, 3, shape).astype(np.int64)
    assert aggAll(AggOpCode.PROD, DenseMatrix.from_numpy(ctx, p), ctx) == orc.agg_all(AggOpCode.PROD, p)[1]
    if shape[0] > 8 and shape[1] > 4:
        v, V = x[2:-3, 1:-2], X.slice(2, shape[0] - 3, 1, shape[1] - 2)
        vc = np.ascontiguousarray(v)
        assert aggAll(AggOpCode.SUM, V, ctx) == orc.agg_all(AggOpCode.SUM, vc)[1]
        assert_exact(aggRow(AggOpCode.MAX, None, V, ctx).to_numpy(), orc.agg_row(AggOpCode.MAX, vc)[1])
        assert_exact(aggCol(AggOpCode.MIN, None, V, ctx).to_numpy(), orc.agg_col(AggOpCode.MIN, vc)[1])


@pytest.mark.parametrize("shape", [(1000, 64), (129, 7), (3, 1000), (4096, 2)])
def test_si64_reorganisation(ctx, shape):
    rng = np.random.default_rng(shape[1])
    x = rng.integers(np.iinfo(np.int64).min, np.iinfo(np.int64).max, shape, dtype=np.int64)
    y = rng.integers(-99, 99, (shape[0], 5)).astype(np.int64)
    X, Y = DenseMatrix.from_numpy(ctx, x), DenseMatrix.from_numpy(ctx, y)
    assert_exact(transpose(None, X, ctx).to_numpy(), orc.transpose(x)[1])
    assert_exact(colBind(None, X, Y, ctx).to_numpy(), orc.col_bind(x, y)[1])
    sel = np.array([[shape[1] - 1], [0], [-1], [shape[1] // 2]], dtype=np.int64)
    assert_exact(extractCol(None, X, DenseMatrix.from_numpy(ctx, sel), ctx).to_numpy(), orc.extract_col(x, sel)[1])
    with pytest.raises(capi.DaphneHipOutOfRange):
        extractCol(None, X, DenseMatrix.from_numpy(ctx, np.array([[shape[1]]], dtype=np.int64)), ctx)
    assert_exact(fill(None, -(2 ** 62) - 3, 7, 9, ctx, dtype=np.int64).to_numpy(), orc.fill(-(2 ** 62) - 3, 7, 9, np.int64)[1])
    assert_exact(fill(None, 2 ** 63 + 5, 33, 2, ctx, dtype=np.uint64).to_numpy(), orc.fill(2 ** 63 + 5, 33, 2, np.uint64)[1])


def test_deferred_verdicts_report_the_first_failure_once(ctx):
    """With verdicts deferred, checked calls return at once (results of valid calls are unchanged) and the first
    failure in call order is raised when the block ends, with the status and text of the immediate form."""
    rng = np.random.default_rng(11)
    a, b = _ints(rng, (700, 4), np.int64), _ints(rng, (700, 4), np.int64)
    b[b == 0] = 3
    z = b.copy()
    z[250, 1] = 0
    A, B, Z = (DenseMatrix.from_numpy(ctx, m) for m in (a, b, z))
    sel_bad = DenseMatrix.from_numpy(ctx, np.array([[1], [17]], dtype=np.int64))
    sel_ok = DenseMatrix.from_numpy(ctx, np.array([[3], [-4]], dtype=np.int64))
    with ctx.deferred_checks():
        q = ewBinaryMat(BinaryOpCode.DIV, None, A, B, ctx)
        r = ewBinaryMat(BinaryOpCode.MOD, None, A, B, ctx)
        e = extractCol(None, A, sel_ok, ctx)
    assert_exact(q.to_numpy(), orc.ew_binary(BinaryOpCode.DIV, a, b)[1])
    assert_exact(r.to_numpy(), orc.ew_binary(BinaryOpCode.MOD, a, b)[1])
    assert_exact(e.to_numpy(), orc.extract_col(a, np.array([[3], [-4]], dtype=np.int64))[1])
    # a failure among valid calls: raised at the end of the block, by the call order's first failing call
    with pytest.raises(capi.DaphneHipOutOfRange, match=r"'17'.*\[0, 4\)"):
        with ctx.deferred_checks():
            ewBinaryMat(BinaryOpCode.DIV, None, A, B, ctx)
            extractCol(None, A, sel_bad, ctx)      # first
            ewBinaryMat(BinaryOpCode.MOD, None, A, Z, ctx)  # second: not the one reported
    ctx.check_deferred()  # nothing left pending
    with pytest.raises(capi.DaphneHipDomainError, match="remainder"):
        with ctx.deferred_checks():
            with ctx.deferred_checks():  # nests
                ewBinaryMat(BinaryOpCode.MOD, None, A, Z, ctx)
            # the inner block ending reports already: the outer one never gets here
    # an exception of the caller's own inside the block leaves the mode and drops what was pending
    with pytest.raises(KeyError):
        with ctx.deferred_checks():
            ewBinaryMat(BinaryOpCode.DIV, None, A, Z, ctx)
            raise KeyError("the caller's own")
    ctx.check_deferred()
    # immediate form as before
    with pytest.raises(capi.DaphneHipDomainError):
        ewBinaryMat(BinaryOpCode.DIV, None, A, Z, ctx)
    assert_exact(ewBinaryMat(BinaryOpCode.DIV, None, A, B, ctx).to_numpy(), orc.ew_binary(BinaryOpCode.DIV, a, b)[1])
