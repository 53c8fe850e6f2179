"""GPU parity: the fused vectorized pipeline against (a) the same operators run one by one through
the stand-alone device kernels and (b) the CPU oracle's restatement of the reference's engine."""
import numpy as np
import pytest

import oracle_binding as orc
from parity import assert_close, assert_exact, variance_floor

pytestmark = pytest.mark.gpu

from daphne_amd import capi
from daphne_amd.kernels import (AggOpCode, BinaryOpCode, DenseMatrix, UnaryOpCode, aggAll, aggCol, aggRow, ewBinaryMat,
                                ewBinaryObjSca, ewUnaryMat)
from daphne_amd.pipeline import ROWREG, SELF, VectorizedPipeline

DTYPES = [np.float32, np.float64]


@pytest.fixture(autouse=True, params=[1, 0], ids=["specialised", "interpreted"])
def pipeline_mode(request, ctx):
    """Every test of this module runs twice on the shared context: with bodies specialised at run time and with the
    generic kernel interpreting them. A test that ran a body must have run it the way the context was told to."""
    mode = request.param
    ctx.set_pipeline_mode(mode)
    yield mode
    ctx.set_pipeline_mode(-1)


def assert_ran_as(mode):
    assert capi.lib().dh_vectorized_pipeline_last_mode() == mode


def zscore_device(ctx, X, thr=64.0):
    """Config-2 style pipeline on the device: two column statistics + one fused kernel."""
    mu = aggCol(AggOpCode.MEAN, None, X, ctx)
    sd = ewUnaryMat(UnaryOpCode.SQRT, None, aggCol(AggOpCode.VAR, None, X, ctx), ctx)
    p = VectorizedPipeline(ctx, X)
    p.ewBinary(BinaryOpCode.SUB, mu).ewBinary(BinaryOpCode.DIV, sd).ewBinary(BinaryOpCode.MUL, SELF)
    p.rowAgg(AggOpCode.SUM)
    r = p.storeRow()
    p.ewBinary(BinaryOpCode.GT, thr)
    s = p.reduceAll(AggOpCode.SUM)
    p.run()
    return mu, sd, r, s


@pytest.mark.parametrize("rows,cols", [(1000, 64), (50001, 64), (777, 16), (513, 40), (300, 7), (64, 256), (5, 1000)])
def test_zscore_pipeline_vs_oracle_engine(ctx, pipeline_mode, rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = (rng.standard_normal((rows, cols)) * 2 + 5).astype(np.float32)
    thr = float(cols)
    st, mu_e, sd_e, r_e, s_e, _ = orc.zscore_pipeline(x, threads=3, thr=thr)
    mu, sd, r, s = zscore_device(ctx, DenseMatrix.from_numpy(ctx, x), thr)
    assert_ran_as(pipeline_mode)
    assert_close(mu.to_numpy(), mu_e)
    assert_close(sd.to_numpy(), sd_e)
    assert_close(r.to_numpy(), r_e)
    # the count may differ only by rows whose r is within tolerance of the threshold
    amb = int((np.abs(r_e - thr) <= 1e-4 * thr).sum())
    assert abs(float(s.to_numpy()[0, 0]) - float(s_e)) <= amb


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,cols", [(1000, 64), (333, 16), (129, 36), (70, 5), (40, 512), (9, 130)])
def test_pipeline_equals_op_by_op(ctx, dt, rows, cols):
    """Same body, fused vs one kernel per operator (how the reference's device worker runs it)."""
    rng = np.random.default_rng(rows * 3 + cols)
    x = (rng.standard_normal((rows, cols)) + 3).astype(dt)
    y = rng.standard_normal((rows, cols)).astype(dt)
    rv = (rng.random((1, cols)) + 0.5).astype(dt)
    cv = (rng.random((rows, 1)) + 0.5).astype(dt)
    X, Y, RV, CV = (DenseMatrix.from_numpy(ctx, a) for a in (x, y, rv, cv))
    # fused
    p = VectorizedPipeline(ctx, X)
    p.ewBinary(BinaryOpCode.ADD, Y).ewBinary(BinaryOpCode.MUL, RV).ewBinary(BinaryOpCode.DIV, CV)
    p.ewBinary(BinaryOpCode.SUB, 0.25).ewUnary(UnaryOpCode.ABS).ewBinary(BinaryOpCode.SUB, 1.0, swap=True)
    tile = p.storeTile()
    p.rowAgg(AggOpCode.MAX)
    rmax = p.storeRow()
    p.toTile().ewBinary(BinaryOpCode.SUB, ROWREG).ewUnary(UnaryOpCode.EXP)
    p.rowAgg(AggOpCode.SUM)
    rsum = p.storeRow()
    tot = p.reduceAll(AggOpCode.SUM)
    p.toTile().ewBinary(BinaryOpCode.DIV, ROWREG)
    soft = p.storeTile()
    p.run()
    # one by one
    t = ewBinaryMat(BinaryOpCode.ADD, None, X, Y, ctx)
    t = ewBinaryMat(BinaryOpCode.MUL, None, t, RV, ctx)
    t = ewBinaryMat(BinaryOpCode.DIV, None, t, CV, ctx)
    t = ewBinaryObjSca(BinaryOpCode.SUB, None, t, 0.25, ctx)
    t = ewUnaryMat(UnaryOpCode.ABS, None, t, ctx)
    t = ewBinaryObjSca(BinaryOpCode.MUL, None, ewBinaryObjSca(BinaryOpCode.SUB, None, t, 1.0, ctx), -1.0, ctx)
    assert_exact(tile.to_numpy(), t.to_numpy())
    m = aggRow(AggOpCode.MAX, None, t, ctx)
    assert_exact(rmax.to_numpy(), m.to_numpy())
    e = ewUnaryMat(UnaryOpCode.EXP, None, ewBinaryMat(BinaryOpCode.SUB, None, t, m, ctx), ctx)
    ssum = aggRow(AggOpCode.SUM, None, e, ctx)
    assert_close(rsum.to_numpy(), ssum.to_numpy())
    assert_close(tot.to_numpy(), np.array([[aggAll(AggOpCode.SUM, ssum, ctx)]], dt), rtol=1e-5 if dt == np.float32 else 1e-12)
    assert_close(soft.to_numpy(), ewBinaryMat(BinaryOpCode.DIV, None, e, ssum, ctx).to_numpy())


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op", [AggOpCode.SUM, AggOpCode.PROD, AggOpCode.MIN, AggOpCode.MAX, AggOpCode.MEAN,
                                AggOpCode.STDDEV, AggOpCode.VAR, AggOpCode.IDXMIN, AggOpCode.IDXMAX])
@pytest.mark.parametrize("rows,cols", [(2000, 16), (50, 64), (33, 24), (7, 300)])
def test_pipeline_row_aggs_vs_oracle(ctx, dt, op, rows, cols):
    rng = np.random.default_rng(rows + cols + int(op))
    if op in (AggOpCode.IDXMIN, AggOpCode.IDXMAX):
        x = rng.integers(0, 5, (rows, cols)).astype(dt)
        x[0, :] = np.nan
        x[1, 0] = np.nan
        x[2, 1:] = np.nan
        x[3, :] = np.inf
    elif op == AggOpCode.PROD:
        x = (1 + 0.01 * rng.standard_normal((rows, cols))).astype(dt)
    else:
        x = (rng.standard_normal((rows, cols)) * 2 + 5).astype(dt)
        if op in (AggOpCode.MIN, AggOpCode.MAX):
            x[1, 0] = np.nan
            x[2, 3] = np.nan
    p = VectorizedPipeline(ctx, DenseMatrix.from_numpy(ctx, x))
    p.rowAgg(op)
    is_idx = op in (AggOpCode.IDXMIN, AggOpCode.IDXMAX)
    out = p.storeRow(as_index=is_idx)
    p.run()
    st, exp = orc.agg_row(op, x)
    if is_idx or op in (AggOpCode.MIN, AggOpCode.MAX):
        assert_exact(out.to_numpy(), exp)
    else:
        atol = variance_floor(x, op == AggOpCode.STDDEV) if op in (AggOpCode.VAR, AggOpCode.STDDEV) else 0.0
        assert_close(out.to_numpy(), exp, atol=atol)


@pytest.mark.parametrize("dt", DTYPES)
def test_pipeline_kmeans_distance_idxmin(ctx, dt):
    """D = xx - 2*XC + cc ; idx = idxminRow(D) as one fused body (k-means assignment step)."""
    rng = np.random.default_rng(8)
    rows, k = 5000, 16
    xc = rng.standard_normal((rows, k)).astype(dt)
    xx = (rng.random((rows, 1)) * 3).astype(dt)
    cc = (rng.random((1, k)) * 3).astype(dt)
    p = VectorizedPipeline(ctx, DenseMatrix.from_numpy(ctx, xc))
    p.ewBinary(BinaryOpCode.MUL, -2.0).ewBinary(BinaryOpCode.ADD, DenseMatrix.from_numpy(ctx, xx))
    p.ewBinary(BinaryOpCode.ADD, DenseMatrix.from_numpy(ctx, cc))
    p.rowAgg(AggOpCode.IDXMIN)
    idx = p.storeRow(as_index=True)
    p.run()
    d = orc.ew_binary(0, orc.ew_binary(0, orc.ew_binary_sca(2, xc, -2.0)[1], xx)[1], cc)[1]
    assert_exact(idx.to_numpy(), orc.agg_row(AggOpCode.IDXMIN, d)[1])


@pytest.mark.parametrize("dt", DTYPES)
def test_pipeline_reduce_min_max_and_views(ctx, dt):
    rng = np.random.default_rng(9)
    big = rng.standard_normal((400, 96)).astype(dt)
    B = DenseMatrix.from_numpy(ctx, big)
    v, V = big[10:390, 8:72], B.slice(10, 390, 8, 72)
    p = VectorizedPipeline(ctx, V)
    p.ewBinary(BinaryOpCode.MUL, 2.0)
    mn = p.reduceAll(AggOpCode.MIN)
    mx = p.reduceAll(AggOpCode.MAX)
    p.run()
    assert_exact(mn.to_numpy(), np.array([[v.min() * 2]], dt))
    assert_exact(mx.to_numpy(), np.array([[v.max() * 2]], dt))


def test_pipeline_errors(ctx):
    x = DenseMatrix.from_numpy(ctx, np.ones((10, 8), np.float32))
    p = VectorizedPipeline(ctx, x)
    p.ewBinary(999, 1.0)
    with pytest.raises(capi.DaphneHipError, match="unknown BinaryOpCode"):
        p.run()
    p = VectorizedPipeline(ctx, DenseMatrix.from_numpy(ctx, -np.ones((10, 8), np.float32)))
    p.ewUnary(UnaryOpCode.SQRT)
    p.storeTile()
    with pytest.raises(capi.DaphneHipDomainError):
        p.run()
    wide = DenseMatrix.from_numpy(ctx, np.ones((2, 5000), np.float32))
    p = VectorizedPipeline(ctx, wide)
    p.ewUnary(UnaryOpCode.ABS)
    p.storeTile()
    with pytest.raises(capi.DaphneHipError, match="do not fit the register tile"):
        p.run()
    with pytest.raises(capi.DaphneHipError, match="row/column vector"):
        VectorizedPipeline(ctx, x).ewBinary(BinaryOpCode.ADD, DenseMatrix.from_numpy(ctx, np.ones((3, 3), np.float32)))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,cols", [(4096, 64), (1000, 16), (257, 40), (33, 7), (100, 512)])
def test_pipeline_division_by_row_vector_is_ieee_division(ctx, pipeline_mode, dt, rows, cols):
    """t / rowvec inside a specialised body takes a short division sequence when every operand is well inside the
    exponent range and the general one otherwise; either way the quotient is the correctly rounded one, bit for bit
    (numpy divides in IEEE arithmetic, as the reference's CPU and CUDA kernels do)."""
    rng = np.random.default_rng(rows + cols)
    # (a) everything in the comfortable range, spread over many binades
    x = (rng.standard_normal((rows, cols)) * np.exp2(rng.integers(-30, 30, (rows, cols)))).astype(dt)
    x[x == 0] = 1
    d = ((rng.random((1, cols)) + 0.5) * np.exp2(rng.integers(-30, 30, (1, cols))) * rng.choice([-1, 1], (1, cols))).astype(dt)
    # (b) the same with rows that leave the range: zeros of both signs, infinities, NaN, subnormals, huge and tiny values
    x2 = x.copy()
    fi = np.finfo(dt)
    specials = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, fi.tiny / 8, -fi.tiny / 4, fi.max, -fi.max / 3, fi.tiny,
                         fi.eps, 1 / fi.eps], dtype=dt)
    idx = rng.integers(0, rows * cols, 200)
    x2.reshape(-1)[idx] = specials[rng.integers(0, specials.size, idx.size)]
    # (c) a divisor outside the range
    d2 = d.copy()
    d2[0, 0] = fi.tiny / 2
    d2[0, cols // 2] = fi.max / 2
    for xa, da in ((x, d), (x2, d), (x, d2), (x2, d2)):
        X, D = DenseMatrix.from_numpy(ctx, xa), DenseMatrix.from_numpy(ctx, da)
        p = VectorizedPipeline(ctx, X)
        p.ewBinary(BinaryOpCode.DIV, D)
        out = p.storeTile()
        p.run()
        assert_ran_as(pipeline_mode)
        with np.errstate(all="ignore"):
            want = xa / da
        got = out.to_numpy()
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan)
        assert np.array_equal(got[~nan].view(np.uint32 if dt == np.float32 else np.uint64),
                              want[~nan].view(np.uint32 if dt == np.float32 else np.uint64))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,cols", [(3000, 64), (257, 40), (33, 7)])
def test_interpreted_body_equals_specialised_body(ctx, dt, rows, cols):
    """The generic kernel and the run-time specialised one instantiate the same body: same results, bit for bit."""
    rng = np.random.default_rng(rows + cols)
    x = (rng.standard_normal((rows, cols)) * 2 + 5).astype(dt)
    rv = (rng.random((1, cols)) + 0.5).astype(dt)
    X, RV = DenseMatrix.from_numpy(ctx, x), DenseMatrix.from_numpy(ctx, rv)
    outs = {}
    for mode in (1, 0):
        ctx.set_pipeline_mode(mode)
        p = VectorizedPipeline(ctx, X)
        p.ewBinary(BinaryOpCode.SUB, 5.0).ewBinary(BinaryOpCode.DIV, RV).ewBinary(BinaryOpCode.MUL, SELF)
        tile = p.storeTile()
        p.rowAgg(AggOpCode.SUM)
        r = p.storeRow()
        p.ewBinary(BinaryOpCode.GT, float(cols))
        s = p.reduceAll(AggOpCode.SUM)
        p.run()
        assert_ran_as(mode)
        outs[mode] = (tile.to_numpy(), r.to_numpy(), s.to_numpy())
    for a, b in zip(outs[1], outs[0]):
        assert_exact(a, b)


def test_changing_immediates_reuse_the_compiled_body(ctx, pipeline_mode):
    """A body is compiled per structure, not per value of its scalars: thresholds that change from call to call (and
    NaN / infinite ones, which have no literal form) run the same kernel."""
    if pipeline_mode != 1:
        pytest.skip("only the specialised path compiles anything")
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2000, 24)).astype(np.float32)
    X = DenseMatrix.from_numpy(ctx, x)
    sizes = []
    for k, thr in enumerate([0.5, -0.25, 3.0, float("inf"), float("nan"), 1e-30, 7.75]):
        p = VectorizedPipeline(ctx, X)
        p.ewBinary(BinaryOpCode.MUL, 1.0 + k).ewBinary(BinaryOpCode.GT, thr)
        out = p.storeTile()
        p.run()
        assert_ran_as(1)
        sizes.append(capi.lib().dh_vectorized_pipeline_cache_size())
        with np.errstate(invalid="ignore"):
            want = ((x * np.float32(1.0 + k)) > np.float32(thr)).astype(np.float32)
        assert_exact(out.to_numpy(), want)
    assert len(set(sizes)) == 1, sizes


def test_an_evicted_body_is_compiled_again_and_runs(ctx, pipeline_mode):
    """More distinct bodies than the cache may hold: the least recently used one leaves (and is unloaded once nobody
    is about to launch it); using it again compiles it again, with the same results."""
    if pipeline_mode != 1:
        pytest.skip("only the specialised path compiles anything")
    rng = np.random.default_rng(11)
    x = rng.standard_normal((1500, 32)).astype(np.float32)
    X = DenseMatrix.from_numpy(ctx, x)
    ops = [BinaryOpCode.ADD, BinaryOpCode.SUB, BinaryOpCode.MUL, BinaryOpCode.MAX]
    fns = {BinaryOpCode.ADD: np.add, BinaryOpCode.SUB: np.subtract, BinaryOpCode.MUL: np.multiply, BinaryOpCode.MAX: np.maximum}
    lib = capi.lib()
    before = lib.dh_vectorized_pipeline_set_cache_limit(2)
    try:
        for op in ops + ops[:2]:  # the first two bodies have left the cache by the time they come round again
            p = VectorizedPipeline(ctx, X)
            p.ewBinary(op, 0.75).ewUnary(UnaryOpCode.ABS)
            out = p.storeTile()
            p.run()
            assert_ran_as(1)
            assert lib.dh_vectorized_pipeline_cache_size() <= 2
            assert_exact(out.to_numpy(), np.abs(fns[op](x, np.float32(0.75))))
    finally:
        lib.dh_vectorized_pipeline_set_cache_limit(before)


def test_kernel_stopwatch_times_the_body_kernel_alone(ctx):
    """dh_kernel_timing: a pair of events around the fused pipeline's body kernel per run; the reading sums them, counts
    them and starts again; nothing is recorded while the stopwatch is off."""
    from daphne_amd.kernels import AggOpCode, BinaryOpCode, DenseMatrix, aggCol
    from daphne_amd.pipeline import SELF, VectorizedPipeline

    x = (np.random.default_rng(3).standard_normal((200_000, 32)) + 2).astype(np.float32)
    X = DenseMatrix.from_numpy(ctx, x)
    mu = aggCol(AggOpCode.MEAN, None, X, ctx)
    p = VectorizedPipeline(ctx, X)
    p.ewBinary(BinaryOpCode.SUB, mu).ewBinary(BinaryOpCode.MUL, SELF)
    p.rowAgg(AggOpCode.SUM)
    r = p.storeRow()
    s = p.reduceAll(AggOpCode.SUM)
    p.run()
    assert ctx.kernel_timing_read() == (0.0, 0)
    ctx.kernel_timing(True)
    for _ in range(5):
        p.run()
    total, n = ctx.kernel_timing_read()
    assert n == 5 and 0.0 < total < 50.0
    assert ctx.kernel_timing_read() == (0.0, 0)  # read and reset
    p.run()
    total1, n1 = ctx.kernel_timing_read()
    assert n1 == 1 and 0.0 < total1 < 10.0
    ctx.kernel_timing(False)
    p.run()
    assert ctx.kernel_timing_read() == (0.0, 0)
    want = ((x - x.mean(0, dtype=np.float64).astype(np.float32)) ** 2).sum(1)
    np.testing.assert_allclose(r.to_numpy()[:, 0], want, rtol=1e-4)
    assert abs(float(s.to_numpy()[0, 0]) - float(want.astype(np.float64).sum())) <= 1e-3 * float(want.sum())


def test_a_body_compiled_by_one_process_runs_from_disk_in_the_next(tmp_path):
    """The on-disk cache of compiled bodies: the second process loads the first one's code object and gets its bits."""
    import os
    import subprocess
    import sys
    from pathlib import Path

    ROOT = Path(__file__).resolve().parent.parent
    script = r"""
import sys
import numpy as np
sys.path.insert(0, %r)
from daphne_amd import capi
from daphne_amd.kernels import AggOpCode, BinaryOpCode, DenseMatrix, HIPContext, aggCol
from daphne_amd.pipeline import SELF, VectorizedPipeline
ctx = HIPContext(0)
ctx.set_pipeline_mode(1)
x = (np.random.default_rng(11).standard_normal((50_000, 24)) * 3 + 1).astype(np.float32)
X = DenseMatrix.from_numpy(ctx, x)
mu = aggCol(AggOpCode.MEAN, None, X, ctx)
p = VectorizedPipeline(ctx, X)
p.ewBinary(BinaryOpCode.SUB, mu).ewBinary(BinaryOpCode.MUL, SELF)
p.rowAgg(AggOpCode.SUM)
r = p.storeRow()
p.run()
assert capi.lib().dh_vectorized_pipeline_last_mode() == 1
np.save(sys.argv[1], r.to_numpy())
""" % str(ROOT)
    env = dict(os.environ, DH_PIPELINE_JIT_CACHE=str(tmp_path / "bodies"))
    for name in ("a.npy", "b.npy"):
        done = subprocess.run([sys.executable, "-c", script, str(tmp_path / name)], env=env, capture_output=True, text=True, timeout=300)
        assert done.returncode == 0, done.stdout[-2000:] + done.stderr[-2000:]
        files = sorted((tmp_path / "bodies").glob("*.bin"))
        assert len(files) == 1
        if name == "a.npy":
            stamp = files[0].stat().st_mtime_ns
    assert files[0].stat().st_mtime_ns == stamp  # the second process read it and wrote nothing
    assert_exact(np.load(tmp_path / "a.npy"), np.load(tmp_path / "b.npy"))
