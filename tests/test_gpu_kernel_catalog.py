"""GPU: the generated kernel library called by catalog, the way a compiled DAPHNE program reaches a device kernel.

For every kernel of the device path at least one entry point is looked up in HIPcatalog.json by op mnemonic,
result and argument types and backend (the lookup of src/compiler/lowering/RewriteToCallKernelOpPass.cpp:403-415),
resolved in the library the record names, called with run-time objects, a dispatch id and the DaphneContext, and
compared with the CPU oracle. Inputs are host matrices: the kernels upload them on first use, results stay on the
device until they are read (the placement model of DenseMatrix.cpp:126-234).
"""
import ctypes as C

import numpy as np
import pytest

import oracle_binding as orc
from parity import assert_close, assert_exact

pytestmark = pytest.mark.gpu

CPP = {np.dtype(np.float32): "float", np.dtype(np.float64): "double", np.dtype(np.int64): "int64_t",
       np.dtype(np.uint64): "uint64_t", np.dtype(np.int32): "int32_t", np.dtype(np.uint32): "uint32_t"}
BIN = dict(ADD=0, SUB=1, MUL=2, DIV=3, POW=4, MOD=5, LOG=6, EQ=7, NEQ=8, LT=9, LE=10, GT=11, GE=12, MIN=13, MAX=14, AND=15, OR=16,
           BITWISE_AND=17)
UN = dict(MINUS=0, ABS=1, SIGN=2, SQRT=3, EXP=4, LN=5, SIN=6, COS=7, TAN=8, ASIN=9, ACOS=10, ATAN=11, SINH=12, COSH=13, TANH=14,
          FLOOR=15, CEIL=16, ROUND=17, ISNAN=18)
AGG = dict(SUM=0, PROD=1, MIN=2, MAX=3, IDXMIN=4, IDXMAX=5, MEAN=6, STDDEV=7, VAR=8)


def dm(dt):
    return f"DenseMatrix<{CPP[np.dtype(dt)]}>"


def word(op):  # ADD -> Add, BITWISE_AND -> Bitwise_and: how an op code enters a mnemonic
    return op[0] + op[1:].lower()


@pytest.fixture(scope="module")
def rt():
    from catalog_caller import Runtime

    r = Runtime()
    yield r
    r.close()


@pytest.fixture
def rng():
    return np.random.default_rng(7)


def by_catalog(rt, mnemonic, res, args, *values):
    rec = rt.find(mnemonic, res, args)
    return rt.call(rec["kernelFuncName"], *values)


FP = [np.float32, np.float64]


@pytest.mark.parametrize("dt", FP + [np.int64, np.uint32])
@pytest.mark.parametrize("op", ["ADD", "MUL", "DIV", "GE", "MAX"])
def test_ew_binary_mat(rt, rng, dt, op):
    a = rng.integers(1, 50, (37, 21)).astype(dt)
    b = rng.integers(1, 9, (37, 21)).astype(dt)
    A, B = rt.matrix(a), rt.matrix(b)
    res = by_catalog(rt, "ew" + word(op), [dm(dt)], [dm(dt), dm(dt)], A, B)
    assert res.where() == 2 and A.where() == 3  # result on the device only; the input now in both places
    exp = orc.ew_binary(BIN[op], a, b)[1]
    (assert_close if op == "DIV" and np.dtype(dt).kind == "f" else assert_exact)(res.to_numpy(), exp)
    for m in (A, B, res):
        m.destroy()


@pytest.mark.parametrize("dt", FP)
def test_ew_binary_broadcast_and_scalar(rt, rng, dt):
    a = rng.standard_normal((50, 33)).astype(dt)
    rv = rng.standard_normal((1, 33)).astype(dt)
    A, RV = rt.matrix(a), rt.matrix(rv)
    res = by_catalog(rt, "ewSub", [dm(dt)], [dm(dt), dm(dt)], A, RV)
    assert_exact(res.to_numpy(), orc.ew_binary(BIN["SUB"], a, rv)[1])
    sca = by_catalog(rt, "ewPow", [dm(dt)], [dm(dt), CPP[np.dtype(dt)]], A, 2.0)
    assert_close(sca.to_numpy(), orc.ew_binary_sca(BIN["POW"], a, 2.0)[1])
    for m in (A, RV, res, sca):
        m.destroy()


@pytest.mark.parametrize("dt", FP)
@pytest.mark.parametrize("op", ["EXP", "ABS", "FLOOR", "TANH", "ISNAN"])
def test_ew_unary_mat(rt, rng, dt, op):
    a = (rng.standard_normal((41, 19)) * 3).astype(dt)
    a[3, 4] = np.nan
    A = rt.matrix(a)
    res = by_catalog(rt, "ew" + word(op), [dm(dt)], [dm(dt)], A)
    exp = orc.ew_unary(UN[op], a)[1]
    (assert_close if op in ("EXP", "TANH") else assert_exact)(res.to_numpy(), exp)
    A.destroy(), res.destroy()


@pytest.mark.parametrize("dt", FP)
@pytest.mark.parametrize("op", ["SUM", "MIN", "MAX", "MEAN", "VAR", "STDDEV"])
def test_agg_all_row_col(rt, rng, dt, op):
    a = (rng.standard_normal((300, 17)) * 2 + 5).astype(dt)
    A = rt.matrix(a)
    vt = CPP[np.dtype(dt)]
    got = by_catalog(rt, word(op).lower() + "All", [vt], [dm(dt)], A)
    assert_close(np.asarray(got, dt), np.asarray(orc.agg_all(AGG[op], a)[1], dt))
    for dim, fn in (("Row", orc.agg_row), ("Col", orc.agg_col)):
        res = by_catalog(rt, word(op).lower() + dim, [dm(dt)], [dm(dt)], A)
        exp = fn(AGG[op], a)[1]
        (assert_exact if op in ("MIN", "MAX") else assert_close)(res.to_numpy(), exp)
        res.destroy()
    A.destroy()


@pytest.mark.parametrize("dt", FP + [np.int64])
@pytest.mark.parametrize("op", ["IDXMIN", "IDXMAX"])
def test_positions_of_extrema_are_size_t_matrices(rt, rng, dt, op):
    a = rng.integers(0, 6, (200, 13)).astype(dt)  # many ties: the first position wins
    A = rt.matrix(a)
    for dim, fn in (("Row", orc.agg_row), ("Col", orc.agg_col)):
        res = by_catalog(rt, op.lower() + dim, ["DenseMatrix<size_t>"], [dm(dt)], A)
        assert res.dtype == np.uint64
        assert_exact(res.to_numpy(), fn(AGG[op], a)[1])
        res.destroy()
    A.destroy()


def test_int64_aggregations(rt, rng):
    a = rng.integers(-1000, 1000, (123, 45)).astype(np.int64)
    A = rt.matrix(a)
    assert by_catalog(rt, "sumAll", ["int64_t"], [dm(np.int64)], A) == int(a.sum())
    res = by_catalog(rt, "maxCol", [dm(np.int64)], [dm(np.int64)], A)
    assert_exact(res.to_numpy(), a.max(axis=0, keepdims=True))
    A.destroy(), res.destroy()


@pytest.mark.parametrize("dt", FP)
def test_matmul_syrk_gemv_solve(rt, rng, dt):
    a = (rng.random((70, 40)) - 0.5).astype(dt)
    b = (rng.random((70, 30)) - 0.5).astype(dt)
    A, B = rt.matrix(a), rt.matrix(b)
    res = by_catalog(rt, "matMul", [dm(dt)], [dm(dt), dm(dt), "bool", "bool"], A, B, True, False)  # t(a) b
    assert res.shape == (40, 30)
    assert_close(res.to_numpy(), orc.matmul(a, b, True, False)[1], elementwise=False)
    s = by_catalog(rt, "syrk", [dm(dt)], [dm(dt), "bool"], A, True)
    assert_close(s.to_numpy(), orc.syrk(a, True)[1], elementwise=False)
    assert_exact(s.to_numpy(), s.to_numpy().T)
    v = (rng.random((70, 1)) - 0.5).astype(dt)
    V = rt.matrix(v)
    g = by_catalog(rt, "gemv", [dm(dt)], [dm(dt), dm(dt)], A, V)  # t(mat) vec
    assert_close(g.to_numpy(), orc.gemv(a, v)[1], elementwise=False)
    spd = (a.T @ a + 40 * np.eye(40)).astype(dt)
    rhs = rng.random((40, 1)).astype(dt)
    S, R = rt.matrix(spd), rt.matrix(rhs)
    x = by_catalog(rt, "solve", [dm(dt)], [dm(dt), dm(dt)], S, R)
    assert_close(x.to_numpy(), orc.solve(spd, rhs)[1], rtol=1e-3 if dt == np.float32 else 1e-9, elementwise=False)
    for m in (A, B, res, s, V, g, S, R, x):
        m.destroy()


@pytest.mark.parametrize("dt", FP)
def test_dnn_forward_kernels(rt, rng, dt):
    N, Cc, H, W, F, Hf, Wf = 5, 3, 12, 12, 4, 3, 3
    vt = CPP[np.dtype(dt)]
    x = rng.standard_normal((N, Cc * H * W)).astype(dt)
    w = rng.standard_normal((F, Cc * Hf * Wf)).astype(dt)
    bias = rng.standard_normal((F, 1)).astype(dt)
    X, Wm, Bm = rt.matrix(x), rt.matrix(w), rt.matrix(bias)
    geo = (N, Cc, H, W, Hf, Wf, 1, 1, 1, 1)
    conv, rh, rw = by_catalog(rt, "Convolution_Forward", [dm(dt), "size_t", "size_t"], [dm(dt)] * 3 + ["size_t"] * 10, X, Wm, Bm, *geo)
    st, exp, eh, ew = orc.conv2d(x, w, bias, *geo)
    assert (rh, rw) == (eh, ew)
    assert_close(conv.to_numpy(), exp, elementwise=False)
    relu = by_catalog(rt, "NN_Relu_Forward", [dm(dt)], [dm(dt)], conv)
    assert_exact(relu.to_numpy(), orc.relu(conv.to_numpy())[1])
    pgeo = (N, F, rh, rw, 2, 2, 2, 2, 0, 0)
    # the two size_t results of pooling are passed by value by the generated function (and so is the reference's)
    for mnem, fn in (("NN_Max_Forward", orc.maxpool), ("NN_Avg_Forward", orc.avgpool)):
        pool = by_catalog(rt, mnem, [dm(dt), "size_t", "size_t"], [dm(dt)] + ["size_t"] * 10, relu, *pgeo)
        exp = fn(relu.to_numpy(), *pgeo)[1]
        (assert_exact if mnem == "NN_Max_Forward" else assert_close)(pool.to_numpy(), exp)
        if mnem == "NN_Max_Forward":
            pooled = pool
        else:
            pool.destroy()
    feat = pooled.shape[1]
    wa = (rng.standard_normal((feat, 10)) * 0.1).astype(dt)
    ba = rng.standard_normal((1, 10)).astype(dt)
    WA, BA = rt.matrix(wa), rt.matrix(ba)
    aff = by_catalog(rt, "NN_Affine_Forward", [dm(dt)], [dm(dt)] * 3, pooled, WA, BA)
    assert_close(aff.to_numpy(), orc.matmul(pooled.to_numpy(), wa)[1] + ba, elementwise=False)
    sm = by_catalog(rt, "Softmax", [dm(dt)], [dm(dt)], aff)
    assert_close(sm.to_numpy(), orc.softmax(aff.to_numpy())[1])
    badd = by_catalog(rt, "BiasAdd", [dm(dt)], [dm(dt), dm(dt)], conv, Bm)
    assert_exact(badd.to_numpy(), orc.bias_add(conv.to_numpy(), bias)[1])
    gamma, beta, mean = (rng.standard_normal((F, 1)).astype(dt) for _ in range(3))
    var = (rng.random((F, 1)) + 0.5).astype(dt)
    G, Be, Me, Va = (rt.matrix(m) for m in (gamma, beta, mean, var))
    bn = by_catalog(rt, "BatchNormInferenceForward", [dm(dt)], [dm(dt)] * 5 + [vt], conv, G, Be, Me, Va, 1e-5)
    assert_close(bn.to_numpy(), orc.batchnorm(conv.to_numpy(), gamma, beta, mean, var, 1e-5)[1])
    for m in (X, Wm, Bm, conv, relu, pooled, WA, BA, aff, sm, badd, G, Be, Me, Va, bn):
        m.destroy()


@pytest.mark.parametrize("dt", FP)
def test_operator_chains_as_one_kernel(rt, rng, dt):
    """The kernels that stand for a chain of operators (kernels/HIP/FusedOperators.h), looked up like any other kernel,
    against the chain itself run through the catalog: conv -> relu -> max-pool, affine -> relu and the k-means
    assignment bit for bit; the normal equations and the k-means means within rounding (sums in another order)."""
    sz = "size_t"
    # conv2d -> relu -> max_pool2d (2 x 2 / 2), LeNet's second block at a small batch
    N, Cc, H, W, F, Hf, Wf = 6, 8, 14, 14, 16, 5, 5
    x = rng.standard_normal((N, Cc * H * W)).astype(dt)
    w = (rng.standard_normal((F, Cc * Hf * Wf)) * 0.1).astype(dt)
    bias = rng.standard_normal((F, 1)).astype(dt)
    X, Wm, Bm = rt.matrix(x), rt.matrix(w), rt.matrix(bias)
    geo = (N, Cc, H, W, Hf, Wf, 1, 1, 2, 2)
    conv, rh, rw = by_catalog(rt, "Convolution_Forward", [dm(dt), sz, sz], [dm(dt)] * 3 + [sz] * 10, X, Wm, Bm, *geo)
    relu = by_catalog(rt, "NN_Relu_Forward", [dm(dt)], [dm(dt)], conv)
    # (the pooling entry point takes its two extent results by value, as the reference's does: only the matrix comes back)
    pool = by_catalog(rt, "NN_Max_Forward", [dm(dt), sz, sz], [dm(dt)] + [sz] * 10, relu, N, F, rh, rw, 2, 2, 2, 2, 0, 0)
    ph, pw = rh // 2, rw // 2
    for epilogue, want, extents in ((3, pool, (ph, pw)), (1, relu, (rh, rw))):
        one, oh, ow = by_catalog(rt, "conv2DForwardFused", [dm(dt), sz, sz], [dm(dt)] * 3 + [sz] * 11, X, Wm, Bm, *geo, epilogue)
        assert (oh, ow) == extents
        assert_exact(one.to_numpy(), want.to_numpy())
        one.destroy()
    # affine -> relu
    feat = pool.shape[1]
    wa = (rng.standard_normal((feat, 24)) * 0.1).astype(dt)
    ba = rng.standard_normal((1, 24)).astype(dt)
    WA, BA = rt.matrix(wa), rt.matrix(ba)
    aff = by_catalog(rt, "NN_Affine_Forward", [dm(dt)], [dm(dt)] * 3, pool, WA, BA)
    arelu = by_catalog(rt, "NN_Relu_Forward", [dm(dt)], [dm(dt)], aff)
    one = by_catalog(rt, "affineForwardFused", [dm(dt)], [dm(dt)] * 3 + [sz], pool, WA, BA, 1)
    assert_exact(one.to_numpy(), arelu.to_numpy())
    for m in (X, Wm, Bm, conv, relu, pool, WA, BA, aff, arelu, one):
        m.destroy()

    # lmDS: A = syrk(X), b = t(X) @ y from one pass over X (100 columns: the symmetric streaming kernel)
    xs = rng.random((6000, 100)).astype(dt)
    ys = (xs @ rng.standard_normal((100, 1)) + 0.01 * rng.standard_normal((6000, 1))).astype(dt)
    XS, YS = rt.matrix(xs), rt.matrix(ys)
    a_seq = by_catalog(rt, "syrk", [dm(dt)], [dm(dt), "bool"], XS, True)
    b_seq = by_catalog(rt, "matMul", [dm(dt)], [dm(dt), dm(dt), "bool", "bool"], XS, YS, True, False)
    a_one, b_one = by_catalog(rt, "normalEquations", [dm(dt), dm(dt)], [dm(dt), dm(dt), CPP[np.dtype(dt)]], XS, YS, 0.0)
    assert a_one.shape == (100, 100) and b_one.shape == (100, 1)
    assert_close(a_one.to_numpy(), a_seq.to_numpy(), elementwise=False)
    assert_close(b_one.to_numpy(), b_seq.to_numpy(), elementwise=False)
    assert_close(a_one.to_numpy(), orc.syrk(xs, True)[1], elementwise=False)
    for m in (XS, YS, a_seq, b_seq, a_one, b_one):
        m.destroy()

    # k-means: idx = idxminRow(((X @ t(C)) * -2 + xx) + cc); enough rows for the streaming product, whose bits the
    # assignment kernel reproduces
    rows, cols, k = 70000, 64, 16
    centres = (rng.standard_normal((k, cols)) * 5).astype(dt)
    xk = (centres[rng.integers(0, k, rows)] + rng.standard_normal((rows, cols))).astype(dt)
    ck = xk[:: rows // k][:k].copy()
    XK, CK = rt.matrix(xk), rt.matrix(ck)
    sq = lambda M: by_catalog(rt, "ewMul", [dm(dt)], [dm(dt), dm(dt)], M, M)
    x2, c2 = sq(XK), sq(CK)
    xx = by_catalog(rt, "sumRow", [dm(dt)], [dm(dt)], x2)
    cc_col = by_catalog(rt, "sumRow", [dm(dt)], [dm(dt)], c2)
    cc = by_catalog(rt, "transpose", [dm(dt)], [dm(dt)], cc_col)
    prod = by_catalog(rt, "matMul", [dm(dt)], [dm(dt), dm(dt), "bool", "bool"], XK, CK, False, True)
    d1 = by_catalog(rt, "ewMul", [dm(dt)], [dm(dt), CPP[np.dtype(dt)]], prod, -2.0)
    d2 = by_catalog(rt, "ewAdd", [dm(dt)], [dm(dt), dm(dt)], d1, xx)
    d3 = by_catalog(rt, "ewAdd", [dm(dt)], [dm(dt), dm(dt)], d2, cc)
    idx_seq = by_catalog(rt, "idxminRow", ["DenseMatrix<size_t>"], [dm(dt)], d3)
    IDX = "DenseMatrix<size_t>"
    idx_one = by_catalog(rt, "kmeansAssign", [IDX], [dm(dt)] * 4, XK, CK, xx, cc)
    assert_exact(idx_one.to_numpy(), idx_seq.to_numpy())
    assert len(np.unique(idx_one.to_numpy())) == k
    cn, counts = by_catalog(rt, "kmeansUpdate", [dm(dt), dm(dt)], [dm(dt), IDX, sz], XK, idx_one, k)
    lab = idx_one.to_numpy()[:, 0]
    want_counts = np.bincount(lab, minlength=k).astype(dt)
    assert_exact(counts.to_numpy()[0], want_counts)
    want_means = np.stack([xk[lab == c].astype(np.float64).mean(axis=0) for c in range(k)]).astype(dt)
    assert_close(cn.to_numpy(), want_means, elementwise=False)
    idx_s, cn_s, counts_s = by_catalog(rt, "kmeansStep", [IDX, dm(dt), dm(dt)], [dm(dt)] * 4, XK, CK, xx, cc)
    assert_exact(idx_s.to_numpy(), idx_one.to_numpy())
    assert_exact(counts_s.to_numpy(), counts.to_numpy())
    assert_close(cn_s.to_numpy(), cn.to_numpy(), elementwise=False)
    for m in (XK, CK, x2, c2, xx, cc_col, cc, prod, d1, d2, d3, idx_seq, idx_one, cn, counts, idx_s, cn_s, counts_s):
        m.destroy()


@pytest.mark.parametrize("dt", FP + [np.int64])
def test_fill_colbind_extractcol_transpose(rt, rng, dt):
    vt = CPP[np.dtype(dt)]
    f = by_catalog(rt, "fill", [dm(dt)], [vt, "size_t", "size_t"], 7, 5, 9)
    assert_exact(f.to_numpy(), np.full((5, 9), 7, dt))
    a = rng.integers(-9, 9, (31, 6)).astype(dt)
    b = rng.integers(-9, 9, (31, 3)).astype(dt)
    A, B = rt.matrix(a), rt.matrix(b)
    cb = by_catalog(rt, "colBind", [dm(dt)], [dm(dt), dm(dt)], A, B)
    assert_exact(cb.to_numpy(), np.hstack([a, b]))
    sel = np.array([[5], [0], [0], [3]], np.int64)
    S = rt.matrix(sel)
    ec = by_catalog(rt, "extractCol", [dm(dt)], [dm(dt), dm(np.int64)], A, S)
    assert_exact(ec.to_numpy(), a[:, sel[:, 0]])
    tr = by_catalog(rt, "transpose", [dm(dt)], [dm(dt)], A)
    assert_exact(tr.to_numpy(), a.T)
    for m in (f, A, B, cb, S, ec, tr):
        m.destroy()


def test_transpose_of_positions(rt, rng):
    a = rng.integers(0, 2**40, (12, 5)).astype(np.uint64)
    A = rt.matrix(a)
    tr = by_catalog(rt, "transpose", ["DenseMatrix<size_t>"], ["DenseMatrix<size_t>"], A)
    assert_exact(tr.to_numpy(), a.T)
    A.destroy(), tr.destroy()


@pytest.mark.parametrize("dt", FP)
def test_training_kernels(rt, rng, dt):
    N, Cc, H, W = 4, 3, 8, 8
    x = rng.standard_normal((N, Cc * H * W)).astype(dt)
    pgeo = (N, Cc, H, W, 2, 2, 2, 2, 0, 0)
    dout = rng.standard_normal((N, Cc * 4 * 4)).astype(dt)
    X, D = rt.matrix(x), rt.matrix(dout)
    for mnem, fn in (("maxPoolBackward", orc.maxpool_backward), ("avgPoolBackward", orc.avgpool_backward)):
        res = by_catalog(rt, mnem, [dm(dt)], [dm(dt), dm(dt)] + ["size_t"] * 10, X, D, *pgeo)
        assert_close(res.to_numpy(), fn(x, dout, *pgeo)[1])
        res.destroy()
    F, Hf, Wf = 2, 3, 3
    w = rng.standard_normal((F, Cc * Hf * Wf)).astype(dt)
    dy = rng.standard_normal((N, F * H * W)).astype(dt)  # stride 1, pad 1
    Wm, DY = rt.matrix(w), rt.matrix(dy)
    # conv2DBackwardData(filter, output, strides, pads, N, C, H, W, F, C, Hf, Wf) -> data; `output` goes by reference and
    # therefore counts as a result in the catalog record, as in the reference
    dx = by_catalog(rt, "conv2DBackwardData", [dm(dt), dm(dt)], [dm(dt)] + ["size_t"] * 12, Wm, DY, 1, 1, 1, 1, N, Cc, H, W, F, Cc,
                    Hf, Wf)
    dx = dx[-1] if isinstance(dx, tuple) else dx
    assert_close(dx.to_numpy(), orc.conv2d_backward_data(w, dy, N, Cc, H, W, F, Hf, Wf, 1, 1, 1, 1)[1], elementwise=False)
    dw = by_catalog(rt, "conv2DBackwardFilter", [dm(dt)], [dm(dt), dm(dt)] + ["size_t"] * 12, X, DY, 1, 1, 1, 1, N, Cc, H, W, F, Cc,
                    Hf, Wf)
    assert_close(dw.to_numpy(), orc.conv2d_backward_filter(x, dy, N, Cc, H, W, F, Hf, Wf, 1, 1, 1, 1)[1], elementwise=False)
    for m in (X, D, Wm, DY, dx, dw):
        m.destroy()


def test_create_hip_context_entry_point(rt):
    h = rt.harness
    bare = h.th_ctx_create_bare()
    assert h.th_ctx_uses_hip(C.c_void_p(bare)) == 0
    fn = getattr(rt.libs[next(iter(rt.libs))], "HIP_createHIPContext")
    fn.argtypes, fn.restype = [C.c_int, C.c_void_p], None
    fn(-1, bare)  # -1: a call site that is not registered (ErrorHandler: UNREGISTERED)
    assert h.th_ctx_uses_hip(C.c_void_p(bare)) == 1
    h.th_ctx_destroy(C.c_void_p(bare))


def test_statistics_count_calls_by_dispatch_id(rt, rng):
    a = rng.standard_normal((8, 8)).astype(np.float32)
    A = rt.matrix(a)
    name = rt.find("ewAbs", [dm(np.float32)], [dm(np.float32)])["kernelFuncName"]
    kid = rt.register(name, "stats.daphne", 2, 5)
    rt.harness.th_set_statistics(rt.ctx, 1)
    for _ in range(3):
        rt.call(name, A, kid=kid).destroy()
    rt.harness.th_set_statistics(rt.ctx, 0)
    rt.call(name, A, kid=kid).destroy()
    assert rt.harness.th_kernel_calls(rt.ctx, kid) == 3
    A.destroy()


def test_device_memory_returns_when_matrices_go(rt, rng):
    before = rt.harness.th_device_allocations(rt.ctx)
    a = rng.standard_normal((64, 64)).astype(np.float64)
    A = rt.matrix(a)
    r = by_catalog(rt, "ewExp", [dm(np.float64)], [dm(np.float64)], A)
    assert rt.harness.th_device_allocations(rt.ctx) == before + 2
    A.destroy(), r.destroy()
    assert rt.harness.th_device_allocations(rt.ctx) == before


# ---------------------------------------------------------------------------------------------
# vectorized pipeline: one fused body over row shares, outputs combined on the device
# ---------------------------------------------------------------------------------------------
class Instr(C.Structure):
    _fields_ = [("kind", C.c_int32), ("op", C.c_int32), ("domain", C.c_int32), ("operand", C.c_int32), ("index", C.c_int32),
                ("swap", C.c_int32), ("scalar", C.c_double)]


EW_BINARY, EW_UNARY, ROW_AGG, STORE_TILE, STORE_ROW, STORE_ROW_IDX, REDUCE_ALL = range(7)
OPD_SCALAR, OPD_SELF, OPD_ROWVEC = 0, 1, 2
IN_PRIMARY, IN_MATRIX, IN_ROWVEC, IN_COLVEC = range(4)
OUT_TILE, OUT_ROW, OUT_ALL = range(3)
SPLIT_NONE, SPLIT_ROWS = 0, 1
COMB_ROWS, COMB_COLS, COMB_ADD, COMB_MIN, COMB_MAX = 1, 2, 3, 4, 5


def run_zscore_body(rt, X, MU, SD, thr, rows):
    """rowSums(((X - mu) / sd)^2) by ROWS and the count of rows above `thr` by ADD: the body of the z-score workload."""
    prog = (Instr * 7)(Instr(EW_BINARY, BIN["SUB"], 0, OPD_ROWVEC, 0, 0, 0.0), Instr(EW_BINARY, BIN["DIV"], 0, OPD_ROWVEC, 1, 0, 0.0),
                       Instr(EW_BINARY, BIN["MUL"], 0, OPD_SELF, 0, 0, 0.0), Instr(ROW_AGG, AGG["SUM"], 0, 0, 0, 0, 0.0),
                       Instr(STORE_ROW, 0, 1, 0, 0, 0, 0.0), Instr(EW_BINARY, BIN["GT"], 1, OPD_SCALAR, 0, 0, float(thr)),
                       Instr(REDUCE_ALL, AGG["SUM"], 1, 0, 0, 0, 0.0))
    ins = (C.c_void_p * 3)(X.h, MU.h, SD.h)
    outs = (C.c_void_p * 2)()
    st = rt.harness.th_run_fused_pipeline_f32(
        rt.ctx, prog, 7, ins, (C.c_int * 3)(IN_PRIMARY, IN_ROWVEC, IN_ROWVEC), (C.c_int * 3)(0, 0, 1),
        (C.c_int64 * 3)(SPLIT_ROWS, SPLIT_NONE, SPLIT_NONE), 3, outs, (C.c_int * 2)(OUT_ROW, OUT_ALL), (C.c_int * 2)(0, 0),
        (C.c_int64 * 2)(rows, 1), (C.c_int64 * 2)(1, 1), (C.c_int64 * 2)(COMB_ROWS, COMB_ADD), 2)
    assert st == 0, rt.harness.th_last_error().decode()
    from catalog_caller import Matrix

    return Matrix(rt, outs[0], np.float32), Matrix(rt, outs[1], np.float32)


@pytest.mark.parametrize("shares,batch", [(1, 0), (2, 0), (7, 0), (3, 1000), (1, 4096)])
def test_pipeline_in_row_shares_vs_oracle_engine(rt, shares, batch):
    rows, cols, thr = 20011, 64, 64.0
    x = (np.random.default_rng(3).standard_normal((rows, cols)) * 2 + 5).astype(np.float32)
    st, mu_e, sd_e, r_e, s_e, _ = orc.zscore_pipeline(x, threads=3, thr=thr)
    assert st == 0
    X = rt.matrix(x)
    f32 = dm(np.float32)
    MU = by_catalog(rt, "meanCol", [f32], [f32], X)
    VAR = by_catalog(rt, "varCol", [f32], [f32], X)
    SD = by_catalog(rt, "ewSqrt", [f32], [f32], VAR)
    assert_close(MU.to_numpy(), mu_e)
    assert_close(SD.to_numpy(), sd_e)
    rt.harness.th_set_vect(rt.ctx, shares, batch)
    try:
        R, S = run_zscore_body(rt, X, MU, SD, thr, rows)
    finally:
        rt.harness.th_set_vect(rt.ctx, 1, 0)
    assert R.where() == 2 and S.where() == 2
    r = R.to_numpy()
    assert_close(r, r_e)
    if shares == 1 and batch == 0:
        test_pipeline_in_row_shares_vs_oracle_engine.whole = r.copy()
    else:  # ROWS: every row is computed by the same instructions wherever the share boundaries are
        assert_exact(r, test_pipeline_in_row_shares_vs_oracle_engine.whole)
    ambiguous = int((np.abs(r_e - thr) <= thr * 1e-4).sum())
    assert abs(float(S.to_numpy()[0, 0]) - float(s_e)) <= ambiguous
    assert float(S.to_numpy()[0, 0]) == float((r > thr).sum())  # ADD over the shares of this run's own rows: exact
    for m in (X, MU, VAR, SD, R, S):
        m.destroy()
