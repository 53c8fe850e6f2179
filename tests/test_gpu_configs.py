"""GPU: the five benchmark configurations end to end through the device kernels.

Where the CPU oracle finishes in seconds the whole result is compared against it (same seeded inputs);
at the full sizes only size-independent properties are checked (independent float64 statistics on the
device, batch independence, symmetry, sampled entries in extended precision)."""
import numpy as np
import pytest
import torch

import oracle_binding as orc
from parity import assert_close, assert_exact

pytestmark = pytest.mark.gpu

from daphne_amd.kernels import AggOpCode, BinaryOpCode, DenseMatrix, matMul, syrk
from daphne_amd.workloads import KMeans, lenet_forward, lmds, zscore_count


def _orc_lmds(X, y, reg):
    A = orc.syrk(X, True)[1] + (np.eye(X.shape[1]) * reg)
    b = orc.matmul(X, y, True, False)[1]
    return A, b, orc.solve(A, b)[1]


def test_config1_lmds_normal_equations(ctx):
    """X 100000 x 100 f64 U[0,1), w ~ N(0,1), y = X w + N(0, 0.01); A, b, w_hat vs the oracle (<= 1e-10)."""
    rng = np.random.default_rng(42)
    n, m = 100_000, 100
    X = rng.random((n, m))
    w = rng.standard_normal((m, 1))
    y = X @ w + 0.1 * rng.standard_normal((n, 1))
    A_e, b_e, w_e = _orc_lmds(X, y, 1e-3)
    eye = DenseMatrix.from_numpy(ctx, np.eye(m))
    dX, dy = DenseMatrix.from_numpy(ctx, X), DenseMatrix.from_numpy(ctx, y)
    # the normal equations from one pass over X, and operator by operator as the script writes them
    for fused in (True, False):
        A, b, w_hat = lmds(ctx, dX, dy, 1e-3, eye, fused=fused)
        assert_close(A.to_numpy(), A_e, elementwise=False)
        assert_close(b.to_numpy(), b_e, elementwise=False)
        assert_close(w_hat.to_numpy(), w_e, rtol=1e-9, elementwise=False)  # cond(A) ~ 3e2 amplifies the 1e-13 of A, b
        assert np.abs(w_hat.to_numpy() - w).max() < 0.05  # and it recovers the generating weights
        assert_exact(A.to_numpy(), A.to_numpy().T)


def test_config2_full_size_properties(ctx):
    """20M x 64 f32: column statistics against float64 statistics computed independently on the device,
    r against a float64 evaluation of sampled rows, s against the count of r > 64."""
    R, C = 20_000_000, 64
    g = torch.Generator(device="cuda").manual_seed(7)
    Xt = torch.empty(R, C, device="cuda", dtype=torch.float32).normal_(5.0, 2.0, generator=g)
    mu, sd, r, s = zscore_count(ctx, DenseMatrix.from_torch(ctx, Xt), 64.0)
    mu64 = torch.zeros(C, device="cuda", dtype=torch.float64)
    m2 = torch.zeros(C, device="cuda", dtype=torch.float64)
    for lo in range(0, R, 2_000_000):
        mu64 += Xt[lo:lo + 2_000_000].to(torch.float64).sum(0)
    mu64 /= R
    for lo in range(0, R, 2_000_000):
        m2 += ((Xt[lo:lo + 2_000_000].to(torch.float64) - mu64) ** 2).sum(0)
    sd64 = torch.sqrt(m2 / R)
    assert_close(mu.to_numpy()[0], mu64.cpu().numpy().astype(np.float32), rtol=1e-5)
    assert_close(sd.to_numpy()[0], sd64.cpu().numpy().astype(np.float32), rtol=1e-5)
    rows = torch.randint(0, R, (4096,), device="cuda")
    z = (Xt[rows].to(torch.float64) - mu64) / sd64
    r_h = r.to_numpy()[:, 0]
    assert_close(r_h[rows.cpu().numpy()], (z * z).sum(1).cpu().numpy().astype(np.float32), rtol=1e-4)
    assert float(s.to_numpy()[0, 0]) == float((r_h > 64.0).sum())
    del Xt
    torch.cuda.empty_cache()


def _orc_kmeans_iter(X, C, xx):
    XC = orc.matmul(X, C, False, True)[1]
    cc = orc.agg_row(AggOpCode.SUM, orc.ew_binary(BinaryOpCode.MUL, C, C)[1])[1]
    D = orc.ew_binary(0, orc.ew_binary(0, orc.ew_binary_sca(2, XC, -2.0)[1], xx)[1], np.ascontiguousarray(cc.T))[1]
    idx = orc.agg_row(AggOpCode.IDXMIN, D)[1]
    P = (idx == np.arange(C.shape[0], dtype=np.uint64)[None, :]).astype(X.dtype)
    PtX = orc.matmul(P, X, True, False)[1]
    cnt = orc.agg_col(AggOpCode.SUM, P)[1]
    return orc.ew_binary(BinaryOpCode.DIV, PtX, np.ascontiguousarray(cnt.T))[1], idx, D


@pytest.mark.parametrize("fused", [True, "two_passes", False], ids=["one_pass", "two_passes", "operator_sequence"])
def test_config3_kmeans_against_oracle(ctx, fused):
    """Mixture of 16 Gaussians, 10 Lloyd iterations at an oracle-feasible size; indices bit-exact on rows
    whose two smallest distances are not a near-tie (the GEMMs sum in different orders), centroids 1e-4."""
    rng = np.random.default_rng(3)
    k, f, n = 16, 64, 32_000
    centres = rng.standard_normal((k, f)) * 5
    X = (centres[np.arange(n) % k] + rng.standard_normal((n, f))).astype(np.float32)
    C0 = np.ascontiguousarray(X[np.arange(k) * (n // k) + np.arange(k)])  # one seed row per generating cluster
    xx = orc.agg_row(AggOpCode.SUM, orc.ew_binary(BinaryOpCode.MUL, X, X)[1])[1]
    km = KMeans(ctx, DenseMatrix.from_numpy(ctx, X), k)
    assert_close(km.xx.to_numpy(), xx)
    Cd, Ce = DenseMatrix.from_numpy(ctx, C0), C0
    ties_total = 0
    for it in range(10):
        Cd = km.iterate(Cd, fused=fused)
        Ce, idx_e, D = _orc_kmeans_iter(X, Ce, xx)
        part = np.partition(D, 1, axis=1)
        near_tie = (part[:, 1] - part[:, 0]) <= 1e-3 * np.abs(part[:, 0])
        ties_total += int(near_tie.sum())
        idx_d = km.idx.to_numpy()
        assert_exact(idx_d[~near_tie], idx_e[~near_tie])
        assert_close(Cd.to_numpy(), Ce, rtol=1e-4, elementwise=False)
    assert ties_total < n // 100
    # the assignment recovers the generating mixture
    assert len(np.unique(km.idx.to_numpy())) == k


@pytest.mark.parametrize("fused", [True, "two_passes", False], ids=["one_pass", "two_passes", "operator_sequence"])
def test_config3_seeded_like_the_bench_against_oracle(ctx, fused):
    """The configuration seeds its centroids from rows i * (n / k); with n / k = 8 mod 16 those 16 rows come from only two
    of the 16 Gaussians (bench.py --config 3: 125000 = 8 mod 16). Clusters then go empty, their centroids become 0 / 0 =
    NaN and stay NaN: ten iterations of that degenerate run against the oracle - labels bit-exact off near-ties, the
    same centroids NaN, the same cluster sizes, the others within 1e-4. Clusters that split one Gaussian between them
    make the run sensitive to single labels, so every iteration starts from the oracle's centroids (NaN rows included):
    what is compared is the device's step from each state of the trajectory, not two trajectories drifting apart."""
    rng = np.random.default_rng(4)
    k, f = 16, 64
    stride = 2008                      # = 8 mod 16, like 125000
    n = k * stride
    centres = rng.standard_normal((k, f)) * 5
    X = (centres[np.arange(n) % k] + rng.standard_normal((n, f))).astype(np.float32)
    seeds = np.arange(k) * stride
    assert set((seeds % k).tolist()) == {0, 8}
    C0 = np.ascontiguousarray(X[seeds])
    xx = orc.agg_row(AggOpCode.SUM, orc.ew_binary(BinaryOpCode.MUL, X, X)[1])[1]
    km = KMeans(ctx, DenseMatrix.from_numpy(ctx, X), k)
    Ce = C0
    saw_empty = False
    for it in range(10):
        Cd = km.iterate(DenseMatrix.from_numpy(ctx, Ce), fused=fused)
        with np.errstate(invalid="ignore", divide="ignore"):
            Ce, idx_e, D = _orc_kmeans_iter(X, Ce, xx)
        Dn = np.where(np.isnan(D), np.inf, D)
        part = np.partition(Dn, 1, axis=1)
        with np.errstate(invalid="ignore"):
            near_tie = ~((part[:, 1] - part[:, 0]) > 1e-3 * np.abs(part[:, 0]))
        idx_d = km.idx.to_numpy()
        assert_exact(idx_d[~near_tie], idx_e[~near_tie])
        Cg = Cd.to_numpy()
        nan_e = np.isnan(Ce).any(axis=1)
        saw_empty |= bool(nan_e.any())
        if not near_tie.any():
            assert_exact(np.isnan(Cg), np.isnan(Ce))
            assert_exact(km.counts.to_numpy()[0], np.bincount(idx_e[:, 0].astype(np.int64), minlength=k).astype(np.float32))
            assert_close(Cg[~nan_e], Ce[~nan_e], rtol=1e-4, elementwise=False)
        else:  # a row on the fence may change a size by one; the set of dead clusters cannot depend on it here
            assert_exact(np.isnan(Cg).any(axis=1), nan_e)
    assert saw_empty, "the seeding was meant to leave clusters empty"


def test_config3_full_size_properties(ctx):
    """2M x 64: one-hot rows sum to one, counts sum to n, P agrees with idx, centroids equal the per-cluster
    means computed independently in float64 on the device."""
    k, f, n = 16, 64, 2_000_000
    g = torch.Generator(device="cuda").manual_seed(5)
    centres = torch.randn(k, f, device="cuda", generator=g) * 5
    Xt = centres[torch.arange(n, device="cuda") % k] + torch.randn(n, f, device="cuda", generator=g)
    X = DenseMatrix.from_torch(ctx, Xt)
    km = KMeans(ctx, X, k)
    C = DenseMatrix.from_torch(ctx, Xt[torch.arange(k, device="cuda") * (n // k) + torch.arange(k, device="cuda")].contiguous())
    for _ in range(2):
        C = km.iterate(C)
    # the two passes over X against the operator sequence from the same centroids: the same assignment bit for bit
    # (the product comes from the same streaming kernel), the same sizes, centroids to rounding
    C_seq = km.iterate(C, fused=False)
    idx_seq, counts_seq = km.idx.to_numpy().copy(), km.counts.to_numpy().copy()
    C2 = km.iterate(C, fused="two_passes")
    assert_exact(km.idx.to_numpy(), idx_seq)
    assert_exact(km.counts.to_numpy(), counts_seq)
    assert_close(C2.to_numpy(), C_seq.to_numpy(), rtol=1e-5, elementwise=False)
    C = km.iterate(C)
    assert_exact(km.idx.to_numpy(), idx_seq)
    assert_exact(km.counts.to_numpy(), counts_seq)
    assert float(km.counts.to_numpy().sum()) == n
    assert_close(C.to_numpy(), C_seq.to_numpy(), rtol=1e-5, elementwise=False)
    idx = torch.from_numpy(km.idx.to_numpy()[:, 0].astype(np.int64)).cuda()
    P = torch.from_numpy(km.P.to_numpy()).cuda()
    assert bool((P.sum(1) == 1).all()) and float(P.sum()) == n
    assert bool((P.argmax(1) == idx).all())
    means = torch.zeros(k, f, device="cuda", dtype=torch.float64).index_add_(0, idx, Xt.to(torch.float64))
    means /= torch.bincount(idx, minlength=k).to(torch.float64)[:, None]
    assert_close(C.to_numpy(), means.cpu().numpy().astype(np.float32), rtol=1e-4, elementwise=False)
    del Xt, P
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dt,n,tol", [(np.float64, 2048, 1e-10), (np.float32, 4096, 1e-4)])
def test_config4_matmul_sampled_entries_extended_precision(ctx, dt, n, tol):
    rng = np.random.default_rng(11)
    A = (rng.random((n, n)) * 2 - 1).astype(dt)
    B = (rng.random((n, n)) * 2 - 1).astype(dt)
    C = matMul(None, DenseMatrix.from_numpy(ctx, A), DenseMatrix.from_numpy(ctx, B), False, False, ctx).to_numpy()
    ii, jj = rng.integers(0, n, 256), rng.integers(0, n, 256)
    exact = np.array([np.dot(A[i].astype(np.longdouble), B[:, j].astype(np.longdouble)) for i, j in zip(ii, jj)])
    scale = float(np.abs(C).max())
    assert np.abs(C[ii, jj].astype(np.longdouble) - exact).max() <= tol * scale


def test_config4_syrk_tall_prefix_and_symmetry(ctx):
    """Syrk f64 on a tall 200000 x 1024 matrix (split-K path): symmetric, equals matMul(t(X), X), and a
    4096-row prefix equals the CPU oracle."""
    rng = np.random.default_rng(12)
    X = rng.random((200_000, 1024)) * 2 - 1
    dX = DenseMatrix.from_numpy(ctx, X)
    S = syrk(None, dX, True, ctx).to_numpy()
    assert_exact(S, S.T)
    assert_close(S, matMul(None, dX, dX, True, False, ctx).to_numpy(), elementwise=False)
    Xp = np.ascontiguousarray(X[:4096, :256])
    assert_close(syrk(None, DenseMatrix.from_numpy(ctx, Xp), True, ctx).to_numpy(), orc.syrk(Xp, True)[1], elementwise=False)


def _sampled_products(A_rows, B_cols):
    """All pairwise dot products of the given rows and columns (host arrays, K values each) in extended precision,
    with the sum of absolute terms that bounds the rounding error of any summation order."""
    a, b = A_rows.astype(np.longdouble), B_cols.astype(np.longdouble)
    return a @ b.T, np.abs(a) @ np.abs(b).T


@pytest.mark.parametrize("dt,n,tol", [(np.float64, 8192, 1e-10), (np.float32, 16384, 1e-4)])
def test_config4_matmul_at_the_quoted_sizes(ctx, dt, n, tol):
    """MatMul at the sizes the throughput is quoted on (8192^3 f64, 16384^3 f32: grids whose tile count is a multiple
    of the XCD count, the regrouped tile order). Inputs are generated on the device; 16 rows x 16 columns = 256
    results are checked against extended-precision dot products on the host, and a 512-row band of the result against
    the same kernel run on that band alone (other grid, other tile order; every entry of the band is compared)."""
    import torch

    tdt = torch.float64 if dt == np.float64 else torch.float32
    gen = torch.Generator(device="cuda").manual_seed(21)
    A = torch.rand(n, n, device="cuda", dtype=tdt, generator=gen) * 2 - 1
    B = torch.rand(n, n, device="cuda", dtype=tdt, generator=gen) * 2 - 1
    Cm = torch.full((n, n), float("nan"), device="cuda", dtype=tdt)
    matMul(DenseMatrix.from_torch(ctx, Cm), DenseMatrix.from_torch(ctx, A), DenseMatrix.from_torch(ctx, B), False, False, ctx)
    torch.cuda.synchronize()
    assert not bool(torch.isnan(Cm).any()), "some tile of the result was not written"
    rng = np.random.default_rng(22)
    # rows and columns from the first, the last and random tiles
    ii = np.unique(np.concatenate([[0, n - 1, 127, 128], rng.integers(0, n, 12)]))[:16]
    jj = np.unique(np.concatenate([[0, n - 1, 255, 256], rng.integers(0, n, 12)]))[:16]
    ti, tj = torch.as_tensor(ii, device="cuda"), torch.as_tensor(jj, device="cuda")
    exact, bound = _sampled_products(A[ti].cpu().numpy(), B[:, tj].T.contiguous().cpu().numpy())
    got = Cm[ti][:, tj].cpu().numpy().astype(np.longdouble)
    assert exact.size >= 256 - 32
    assert (np.abs(got - exact) <= tol * bound).all(), float((np.abs(got - exact) / bound).max())
    band = slice(n // 2 - 256, n // 2 + 256)
    Cb = torch.empty(512, n, device="cuda", dtype=tdt)
    matMul(DenseMatrix.from_torch(ctx, Cb), DenseMatrix.from_torch(ctx, A[band]), DenseMatrix.from_torch(ctx, B), False, False, ctx)
    torch.cuda.synchronize()
    assert float((Cb - Cm[band]).abs().max()) <= tol * float(Cm[band].abs().max())
    del A, B, Cm, Cb
    torch.cuda.empty_cache()


def test_config4_syrk_at_the_quoted_size(ctx):
    """Syrk f64 t(X) X with X 1,000,000 x 1024 (the full split over the rows, the slab reduction and the mirror
    step): bit-exact symmetry, all 16 x 16 results among 16 sampled columns against extended-precision dot products,
    and the whole result against MatMul(t(X), X) norm-wise."""
    import torch

    rows, n = 1_000_000, 1024
    gen = torch.Generator(device="cuda").manual_seed(23)
    X = torch.rand(rows, n, device="cuda", dtype=torch.float64, generator=gen) * 2 - 1
    S = torch.full((n, n), float("nan"), device="cuda", dtype=torch.float64)
    dX = DenseMatrix.from_torch(ctx, X)
    syrk(DenseMatrix.from_torch(ctx, S), dX, True, ctx)
    torch.cuda.synchronize()
    assert not bool(torch.isnan(S).any())
    assert bool((S == S.T).all())
    cols = np.unique(np.concatenate([[0, n - 1, 63, 64, 511, 512], np.random.default_rng(24).integers(0, n, 12)]))[:16]
    Xc = X[:, torch.as_tensor(cols, device="cuda")].T.contiguous().cpu().numpy()  # 16 x 1e6
    exact, bound = _sampled_products(Xc, Xc)
    got = S[torch.as_tensor(cols, device="cuda")][:, torch.as_tensor(cols, device="cuda")].cpu().numpy().astype(np.longdouble)
    assert (np.abs(got - exact) <= 1e-10 * bound).all(), float((np.abs(got - exact) / bound).max())
    M = torch.empty(n, n, device="cuda", dtype=torch.float64)
    matMul(DenseMatrix.from_torch(ctx, M), dX, dX, True, False, ctx)
    torch.cuda.synchronize()
    assert float((S - M).abs().max()) <= 1e-10 * float(M.abs().max())
    del X, S, M, dX
    torch.cuda.empty_cache()


def _lenet_weights(rng):
    he = lambda shape, fan: (rng.standard_normal(shape) * np.sqrt(2.0 / fan)).astype(np.float32)
    small = lambda shape: (rng.standard_normal(shape) * 0.1).astype(np.float32)
    return {"w1": he((32, 25), 25), "b1": small((32, 1)), "w2": he((64, 800), 800), "b2": small((64, 1)),
            "w3": he((3136, 512), 3136), "b3": small((1, 512)), "w4": he((512, 10), 512), "b4": small((1, 10))}


def _orc_lenet(x, W, N):
    relu = lambda a: orc.ew_binary_sca(BinaryOpCode.MAX, a, 0.0)[1]
    h = relu(orc.conv2d(x, W["w1"], W["b1"], N, 1, 28, 28, 5, 5, 1, 1, 2, 2)[1])
    h = orc.maxpool(h, N, 32, 28, 28, 2, 2, 2, 2, 0, 0)[1]
    h = relu(orc.conv2d(h, W["w2"], W["b2"], N, 32, 14, 14, 5, 5, 1, 1, 2, 2)[1])
    h = orc.maxpool(h, N, 64, 14, 14, 2, 2, 2, 2, 0, 0)[1]
    h = relu(orc.ew_binary(0, orc.matmul(h, W["w3"])[1], W["b3"])[1])
    h = orc.ew_binary(0, orc.matmul(h, W["w4"])[1], W["b4"])[1]
    return orc.softmax(h)[1]


def test_config5_lenet_against_oracle_and_batch_independence(ctx):
    rng = np.random.default_rng(13)
    W = _lenet_weights(rng)
    Wd = {k: DenseMatrix.from_numpy(ctx, v) for k, v in W.items()}
    x = rng.random((4096, 784)).astype(np.float32)
    small = np.ascontiguousarray(x[:24])
    exp = _orc_lenet(small, W, 24)
    got_small = lenet_forward(ctx, DenseMatrix.from_numpy(ctx, small), Wd, 24).to_numpy()
    assert_close(got_small, exp, rtol=1e-4, elementwise=False)
    full = lenet_forward(ctx, DenseMatrix.from_numpy(ctx, x), Wd, 4096).to_numpy()
    assert full.shape == (4096, 10)
    # one kernel per operator gives the same numbers as the layers with fused epilogues, bit for bit
    assert_exact(lenet_forward(ctx, DenseMatrix.from_numpy(ctx, x), Wd, 4096, fused=False).to_numpy(), full)
    assert_exact(lenet_forward(ctx, DenseMatrix.from_numpy(ctx, small), Wd, 24, fused=False).to_numpy(), got_small)
    assert_close(full[:24], got_small, rtol=1e-5, elementwise=False)  # images do not interact
    assert np.allclose(full.sum(1), 1.0, rtol=1e-5)
