"""GPU parity: Conv2D / MaxPool / BiasAdd / BatchNorm / Softmax (through the C ABI) vs the CPU oracle."""
import numpy as np
import pytest

import oracle_binding as orc
from parity import assert_close, assert_exact

pytestmark = pytest.mark.gpu

from daphne_amd import capi
from daphne_amd.kernels import (DenseMatrix, batchNormInferenceForward, biasAdd, conv2dForward, conv2dForwardFused,
                                maxPoolForward, reluForward, softmax)

DTYPES = [np.float32, np.float64]

CONV_CASES = [  # N, C, H, W, F, Hf, Wf, sh, sw, ph, pw
    (2, 3, 3, 3, 1, 2, 2, 2, 2, 1, 1),
    (1, 1, 3, 3, 1, 2, 2, 1, 1, 0, 0),
    (5, 1, 28, 28, 32, 5, 5, 1, 1, 2, 2),
    (3, 32, 14, 14, 64, 5, 5, 1, 1, 2, 2),
    (4, 3, 17, 13, 70, 3, 5, 2, 1, 1, 2),
    (2, 8, 9, 9, 130, 3, 3, 1, 2, 0, 1),
    (130, 2, 5, 6, 5, 1, 1, 1, 1, 0, 0),
    (1, 4, 7, 7, 3, 7, 7, 1, 1, 0, 0),
    # images of at least 127 output pixels (the tile of 128 pixels spans at most two images): channel stages with a
    # partial last stage, strides, wide rows, 1x1 filters, K tails
    (3, 20, 16, 16, 24, 3, 3, 1, 1, 1, 1),
    (2, 4, 33, 31, 10, 3, 3, 2, 2, 1, 1),
    (2, 2, 12, 200, 6, 3, 5, 1, 1, 1, 2),
    (3, 16, 12, 12, 64, 1, 1, 1, 1, 0, 0),
    (2, 7, 20, 9, 33, 4, 2, 1, 1, 0, 0),
    (1, 40, 15, 15, 16, 3, 3, 1, 1, 1, 1),
    (7, 3, 13, 11, 5, 3, 3, 1, 1, 1, 1),
    # shapes for the kernel that keeps the image in LDS: pixel chunks (1600 pixels, 13 blocks a wave), three channel
    # stages, a partial last stage (26 + 25 channels in float, 17 x 3 in double), 8 filters on a large image (one
    # filter block per workgroup, 8 pixel parts), stride 2 with 20 filters (two filter blocks, 4 pixel parts)
    (2, 6, 40, 40, 64, 3, 3, 1, 1, 1, 1),
    (2, 96, 14, 14, 32, 5, 5, 1, 1, 2, 2),
    (2, 51, 14, 14, 48, 4, 4, 1, 1, 1, 1),
    (2, 4, 32, 32, 8, 3, 3, 1, 1, 1, 1),
    (1, 5, 30, 30, 20, 3, 3, 2, 2, 0, 0),
    # small feature maps: several images per workgroup (8 + 1 of 7 x 7, 12 + 8 of 4 x 4, 3 + 3 + 1 without a border and
    # in four channel stages)
    (9, 16, 7, 7, 32, 3, 3, 1, 1, 1, 1),
    (20, 8, 4, 4, 64, 3, 3, 1, 1, 1, 1),
    (7, 64, 14, 14, 32, 5, 5, 1, 1, 0, 0),
    # channels in whole groups of 16 (8 in double): the LDS image with its channels interleaved - strides, a partial
    # filter block, three stages of 16 channels, 24 channels (interleaved in double only), odd planes
    (6, 16, 15, 13, 20, 3, 3, 2, 2, 1, 1),
    (2, 48, 12, 12, 40, 3, 3, 1, 2, 0, 1),
    (4, 24, 10, 10, 33, 3, 3, 1, 1, 1, 1),
    (5, 32, 9, 11, 64, 2, 4, 1, 1, 1, 0),
    # fewer than 32 filter taps: 33 filters (a partial filter block) and
    # uneven strides, 17 filters with wide padding, 31 taps in a column, more than 256 pixels per image
    (3, 1, 19, 23, 33, 3, 5, 2, 3, 1, 2),
    (2, 3, 9, 9, 17, 3, 3, 1, 1, 2, 2),
    (2, 1, 40, 40, 9, 31, 1, 1, 1, 15, 0),
    (70, 1, 28, 28, 6, 5, 5, 1, 1, 0, 0),
]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d(ctx, dt, case):
    N, C, H, W, F, Hf, Wf, sh, sw, ph, pw = case
    rng = np.random.default_rng(sum(case))
    x = rng.random((N, C * H * W)).astype(dt)
    w = (rng.standard_normal((F, C * Hf * Wf)) * np.sqrt(2.0 / (C * Hf * Wf))).astype(dt)
    b = (rng.standard_normal((F, 1)) * 0.1).astype(dt)
    st, exp, eh, ew_ = orc.conv2d(x, w, b, N, C, H, W, Hf, Wf, sh, sw, ph, pw)
    assert st == 0
    X, Wd, B = DenseMatrix.from_numpy(ctx, x), DenseMatrix.from_numpy(ctx, w), DenseMatrix.from_numpy(ctx, b)
    got, gh, gw = conv2dForward(None, X, Wd, B, N, C, H, W, Hf, Wf, sh, sw, ph, pw, ctx)
    assert (gh, gw) == (eh, ew_)
    assert_close(got.to_numpy(), exp, elementwise=False)
    # without bias (allowed by the reference's CUDA kernel)
    st, exp0, _, _ = orc.conv2d(x, w, None, N, C, H, W, Hf, Wf, sh, sw, ph, pw)
    got0, _, _ = conv2dForward(None, X, Wd, None, N, C, H, W, Hf, Wf, sh, sw, ph, pw, ctx)
    assert_close(got0.to_numpy(), exp0, elementwise=False)


FUSED_CONV_CASES = CONV_CASES + [
    # the layers of the LeNet configuration at a batch that leaves partial pixel blocks, odd result planes (the last
    # row and column fall outside every 2 x 2 window), planes of a single window, many filters
    (37, 1, 28, 28, 32, 5, 5, 1, 1, 2, 2),
    (19, 32, 14, 14, 64, 5, 5, 1, 1, 2, 2),
    (5, 3, 15, 13, 20, 3, 3, 1, 1, 1, 1),
    (6, 2, 11, 11, 70, 3, 3, 1, 1, 0, 0),
    (40, 5, 4, 4, 16, 3, 3, 1, 1, 0, 0),
    (3, 1, 64, 64, 8, 5, 5, 1, 1, 2, 2),
    # one channel, even result planes (a thread per 2 x 2 quad of pixels): 3 x 3 with and without padding, filter
    # counts that are no multiple of four
    (9, 1, 12, 10, 7, 3, 3, 1, 1, 1, 1),
    (5, 1, 10, 8, 5, 3, 3, 1, 1, 0, 0),
    (300, 1, 28, 28, 6, 5, 5, 1, 1, 2, 2),
]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", FUSED_CONV_CASES)
def test_conv2d_fused_epilogues_equal_the_operator_sequence(ctx, dt, case):
    """conv2d -> relu -> max_pool2d(2 x 2, stride 2) in one call gives the numbers of the three kernels bit for bit
    (the fused kernel where the image fits LDS, the sequence through a temporary elsewhere), and those of the oracle."""
    N, C, H, W, F, Hf, Wf, sh, sw, ph, pw = case
    rng = np.random.default_rng(sum(case) + 5)
    x = (rng.random((N, C * H * W)) - 0.3).astype(dt)
    w = (rng.standard_normal((F, C * Hf * Wf)) * np.sqrt(2.0 / (C * Hf * Wf))).astype(dt)
    b = (rng.standard_normal((F, 1)) * 0.1).astype(dt)
    X, Wd, B = DenseMatrix.from_numpy(ctx, x), DenseMatrix.from_numpy(ctx, w), DenseMatrix.from_numpy(ctx, b)
    conv, P, Q = conv2dForward(None, X, Wd, B, N, C, H, W, Hf, Wf, sh, sw, ph, pw, ctx)
    relu = reluForward(None, conv, ctx)
    got, gh, gw = conv2dForwardFused(None, X, Wd, B, N, C, H, W, Hf, Wf, sh, sw, ph, pw, ctx, relu=True, pool=False)
    assert (gh, gw) == (P, Q)
    assert_exact(got.to_numpy(), relu.to_numpy())
    assert (relu.to_numpy() == 0).any() and (relu.to_numpy() > 0).any()
    got0, _, _ = conv2dForwardFused(None, X, Wd, None, N, C, H, W, Hf, Wf, sh, sw, ph, pw, ctx, relu=True, pool=False)
    conv0, _, _ = conv2dForward(None, X, Wd, None, N, C, H, W, Hf, Wf, sh, sw, ph, pw, ctx)
    assert_exact(got0.to_numpy(), reluForward(None, conv0, ctx).to_numpy())
    if P < 2 or Q < 2:
        with pytest.raises(capi.DaphneHipError, match="window 2x2 does not fit"):
            conv2dForwardFused(None, X, Wd, B, N, C, H, W, Hf, Wf, sh, sw, ph, pw, ctx, relu=True, pool=True)
        return
    for with_relu, before_pool in ((True, relu), (False, conv)):
        pooled, ph_, pw_ = maxPoolForward(None, before_pool, N, F, P, Q, 2, 2, 2, 2, 0, 0, ctx)
        got, gh, gw = conv2dForwardFused(None, X, Wd, B, N, C, H, W, Hf, Wf, sh, sw, ph, pw, ctx, relu=with_relu, pool=True)
        assert (gh, gw) == (ph_, pw_) == (P // 2, Q // 2)
        assert_exact(got.to_numpy(), pooled.to_numpy())
    st, oc, _, _ = orc.conv2d(x, w, b, N, C, H, W, Hf, Wf, sh, sw, ph, pw)
    st, orl = orc.ew_binary_sca(14, oc, 0.0)
    st, op, _, _ = orc.maxpool(orl, N, F, P, Q, 2, 2, 2, 2, 0, 0)
    assert_close(got.to_numpy(), op, elementwise=False)


@pytest.mark.parametrize("dt", DTYPES)
def test_conv2d_one_channel_special_values(ctx, dt):
    """NaN, infinities and zeros of both signs go through the one-channel kernel's pooled store as through the three
    separate kernels (the pooled store leaves the rectifier out: a running maximum from zero does not need it)."""
    N, H, W, F = 6, 12, 12, 5
    rng = np.random.default_rng(31)
    x = (rng.random((N, H * W)) - 0.5).astype(dt)
    x[0, 17], x[1, 40], x[2, 5], x[3, 77] = np.nan, np.inf, -np.inf, -0.0
    x[4, :] = -0.0
    w = rng.standard_normal((F, 25)).astype(dt)
    w[1, :] = 0.0
    w[2, :] = -np.abs(w[2, :])
    b = np.array([[0.1], [-0.0], [0.0], [-0.2], [0.3]], dtype=dt)
    X, Wd, B = DenseMatrix.from_numpy(ctx, x), DenseMatrix.from_numpy(ctx, w), DenseMatrix.from_numpy(ctx, b)
    conv, P, Q = conv2dForward(None, X, Wd, B, N, 1, H, W, 5, 5, 1, 1, 2, 2, ctx)
    for with_relu in (True, False):
        before = reluForward(None, conv, ctx) if with_relu else conv
        pooled, _, _ = maxPoolForward(None, before, N, F, P, Q, 2, 2, 2, 2, 0, 0, ctx)
        got, _, _ = conv2dForwardFused(None, X, Wd, B, N, 1, H, W, 5, 5, 1, 1, 2, 2, ctx, relu=with_relu, pool=True)
        g, e = got.to_numpy(), pooled.to_numpy()
        assert_exact(g, e)
        assert (np.signbit(g) == np.signbit(e))[~np.isnan(e)].all()
        unp, _, _ = conv2dForwardFused(None, X, Wd, B, N, 1, H, W, 5, 5, 1, 1, 2, 2, ctx, relu=with_relu, pool=False)
        assert_exact(unp.to_numpy(), before.to_numpy())
        assert (np.signbit(unp.to_numpy()) == np.signbit(before.to_numpy()))[~np.isnan(before.to_numpy())].all()
    assert np.isnan(conv.to_numpy()).any() and np.isinf(conv.to_numpy()).any()
    st, oc, _, _ = orc.conv2d(x, w, b, N, 1, H, W, 5, 5, 1, 1, 2, 2)
    finite = np.isfinite(oc)
    assert (np.isfinite(conv.to_numpy()) == finite).all()
    assert_close(conv.to_numpy()[finite], oc[finite], elementwise=False)


def test_conv2d_fused_rejects_unknown_flags(ctx):
    x, w = DenseMatrix.from_numpy(ctx, np.ones((1, 16), np.float32)), DenseMatrix.from_numpy(ctx, np.ones((1, 4), np.float32))
    res = DenseMatrix(ctx, 1, 9, np.float32)
    import ctypes as C
    rh, rw = C.c_size_t(), C.c_size_t()
    st = capi.lib().dh_conv2d_forward_fused_f32(ctx._h, res.ptr, C.byref(rh), C.byref(rw), x.ptr, w.ptr, 1, 4, None, 1, 1, 4, 4, 2, 2,
                                                1, 1, 0, 0, 8)
    assert st != 0 and b"unknown epilogue" in capi.lib().dh_last_error()


@pytest.mark.parametrize("dt", DTYPES)
def test_conv2d_integer_valued_exact(ctx, dt):
    rng = np.random.default_rng(4)
    N, C, H, W, F, Hf, Wf = 3, 5, 11, 12, 40, 3, 3
    x = rng.integers(-3, 4, (N, C * H * W)).astype(dt)
    w = rng.integers(-3, 4, (F, C * Hf * Wf)).astype(dt)
    b = rng.integers(-3, 4, (F, 1)).astype(dt)
    st, exp, _, _ = orc.conv2d(x, w, b, N, C, H, W, Hf, Wf, 1, 1, 1, 1)
    got, _, _ = conv2dForward(None, DenseMatrix.from_numpy(ctx, x), DenseMatrix.from_numpy(ctx, w),
                              DenseMatrix.from_numpy(ctx, b), N, C, H, W, Hf, Wf, 1, 1, 1, 1, ctx)
    assert_exact(got.to_numpy(), exp)


@pytest.mark.parametrize("dt", DTYPES)
def test_conv2d_non_finite_inputs_stay_local(ctx, dt):
    """An infinity or NaN in the image reaches exactly the outputs whose window covers it - in particular the zero
    padding of the K dimension (45 taps in tiles of 16 / 8) must not multiply it into anything."""
    rng = np.random.default_rng(9)
    N, C, H, W, F, Hf, Wf = 2, 5, 12, 12, 9, 3, 3
    x = rng.random((N, C * H * W)).astype(dt)
    x[0, 0] = np.inf          # image 0, channel 0, (0, 0)
    x[1, 3 * H * W + 5 * W + 7] = np.nan
    w = (rng.random((F, C * Hf * Wf)) + 0.5).astype(dt)
    st, exp, _, _ = orc.conv2d(x, w, None, N, C, H, W, Hf, Wf, 1, 1, 1, 1)
    got, _, _ = conv2dForward(None, DenseMatrix.from_numpy(ctx, x), DenseMatrix.from_numpy(ctx, w), None, N, C, H, W, Hf, Wf,
                              1, 1, 1, 1, ctx)
    got = got.to_numpy()
    assert np.array_equal(np.isfinite(got), np.isfinite(exp))
    assert np.array_equal(np.isnan(got), np.isnan(exp))
    fin = np.isfinite(exp)
    assert_close(got[fin], exp[fin], elementwise=False)


def test_conv2d_filter_mismatch(ctx):
    x = DenseMatrix.from_numpy(ctx, np.ones((1, 9), np.float32))
    w = DenseMatrix.from_numpy(ctx, np.ones((1, 5), np.float32))
    with pytest.raises(capi.DaphneHipInvalidArgument, match="Convolution kernel dimension mismatch"):
        conv2dForward(None, x, w, None, 1, 1, 3, 3, 2, 2, 1, 1, 0, 0, ctx)


POOL_CASES = [  # N, C, H, W, ph, pw, sh, sw, padh, padw
    (2, 3, 5, 5, 2, 2, 2, 2, 1, 1),
    (2, 3, 5, 5, 2, 2, 1, 1, 0, 0),
    (3, 32, 28, 28, 2, 2, 2, 2, 0, 0),
    (3, 64, 14, 14, 2, 2, 2, 2, 0, 0),
    (2, 2, 9, 7, 3, 3, 2, 2, 1, 1),
    (2, 2, 9, 7, 3, 2, 3, 3, 0, 0),
    (4, 5, 6, 1, 6, 1, 1, 1, 0, 0),   # P == Q == 1 and W == 1: the reference's quick path
    (1, 1, 4, 4, 4, 4, 1, 1, 0, 0),
    (333, 64, 14, 14, 3, 3, 2, 2, 1, 1),  # several planes per workgroup staged in LDS, short last workgroup
    (301, 33, 7, 7, 3, 3, 1, 1, 1, 1),    # planes of 49 values: workgroups of a multiple of four planes, scalar tail
    (5, 7, 5, 5, 3, 3, 2, 2, 0, 0),
    (1, 3, 7, 9, 2, 3, 1, 2, 1, 0),       # fewer planes than fill a vector-aligned workgroup
    (2, 2, 80, 80, 3, 3, 2, 2, 1, 1),     # planes too large for the LDS kernel
    (2, 3, 64, 64, 5, 5, 3, 3, 2, 2),     # one 16 KB plane per workgroup (float)
    (7, 11887, 14, 14, 3, 3, 2, 2, 1, 1), # thousands of workgroups, short last one
]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", POOL_CASES)
def test_maxpool(ctx, dt, case):
    N, C, H, W, ph, pw, sh, sw, padh, padw = case
    rng = np.random.default_rng(sum(case))
    x = (rng.standard_normal((N, C * H * W))).astype(dt)  # negative values: the result is max(0, window)
    st, exp, eh, ew_ = orc.maxpool(x, N, C, H, W, ph, pw, sh, sw, padh, padw)
    assert st == 0
    got, gh, gw = maxPoolForward(None, DenseMatrix.from_numpy(ctx, x), N, C, H, W, ph, pw, sh, sw, padh, padw, ctx)
    assert (gh, gw) == (eh, ew_)
    assert_exact(got.to_numpy(), exp)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,C,HW", [(2, 3, 9), (7, 32, 784), (5, 64, 196), (9, 10, 1), (3, 5, 7), (100, 1, 33)])
def test_bias_add(ctx, dt, rows, C, HW):
    rng = np.random.default_rng(rows + C + HW)
    x = rng.standard_normal((rows, C * HW)).astype(dt)
    for bshape in ((C, 1), (1, C)):  # CPU test uses C x 1, the CUDA test 1 x C
        b = rng.standard_normal(bshape).astype(dt)
        st, exp = orc.bias_add(x, b)
        got = biasAdd(None, DenseMatrix.from_numpy(ctx, x), DenseMatrix.from_numpy(ctx, b), ctx).to_numpy()
        assert_exact(got, exp)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,C,HW", [(1, 1, 9), (2, 3, 9), (6, 16, 49), (5, 7, 3)])
def test_batchnorm_inference(ctx, dt, rows, C, HW):
    rng = np.random.default_rng(rows * 7 + C)
    x = rng.standard_normal((rows, C * HW)).astype(dt)
    eps = 1e-5
    for stat_index, S in ((0, C), (1, rows)):
        gamma = (rng.random((S, 1)) + 0.5).astype(dt)
        beta = rng.standard_normal((S, 1)).astype(dt)
        mean = rng.standard_normal((S, 1)).astype(dt)
        var = (rng.random((S, 1)) + 0.1).astype(dt)
        st, exp = orc.batchnorm(x, gamma, beta, mean, var, eps, stat_index)
        assert st == 0
        d = lambda a: DenseMatrix.from_numpy(ctx, a)
        got = batchNormInferenceForward(None, d(x), d(gamma), d(beta), d(mean), d(var), eps, ctx, stat_index).to_numpy()
        assert_close(got, exp, rtol=2e-5 if dt == np.float32 else 1e-12, elementwise=False)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,cols", [(3, 3), (1, 9), (4096, 10), (7, 1), (33, 1000), (5, 64),
                                       # short rows staged through LDS: a partial last workgroup, a scalar tail, 31 values
                                       (5000, 10), (1030, 7), (2000, 31), (1500, 1), (1024, 12),
                                       # two rows a thread (2^18 rows or more, up to 10 floats / 5 doubles a row)
                                       (262444, 10), (300001, 5), (262145, 3)])
def test_softmax(ctx, dt, rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = (rng.standard_normal((rows, cols)) * 4).astype(dt)
    if rows > 2 and cols > 2:
        x[1, 1] = np.nan
        x[2, 0] = np.inf
    st, exp = orc.softmax(x)
    got = softmax(None, DenseMatrix.from_numpy(ctx, x), ctx).to_numpy()
    assert_close(got, exp)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("seed", range(12))
def test_conv2d_random_shapes_with_whole_channel_groups(ctx, dt, seed):
    """Seeded random shapes whose channel counts come in whole groups of 16 (8 in double) - the LDS image with its
    channels interleaved where it fits, the plane layout or the tiled kernel elsewhere - against the oracle, plain and
    with ReLU and pooling folded in."""
    rng = np.random.default_rng(1000 + seed)
    C = int(rng.choice([8, 16, 24, 32, 48, 64]))
    Hf, Wf = int(rng.integers(1, 6)), int(rng.integers(1, 6))
    sh, sw = int(rng.integers(1, 3)), int(rng.integers(1, 3))
    ph, pw = int(rng.integers(0, (Hf + 1) // 2 + 1)), int(rng.integers(0, (Wf + 1) // 2 + 1))
    H, W = int(rng.integers(max(Hf, 6), 23)), int(rng.integers(max(Wf, 6), 23))
    F = int(rng.choice([17, 20, 32, 33, 48, 64, 70]))
    N = int(rng.integers(1, 12))
    x = (rng.random((N, C * H * W)) - 0.4).astype(dt)
    w = (rng.standard_normal((F, C * Hf * Wf)) * np.sqrt(2.0 / (C * Hf * Wf))).astype(dt)
    b = (rng.standard_normal((F, 1)) * 0.1).astype(dt)
    st, exp, eh, ew_ = orc.conv2d(x, w, b, N, C, H, W, Hf, Wf, sh, sw, ph, pw)
    assert st == 0
    X, Wd, B = DenseMatrix.from_numpy(ctx, x), DenseMatrix.from_numpy(ctx, w), DenseMatrix.from_numpy(ctx, b)
    got, gh, gw = conv2dForward(None, X, Wd, B, N, C, H, W, Hf, Wf, sh, sw, ph, pw, ctx)
    assert (gh, gw) == (eh, ew_)
    assert_close(got.to_numpy(), exp, elementwise=False)
    if eh >= 2 and ew_ >= 2:
        fused, fh, fw = conv2dForwardFused(None, X, Wd, B, N, C, H, W, Hf, Wf, sh, sw, ph, pw, ctx, relu=True, pool=True)
        r = np.maximum(got.to_numpy().reshape(N, F, eh, ew_), 0)
        want = r[:, :, : eh // 2 * 2, : ew_ // 2 * 2].reshape(N, F, eh // 2, 2, ew_ // 2, 2).max(axis=(3, 5))
        assert (fh, fw) == (eh // 2, ew_ // 2)
        assert_exact(fused.to_numpy(), want.reshape(N, -1).astype(dt))  # the epilogue on the same sums: bit for bit
