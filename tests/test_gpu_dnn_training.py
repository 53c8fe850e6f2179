"""GPU parity: DNN training kernels (batch-norm training forward, batch-norm / pooling / convolution backward) through
the C ABI against the CPU oracle. Tolerances: relative 1e-4 (float) / 1e-10 (double), norm-wise where sums of many
terms are compared (the device accumulates per-channel and per-filter sums in double, in a different order than the
oracle's sequential loops); pooling gradients are bit-exact (same order of additions)."""
import numpy as np
import pytest

import oracle_binding as orc
from parity import assert_close, assert_exact

pytestmark = pytest.mark.gpu

from daphne_amd import capi
from daphne_amd.kernels import (DenseMatrix, avgPoolBackward, batchNorm2DBackward, batchNorm2DTrainForward, conv2DBackwardData,
                                conv2DBackwardFilter, conv2dForward, maxPoolBackward)

DTYPES = [np.float32, np.float64]


def D(ctx, a):
    return DenseMatrix.from_numpy(ctx, a)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("N,C,H,W", [(2, 3, 3, 3), (64, 8, 14, 14), (7, 5, 9, 11), (1, 1, 1, 1), (300, 3, 8, 8), (3, 130, 2, 2),
                                     # a channel's values beyond a workgroup's LDS (the general passes), many channels that
                                     # fit (one read), and a size where the forward fits and the backward in double does not
                                     (513, 4, 7, 9), (40, 70, 5, 5), (128, 16, 6, 10)])
def test_batchnorm_train_forward_and_backward(ctx, dt, N, C, H, W):
    rng = np.random.default_rng(N * 7 + C)
    x = (rng.standard_normal((N, C * H * W)) * 2 + 1).astype(dt)
    gamma, beta = (rng.random((C, 1)) + 0.5).astype(dt), rng.standard_normal((C, 1)).astype(dt)
    em, ev = rng.standard_normal((C, 1)).astype(dt), (rng.random((C, 1)) + 0.5).astype(dt)
    eps, mu = 1e-5, 0.25
    st, res_e, nm_e, nv_e, mean_e, iv_e = orc.batchnorm_train_forward(x, gamma, beta, em, ev, eps, mu)
    assert st == 0
    res, nm, nv, mean, iv = batchNorm2DTrainForward(D(ctx, x), D(ctx, gamma), D(ctx, beta), D(ctx, em), D(ctx, ev), eps, mu, ctx)
    # the oracle's float statistics are sequential float sums; compare against them norm-wise and, for the statistics,
    # also against double-precision numpy (the device sums in double)
    xc = x.astype(np.float64).reshape(N, C, H * W).transpose(1, 0, 2).reshape(C, -1)
    m64, v64 = xc.mean(axis=1, keepdims=True), xc.var(axis=1, keepdims=True)
    tol = 1e-4 if dt == np.float32 else 1e-10
    np.testing.assert_allclose(mean.to_numpy(), m64, rtol=tol, atol=tol)
    np.testing.assert_allclose(iv.to_numpy(), 1 / np.sqrt(v64 + eps), rtol=tol)
    np.testing.assert_allclose(nm.to_numpy(), (1 - mu) * em + mu * m64, rtol=tol, atol=tol)
    np.testing.assert_allclose(nv.to_numpy(), (1 - mu) * ev + mu * v64, rtol=tol, atol=tol)
    if N * H * W > 1:
        assert_close(res.to_numpy(), res_e, rtol=(2e-4 if dt == np.float32 else 1e-9), elementwise=False)
        assert_close(mean.to_numpy(), mean_e, rtol=tol, elementwise=False)
        assert_close(iv.to_numpy(), iv_e, rtol=tol, elementwise=False)

    dout = rng.standard_normal(x.shape).astype(dt)
    st, dX_e, dG_e, dB_e = orc.batchnorm_backward(mean_e, iv_e, x, dout, gamma)
    assert st == 0
    dX, dG, dB = batchNorm2DBackward(D(ctx, mean_e), D(ctx, iv_e), D(ctx, x), D(ctx, dout), D(ctx, gamma), eps, ctx)
    btol = 5e-4 if dt == np.float32 else 1e-9
    assert_close(dB.to_numpy(), dB_e, rtol=btol, elementwise=False)
    assert_close(dG.to_numpy(), dG_e, rtol=btol, elementwise=False)
    assert_close(dX.to_numpy(), dX_e, rtol=btol, elementwise=False)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("p", [(2, 3, 3, 3, 2, 2, 2, 2, 1, 1), (4, 6, 28, 28, 2, 2, 2, 2, 0, 0), (3, 2, 14, 14, 3, 3, 2, 2, 1, 1),
                               (2, 2, 9, 7, 3, 2, 1, 1, 1, 0), (1, 1, 5, 5, 5, 5, 1, 1, 0, 0), (2, 3, 8, 8, 2, 2, 1, 1, 0, 0),
                               (5, 4, 12, 12, 4, 4, 3, 3, 2, 2), (3, 5, 14, 14, 2, 2, 2, 2, 0, 0), (2, 2, 7, 8, 2, 2, 2, 2, 0, 0),
                               (64, 16, 14, 16, 2, 2, 2, 2, 0, 0), (2, 3, 2, 2, 2, 2, 2, 2, 0, 0), (1, 1, 2, 6, 2, 2, 2, 2, 0, 0),
                               (3, 2, 6, 10, 2, 2, 2, 2, 0, 0), (130, 64, 14, 14, 2, 2, 2, 2, 0, 0)])
def test_pooling_backward(ctx, dt, p):
    N, C, H, W, ph, pw, sh, sw, padh, padw = p
    rng = np.random.default_rng(sum(p))
    x = rng.standard_normal((N, C * H * W)).astype(dt)
    x.reshape(-1)[::7] = x.reshape(-1)[3]  # ties inside windows: the first maximum wins
    P, Q = (H + 2 * padh - ph) // sw + 1, (W + 2 * padw - pw) // sh + 1
    dout = rng.standard_normal((N, C * P * Q)).astype(dt)
    for name, f in (("max", maxPoolBackward), ("avg", avgPoolBackward)):
        st, exp = getattr(orc, f"{name}pool_backward")(x, dout, *p)
        assert st == 0
        got = f(None, D(ctx, x), D(ctx, dout), *p, ctx).to_numpy()
        assert_exact(got, exp)  # same additions in the same order


def test_pooling_backward_all_negative_window_goes_to_the_padding(ctx):
    # with zero padding a window of negative values has its maximum on the border: that gradient is dropped
    x = -np.ones((1, 9), np.float32)
    dout = np.ones((1, 4), np.float32)
    p = (1, 1, 3, 3, 2, 2, 2, 2, 1, 1)
    st, exp = orc.maxpool_backward(x, dout, *p)
    got = maxPoolBackward(None, D(ctx, x), D(ctx, dout), *p, ctx).to_numpy()
    assert_exact(got, exp)
    assert got.sum() < dout.sum()


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", [(1, 3, 3, 3, 2, 2, 2, 2, 2, 1, 1), (4, 3, 12, 12, 5, 3, 3, 1, 1, 1, 1), (2, 2, 9, 8, 3, 2, 3, 2, 1, 0, 1),
                                  (3, 1, 5, 5, 2, 5, 5, 1, 1, 2, 2), (2, 4, 14, 14, 6, 5, 5, 1, 1, 2, 2), (2, 2, 8, 8, 2, 3, 2, 2, 3, 1, 0),
                                  (16, 8, 7, 7, 4, 7, 7, 1, 1, 3, 3),
                                  # large enough for the matrix-core paths (frame + forward convolution, patch matrix + GEMM)
                                  (64, 8, 12, 12, 6, 3, 3, 1, 1, 1, 1), (64, 4, 16, 16, 8, 5, 5, 2, 2, 2, 2),
                                  (48, 6, 15, 13, 5, 3, 2, 1, 2, 0, 1), (40, 3, 28, 28, 7, 5, 5, 1, 1, 2, 2),
                                  (96, 5, 12, 12, 3, 2, 2, 3, 3, 1, 1),
                                  # stride 1 (data gradient = forward convolution of dY with its own padding): no padding in the
                                  # forward direction is the widest one here; uneven filter and padding
                                  (30, 4, 24, 24, 5, 5, 5, 1, 1, 0, 0), (64, 8, 12, 13, 6, 3, 2, 1, 1, 0, 1), (33, 8, 10, 10, 16, 4, 4, 1, 1, 3, 3),
                                  # filter gradient with the image resident in LDS: two column chunks of 13 blocks a wave;
                                  # 20 filters (two filter blocks, 4 column parts); 70 filters (two groups) with stride 2;
                                  # 8 filters (one filter block, 8 column parts)
                                  (24, 32, 14, 14, 64, 5, 5, 1, 1, 2, 2), (32, 16, 12, 12, 20, 3, 3, 1, 1, 1, 1),
                                  (20, 24, 31, 31, 70, 3, 3, 2, 2, 1, 1), (17, 48, 16, 16, 8, 3, 3, 1, 1, 1, 1),
                                  # more images than workgroups: the next image is brought into the second LDS frame
                                  # beside the contraction (two channels per pixel block), some workgroups take two images
                                  (300, 10, 12, 12, 64, 5, 5, 1, 1, 2, 2)])
def test_conv_backward(ctx, dt, case):
    N, C, H, W, F, Hf, Wf, sh, sw, ph, pw = case
    rng = np.random.default_rng(sum(case))
    x = rng.standard_normal((N, C * H * W)).astype(dt)
    w = rng.standard_normal((F, C * Hf * Wf)).astype(dt)
    P, Q = (H + 2 * ph - Hf) // sh + 1, (W + 2 * pw - Wf) // sw + 1
    dy = rng.standard_normal((N, F * P * Q)).astype(dt)
    st, dx_e = orc.conv2d_backward_data(w, dy, *case)
    assert st == 0
    dx = conv2DBackwardData(D(ctx, w), D(ctx, dy), sh, sw, ph, pw, N, C, H, W, F, C, Hf, Wf, None, ctx).to_numpy()
    assert_close(dx, dx_e, elementwise=False)
    st, dw_e = orc.conv2d_backward_filter(x, dy, *case)
    assert st == 0
    dw = conv2DBackwardFilter(None, D(ctx, x), D(ctx, dy), sh, sw, ph, pw, N, C, H, W, F, C, Hf, Wf, ctx).to_numpy()
    assert_close(dw, dw_e, elementwise=False)
    # adjoint identities against the device's own forward convolution
    if dt == np.float64:
        y = conv2dForward(None, D(ctx, x), D(ctx, w), D(ctx, np.zeros((F, 1), dt)), N, C, H, W, Hf, Wf, sh, sw, ph, pw, ctx)
        y = (y[0] if isinstance(y, tuple) else y).to_numpy()
        lhs = float((y * dy).sum())
        assert abs(lhs - float((x * dx).sum())) <= 1e-9 * max(1.0, abs(lhs))
        assert abs(lhs - float((w * dw).sum())) <= 1e-9 * max(1.0, abs(lhs))


def test_training_kernels_reject_bad_shapes(ctx):
    x = D(ctx, np.ones((2, 10), np.float32))
    g = D(ctx, np.ones((3, 1), np.float32))
    with pytest.raises(capi.DaphneHipInvalidArgument):
        batchNorm2DTrainForward(x, g, g, g, g, 1e-5, 0.1, ctx)  # 10 columns, 3 channels
    with pytest.raises(capi.DaphneHipInvalidArgument):
        maxPoolBackward(None, x, x, 2, 1, 2, 5, 3, 3, 1, 1, 0, 0, ctx)  # window taller than the image
    with pytest.raises(capi.DaphneHipInvalidArgument):
        conv2DBackwardData(g, x, 1, 1, 0, 0, 2, 1, 2, 5, 1, 1, 3, 3, None, ctx)
