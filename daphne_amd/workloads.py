"""The benchmark workloads, composed from the device kernels the way the reference's scripts
compose its operators (scripts/algorithms/lmDS_.daph:60-75, test/api/cli/algorithms/kmeans.daphne:13-21,
scripts/examples/dnn-conv2d.daph). Host code only sequences kernel calls; all data stays on the device.
"""
from __future__ import annotations

import numpy as np

from .kernels import (AggOpCode, BinaryOpCode, DenseMatrix, HIPContext, UnaryOpCode, affineForward, affineForwardFused, aggCol,
                      aggRow, conv2dForward, conv2dForwardFused, kmeansAssign, kmeansStep, kmeansUpdate, ewBinaryMat, ewBinaryObjSca, ewUnaryMat, matMul, maxPoolForward, normalEquations, softmax, solve,
                      syrk)
from .pipeline import ROWREG, SELF, VectorizedPipeline


# ------------------------------------------------------------------------------------------------
# config 1: linear regression by normal equations (lmDS)
# ------------------------------------------------------------------------------------------------
def lmds(ctx: HIPContext, X: DenseMatrix, y: DenseMatrix, reg: float, eye: DenseMatrix | None = None, fused: bool = True):
    """A = t(X) @ X + reg * I ; b = t(X) @ y ; solve(A, b). Returns (A, b, w).
    fused: the normal equations from one pass over X (dh_normal_equations_*); otherwise operator by operator as
    lmDS_.daph writes them, with `eye` as the identity (the script builds diagMatrix(lambda))."""
    if fused:
        A, b = normalEquations(X, y, reg, ctx)
    else:
        A = syrk(None, X, True, ctx)
        lam = ewBinaryObjSca(BinaryOpCode.MUL, None, eye, reg, ctx)
        ewBinaryMat(BinaryOpCode.ADD, A, A, lam, ctx)  # in place, res aliases lhs
        b = matMul(None, X, y, True, False, ctx)
    w = solve(None, A, b, ctx)
    return A, b, w


# ------------------------------------------------------------------------------------------------
# config 2: z-score, row sums, threshold count
# ------------------------------------------------------------------------------------------------
def zscore_count(ctx: HIPContext, X: DenseMatrix, thr: float):
    """mu = colMeans(X); sd = sqrt(colVars(X)); r = rowSums(((X - mu) / sd)^2); s = sum(r > thr)."""
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


# ------------------------------------------------------------------------------------------------
# config 3: k-means (Lloyd) iteration
# ------------------------------------------------------------------------------------------------
class KMeans:
    """D = rowSums(X^2) - 2 X C^T + rowSums(C^2)^T ; idx = idxminRow(D) ; P = one-hot(idx) ;
    C' = (P^T X) / colSums(P)^T. The X-only term is hoisted out of the loop; the distance assembly,
    the arg-min and the one-hot matrix are one fused pipeline over X C^T."""

    def __init__(self, ctx: HIPContext, X: DenseMatrix, k: int):
        self.ctx, self.X, self.k = ctx, X, k
        dt = X.dtype
        p = VectorizedPipeline(ctx, X)
        p.ewBinary(BinaryOpCode.MUL, SELF).rowAgg(AggOpCode.SUM)
        self.xx = p.storeRow()
        p.run()
        self.seq = DenseMatrix.from_numpy(ctx, np.arange(k, dtype=dt).reshape(1, k))
        self.XC = DenseMatrix(ctx, X.rows, k, dt)
        self.P = DenseMatrix(ctx, X.rows, k, dt)
        self.idx = DenseMatrix(ctx, X.rows, 1, np.uint64)
        self.cc = DenseMatrix(ctx, k, 1, dt)
        self.PtX = DenseMatrix(ctx, k, X.cols, dt)
        self.counts = DenseMatrix(ctx, 1, k, dt)

    def iterate(self, C: DenseMatrix, C_out: DenseMatrix | None = None, fused=True) -> DenseMatrix:
        """fused True: kmeansStep (one pass over X for up to 64 features, two elsewhere); "two_passes":
        kmeansAssign then kmeansUpdate; False: one kernel per operator (or fused pipeline of elementwise operators), with
        XC, the one-hot P and t(P) X in memory. self.idx holds the assignment either way."""
        ctx, X, k = self.ctx, self.X, self.k
        pc = VectorizedPipeline(ctx, C)
        pc.ewBinary(BinaryOpCode.MUL, SELF).rowAgg(AggOpCode.SUM)
        pc.storeRow(self.cc)
        pc.run()                                                       # rowSums(C^2), k x 1
        if fused == "two_passes":
            kmeansAssign(self.idx, X, C, self.xx, self.cc, ctx)
            return kmeansUpdate(C_out, X, self.idx, k, ctx, self.counts)[0]
        if fused:
            return kmeansStep(self.idx, C_out, X, C, self.xx, self.cc, ctx, self.counts)[1]
        matMul(self.XC, X, C, False, True, ctx)                       # X @ t(C)
        cc_row = DenseMatrix(ctx, 1, k, C.dtype, ptr=self.cc.ptr, keepalive=self.cc)  # the same k values as 1 x k
        p = VectorizedPipeline(ctx, self.XC)
        p.ewBinary(BinaryOpCode.MUL, -2.0).ewBinary(BinaryOpCode.ADD, self.xx).ewBinary(BinaryOpCode.ADD, cc_row)
        p.rowAgg(AggOpCode.IDXMIN)
        p.storeRow(self.idx, as_index=True)
        # one-hot: overwrite the tile with the column numbers (isnan() makes every value finite, so that
        # the multiplication by zero really gives zero), then compare with the row's arg-min
        p.toTile().ewUnary(UnaryOpCode.ISNAN).ewBinary(BinaryOpCode.MUL, 0.0).ewBinary(BinaryOpCode.ADD, self.seq)
        p.ewBinary(BinaryOpCode.EQ, ROWREG)
        p.storeTile(self.P)
        p.run()
        matMul(self.PtX, self.P, X, True, False, ctx)                  # t(P) @ X, k x f
        aggCol(AggOpCode.SUM, self.counts, self.P, ctx)                # colSums(P), 1 x k
        counts_col = DenseMatrix(ctx, k, 1, C.dtype, ptr=self.counts.ptr, keepalive=self.counts)
        return ewBinaryMat(BinaryOpCode.DIV, C_out, self.PtX, counts_col, ctx)


# ------------------------------------------------------------------------------------------------
# config 5: LeNet-style CNN inference
# ------------------------------------------------------------------------------------------------
def lenet_forward(ctx: HIPContext, x: DenseMatrix, W: dict, batch: int, timer=None, fused=True):
    """conv 5x5x32 pad 2 + bias -> ReLU -> maxpool 2x2 -> conv 5x5x64 pad 2 + bias -> ReLU -> maxpool 2x2 ->
    affine 3136->512 -> ReLU -> affine 512->10 -> softmax. W: w1 (32 x 25), b1 (32 x 1), w2 (64 x 800),
    b2 (64 x 1), w3 (3136 x 512), b3 (1 x 512), w4 (512 x 10), b4 (1 x 10). fused: each layer's ReLU (and pooling)
    in the epilogue of the kernel before it, same numbers bit for bit; else one kernel per operator, ReLU as
    ewBinaryObjSca(MAX, x, 0) in place. `timer(name)` is called after each layer if given."""
    t = timer or (lambda name: None)
    if fused:
        h, _, _ = conv2dForwardFused(None, x, W["w1"], W["b1"], batch, 1, 28, 28, 5, 5, 1, 1, 2, 2, ctx, relu=True, pool=True)
        t("conv1+bias+relu+pool")
        h, _, _ = conv2dForwardFused(None, h, W["w2"], W["b2"], batch, 32, 14, 14, 5, 5, 1, 1, 2, 2, ctx, relu=True, pool=True)
        t("conv2+bias+relu+pool")
        h = affineForwardFused(None, h, W["w3"], W["b3"], ctx)
        t("affine1+relu")
        h = affineForward(None, h, W["w4"], W["b4"], ctx)
        t("affine2")
        out = softmax(None, h, ctx)
        t("softmax")
        return out
    t = timer or (lambda name: None)
    h, _, _ = conv2dForward(None, x, W["w1"], W["b1"], batch, 1, 28, 28, 5, 5, 1, 1, 2, 2, ctx)
    t("conv1+bias")
    ewBinaryObjSca(BinaryOpCode.MAX, h, h, 0.0, ctx)
    t("relu1")
    h, _, _ = maxPoolForward(None, h, batch, 32, 28, 28, 2, 2, 2, 2, 0, 0, ctx)
    t("pool1")
    h, _, _ = conv2dForward(None, h, W["w2"], W["b2"], batch, 32, 14, 14, 5, 5, 1, 1, 2, 2, ctx)
    t("conv2+bias")
    ewBinaryObjSca(BinaryOpCode.MAX, h, h, 0.0, ctx)
    t("relu2")
    h, _, _ = maxPoolForward(None, h, batch, 64, 14, 14, 2, 2, 2, 2, 0, 0, ctx)
    t("pool2")
    h = affineForward(None, h, W["w3"], W["b3"], ctx)
    t("affine1")
    ewBinaryObjSca(BinaryOpCode.MAX, h, h, 0.0, ctx)
    t("relu3")
    h = affineForward(None, h, W["w4"], W["b4"], ctx)
    t("affine2")
    out = softmax(None, h, ctx)
    t("softmax")
    return out
