#!/usr/bin/env python3
"""Per-kernel throughput table on one MI355X: every device kernel of the library at a large shape, float and double,
against the roofline that bounds it (HBM 8 TB/s for the streaming kernels, the dtype's MFMA peak for contractions).

    python bench_kernels.py [--reps 20] [--dtype f32|f64|both] [--only group|substring]

One JSON line per measurement: {"kernel", "dtype", "shape", "us", "achieved", "unit", "peak", "frac"}. Bytes are the
algorithmic ones (distinct inputs and outputs once each), flops 2mnk / n(n+1)k / 2 N F P Q C Hf Wf. Timing: device
events around `reps` back-to-back launches on the context's stream after one warm-up launch; inputs are generated on
the device. bench.py carries the headline pipeline; this file is the evidence for the single kernels.
"""
from __future__ import annotations

import argparse
import time
import json
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM = 8000.0
MFMA = {"f32": 157.3, "f64": 78.6}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--dtype", default="both", choices=["f32", "f64", "both"])
    ap.add_argument("--only", default="")
    args = ap.parse_args()

    import numpy as np
    import torch

    from daphne_amd import kernels as K
    from daphne_amd.kernels import AggOpCode as A, BinaryOpCode as B, DenseMatrix as DM, UnaryOpCode as U
    from daphne_amd.pipeline import SELF, VectorizedPipeline

    if not torch.cuda.is_available():
        print("bench_kernels.py: no GPU visible", file=sys.stderr)
        return 1
    ctx = K.HIPContext(0)
    gen = torch.Generator(device="cuda").manual_seed(7)

    def timed(fn):
        # untimed calls for 30 ms first: the clocks follow what ran before (a convolution timed right after a run of
        # memory-bound kernels took 850 us instead of 780)
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        while time.perf_counter() - t0 < 0.03:
            for _ in range(4):
                fn()
            torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(args.reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / args.reps * 1e3  # microseconds

    def emit(kernel, dt, shape, us, nbytes=None, flops=None):
        if args.only and args.only not in groups and args.only not in kernel:
            return
        if flops is None:
            ach, unit, peak = nbytes / us / 1e3, "GB/s", HBM
        else:
            ach, unit, peak = flops / us / 1e6, "TFLOP/s", MFMA[dt]
        print(json.dumps({"kernel": kernel, "dtype": dt, "shape": shape, "us": round(us, 1), "achieved": round(ach, 1),
                          "unit": unit, "peak": peak, "frac": round(ach / peak, 3)}), flush=True)

    groups = ("ew", "agg", "pipeline", "reorg", "tall", "gemm", "dnn", "train", "solve")

    def want(group):
        # --only takes a group name (runs that group) or a substring of a kernel name (runs all, prints the matches)
        return not args.only or args.only == group or args.only not in groups

    for dt in (["f32", "f64"] if args.dtype == "both" else [args.dtype]):
        tdt, ndt, sz = (torch.float32, np.float32, 4) if dt == "f32" else (torch.float64, np.float64, 8)
        rows, cols = (20_000_000, 64) if dt == "f32" else (10_000_000, 64)
        nb = rows * cols * sz
        shape = f"{rows}x{cols}"
        X = DM.from_torch(ctx, torch.randn(rows, cols, device="cuda", dtype=tdt, generator=gen) * 2 + 5)
        R = DM(ctx, rows, cols, ndt)
        rowv = DM.from_torch(ctx, torch.rand(1, cols, device="cuda", dtype=tdt, generator=gen) + 1)
        colv = DM.from_torch(ctx, torch.rand(rows, 1, device="cuda", dtype=tdt, generator=gen) + 1)
        r1 = DM(ctx, rows, 1, ndt)
        ri = DM(ctx, rows, 1, np.uint64)
        c1 = DM(ctx, 1, cols, ndt)

        # --- elementwise ---------------------------------------------------------------------------------------
        if want("ew"):
            emit("ewBinaryMat SUB row-vector", dt, shape, timed(lambda: K.ewBinaryMat(B.SUB, R, X, rowv, ctx)), 2 * nb)
            emit("ewBinaryMat DIV column-vector", dt, shape, timed(lambda: K.ewBinaryMat(B.DIV, R, X, colv, ctx)), 2 * nb + rows * sz)
            emit("ewBinaryMat MUL same shape", dt, shape, timed(lambda: K.ewBinaryMat(B.MUL, R, X, X, ctx)), 2 * nb)
            emit("ewBinaryMat ADD two inputs", dt, shape, timed(lambda: K.ewBinaryMat(B.ADD, R, X, R, ctx)), 3 * nb)
            emit("ewBinaryObjSca GT", dt, shape, timed(lambda: K.ewBinaryObjSca(B.GT, R, X, 5.0, ctx)), 2 * nb)
            K.ewUnaryMat(U.ABS, R, X, ctx)
            emit("ewUnaryMat SQRT in place (domain-checked)", dt, shape, timed(lambda: K.ewUnaryMat(U.SQRT, R, R, ctx)), 2 * nb)
            emit("ewUnaryMat EXP on a column", dt, f"{rows}x1", timed(lambda: K.ewUnaryMat(U.EXP, r1, colv, ctx)), 2 * rows * sz)
            emit("reluForward in place", dt, shape, timed(lambda: K.reluForward(R, R, ctx)), 2 * nb)
        # --- aggregations --------------------------------------------------------------------------------------
        if want("agg"):
            emit("aggAll SUM", dt, shape, timed(lambda: K.aggAll(A.SUM, X, ctx)), nb)
            emit("aggAll VAR (two passes)", dt, shape, timed(lambda: K.aggAll(A.VAR, X, ctx)), 2 * nb)
            emit("aggRow SUM", dt, shape, timed(lambda: K.aggRow(A.SUM, r1, X, ctx)), nb + rows * sz)
            emit("aggRow MAX", dt, shape, timed(lambda: K.aggRow(A.MAX, r1, X, ctx)), nb + rows * sz)
            emit("aggRow VAR (two passes over the row)", dt, shape, timed(lambda: K.aggRow(A.VAR, r1, X, ctx)), nb + rows * sz)
            emit("aggRow IDXMIN", dt, shape, timed(lambda: K.aggRow(A.IDXMIN, ri, X, ctx)), nb + rows * 8)
            emit("aggCol SUM", dt, shape, timed(lambda: K.aggCol(A.SUM, c1, X, ctx)), nb)
            emit("aggCol MAX", dt, shape, timed(lambda: K.aggCol(A.MAX, c1, X, ctx)), nb)
            emit("aggCol VAR (one pass)", dt, shape, timed(lambda: K.aggCol(A.VAR, c1, X, ctx)), nb)
            emit("aggColMoments mean+var (one pass)", dt, shape, timed(lambda: K.aggColMoments(X, ctx, res_mean=c1, res_var=rowv)), nb)
            ci = DM(ctx, 1, cols, np.uint64)
            emit("aggCol IDXMAX", dt, shape, timed(lambda: K.aggCol(A.IDXMAX, ci, X, ctx)), nb)
            rowv = DM.from_torch(ctx, torch.rand(1, cols, device="cuda", dtype=tdt, generator=gen) + 1)
        # --- fused pipeline ------------------------------------------------------------------------------------
        if want("pipeline"):
            p = VectorizedPipeline(ctx, X)
            p.ewBinary(B.SUB, c1).ewBinary(B.DIV, rowv).ewBinary(B.MUL, SELF).rowAgg(A.SUM)
            p.storeRow(r1)
            p.ewBinary(B.GT, float(cols))
            p.reduceAll(A.SUM)
            emit("VectorizedPipeline z-score/rowSums/count", dt, shape, timed(p.run), nb + rows * sz)
        # --- data reorganisation -------------------------------------------------------------------------------
        if want("reorg"):
            emit("fill", dt, shape, timed(lambda: K.fill(R, 2.5, rows, cols, ctx)), nb)
            T = DM(ctx, cols, rows, ndt)
            emit("transpose", dt, shape, timed(lambda: K.transpose(T, X, ctx)), 2 * nb)
            T.destroy()
            L = DM.from_torch(ctx, torch.randn(rows, 16, device="cuda", dtype=tdt, generator=gen))
            CB = DM(ctx, rows, cols + 16, ndt)
            emit("colBind 64|16 columns", dt, shape, timed(lambda: K.colBind(CB, X, L, ctx)), 2 * (nb + rows * 16 * sz))
            CB.destroy()
            sel = DM.from_numpy(ctx, np.array([63, 0, 17, 5, 9, 33, 2, 41], dtype=np.int64).reshape(-1, 1))
            E = DM(ctx, rows, 8, ndt)
            t_ext = timed(lambda: K.extractCol(E, X, sel, ctx))
            # two byte conventions for the same launches: what the memory system has to move (every 64-byte segment of
            # a row holds a selected column, so whole rows), and the selected values alone (read once, written once)
            emit("extractCol 8 of 64 columns (sector traffic: whole rows)", dt, shape, t_ext, nb + rows * 8 * sz)
            emit("extractCol 8 of 64 columns (selected values only: 2 x rows x 8)", dt, shape, t_ext, 2 * rows * 8 * sz)
            E.destroy()
            L.destroy()
        # --- tall-and-skinny contractions ----------------------------------------------------------------------
        if want("tall"):
            y = colv
            gv = DM(ctx, cols, 1, ndt)
            emit("tall gemv t(X) y", dt, shape, timed(lambda: K.gemv(gv, X, y, ctx)), nb + rows * sz)
            S = DM(ctx, cols, cols, ndt)
            emit("tall syrk t(X) X", dt, shape, timed(lambda: K.syrk(S, X, True, ctx)), nb)
            Cc = DM.from_torch(ctx, torch.randn(16, cols, device="cuda", dtype=tdt, generator=gen))
            XC = DM(ctx, rows, 16, ndt)
            emit("tall matMul X t(C), C 16x64", dt, shape, timed(lambda: K.matMul(XC, X, Cc, False, True, ctx)), nb + rows * 16 * sz)
            PtX = DM(ctx, 16, cols, ndt)
            emit("tall matMul t(P) X, P rows x 16", dt, shape, timed(lambda: K.matMul(PtX, XC, X, True, False, ctx)), nb + rows * 16 * sz)
            XC.destroy()
            # the k-means passes: X once each, no rows x 16 matrix in memory
            xxv = DM.from_torch(ctx, torch.rand(rows, 1, device="cuda", dtype=tdt, generator=gen))
            ccv = DM.from_torch(ctx, torch.rand(16, 1, device="cuda", dtype=tdt, generator=gen))
            idxv = DM(ctx, rows, 1, np.uint64)
            emit("kmeansAssign (X t(C), distances, row arg-min), C 16x64", dt, shape, timed(lambda: K.kmeansAssign(idxv, X, Cc, xxv, ccv, ctx)),
                 nb + rows * sz + rows * 8)
            cnts = DM(ctx, 1, 16, ndt)
            emit("kmeansUpdate (t(one-hot(idx)) X / sizes), 16 centroids", dt, shape, timed(lambda: K.kmeansUpdate(PtX, X, idxv, 16, ctx, cnts)),
                 nb + rows * 8)
            emit("kmeansStep (assignment and update from one pass over X), C 16x64", dt, shape,
                 timed(lambda: K.kmeansStep(idxv, PtX, X, Cc, xxv, ccv, ctx, cnts)), nb + rows * sz + rows * 8)
            for m_ in (xxv, ccv, idxv, cnts):
                m_.destroy()
        for m in (X, R, colv, r1, ri):
            m.destroy()
        ctx.releaseCached()
        torch.cuda.empty_cache()

        # --- square contractions (shorter than the headline shapes of bench.py --config 4) -------------------------
        if want("gemm"):
            n = 8192 if dt == "f32" else 4096
            Am = DM.from_torch(ctx, torch.rand(n, n, device="cuda", dtype=tdt, generator=gen) - 0.5)
            Bm = DM.from_torch(ctx, torch.rand(n, n, device="cuda", dtype=tdt, generator=gen) - 0.5)
            Cm = DM(ctx, n, n, ndt)
            for ta, tb in ((False, False), (False, True), (True, False), (True, True)):
                emit(f"matMul {'T' if ta else 'N'}{'T' if tb else 'N'}", dt, f"{n}^3", timed(lambda: K.matMul(Cm, Am, Bm, ta, tb, ctx)),
                     flops=2.0 * n ** 3)
            emit("syrk t(X) X", dt, f"{n}x{n}", timed(lambda: K.syrk(Cm, Am, True, ctx)), flops=float(n) * (n + 1) * n)
            emit("syrk X t(X)", dt, f"{n}x{n}", timed(lambda: K.syrk(Cm, Am, False, ctx)), flops=float(n) * (n + 1) * n)
            for m in (Am, Bm, Cm):
                m.destroy()
        # --- DNN ---------------------------------------------------------------------------------------------
        if want("dnn"):
            N = 4096 if dt == "f32" else 2048
            x2 = DM.from_torch(ctx, torch.rand(N, 32 * 14 * 14, device="cuda", dtype=tdt, generator=gen))
            w2 = DM.from_torch(ctx, torch.randn(64, 800, device="cuda", dtype=tdt, generator=gen) * 0.05)
            b2 = DM.from_torch(ctx, torch.randn(64, 1, device="cuda", dtype=tdt, generator=gen) * 0.1)
            o2 = DM(ctx, N, 64 * 196, ndt)
            emit("conv2dForward 32->64 ch, 14x14, 5x5 pad 2 (image resident in LDS)", dt, f"batch {N}",
                 timed(lambda: K.conv2dForward(o2, x2, w2, b2, N, 32, 14, 14, 5, 5, 1, 1, 2, 2, ctx)), flops=2.0 * N * 64 * 196 * 800)
            emit("biasAdd 64 channels", dt, f"{N}x{64 * 196}", timed(lambda: K.biasAdd(o2, o2, b2, ctx)), 2 * N * 64 * 196 * sz)
            one = DM.from_torch(ctx, torch.ones(64, 1, device="cuda", dtype=tdt))
            emit("batchNormInferenceForward 64 channels", dt, f"{N}x{64 * 196}",
                 timed(lambda: K.batchNormInferenceForward(o2, o2, one, b2, b2, one, 1e-5, ctx)), 2 * N * 64 * 196 * sz)
            pl = DM(ctx, N, 64 * 49, ndt)
            emit("conv2dForwardFused 32->64 ch, 14x14, 5x5 pad 2, ReLU + maxPool 2x2 in the epilogue", dt, f"batch {N}",
                 timed(lambda: K.conv2dForwardFused(pl, x2, w2, b2, N, 32, 14, 14, 5, 5, 1, 1, 2, 2, ctx, relu=True, pool=True)),
                 flops=2.0 * N * 64 * 196 * 800)
            x1 = DM.from_torch(ctx, torch.rand(N, 784, device="cuda", dtype=tdt, generator=gen))
            w1 = DM.from_torch(ctx, torch.randn(32, 25, device="cuda", dtype=tdt, generator=gen) * 0.2)
            b1 = DM.from_torch(ctx, torch.randn(32, 1, device="cuda", dtype=tdt, generator=gen) * 0.1)
            o1, p1 = DM(ctx, N, 32 * 784, ndt), DM(ctx, N, 32 * 196, ndt)
            emit("conv2dForward 1->32 ch, 28x28, 5x5 pad 2 (a thread per 2x2 quad of pixels)", dt, f"batch {N}",
                 timed(lambda: K.conv2dForward(o1, x1, w1, b1, N, 1, 28, 28, 5, 5, 1, 1, 2, 2, ctx)), flops=2.0 * N * 32 * 784 * 25)
            emit("conv2dForwardFused 1->32 ch, 28x28, 5x5 pad 2, ReLU + maxPool 2x2 in the epilogue", dt, f"batch {N}",
                 timed(lambda: K.conv2dForwardFused(p1, x1, w1, b1, N, 1, 28, 28, 5, 5, 1, 1, 2, 2, ctx, relu=True, pool=True)),
                 flops=2.0 * N * 32 * 784 * 25)
            for m_ in (x1, w1, b1, o1, p1):
                m_.destroy()
            emit("maxPoolForward 2x2/2 on 14x14", dt, f"{N}x{64 * 196}",
                 timed(lambda: K.maxPoolForward(pl, o2, N, 64, 14, 14, 2, 2, 2, 2, 0, 0, ctx)), 1.25 * N * 64 * 196 * sz)
            emit("avgPoolForward 2x2/2 on 14x14", dt, f"{N}x{64 * 196}",
                 timed(lambda: K.avgPoolForward(pl, o2, N, 64, 14, 14, 2, 2, 2, 2, 0, 0, ctx)), 1.25 * N * 64 * 196 * sz)
            emit("maxPoolForward 3x3/2 pad 1 on 14x14 (planes staged in LDS)", dt, f"{N}x{64 * 196}",
                 timed(lambda: K.maxPoolForward(None, o2, N, 64, 14, 14, 3, 3, 2, 2, 1, 1, ctx)),
                 (1 + 49.0 / 196) * N * 64 * 196 * sz)
            w3 = DM.from_torch(ctx, torch.randn(3136, 512, device="cuda", dtype=tdt, generator=gen) * 0.02)
            b3 = DM.from_torch(ctx, torch.randn(1, 512, device="cuda", dtype=tdt, generator=gen) * 0.1)
            h3 = DM(ctx, N, 512, ndt)
            emit("affineForward 3136 -> 512", dt, f"batch {N}", timed(lambda: K.affineForward(h3, pl, w3, b3, ctx)),
                 flops=2.0 * N * 3136 * 512)
            big = DM.from_torch(ctx, torch.randn(1_000_000, 10, device="cuda", dtype=tdt, generator=gen))
            sm = DM(ctx, 1_000_000, 10, ndt)
            emit("softmax 10 classes", dt, "1000000x10", timed(lambda: K.softmax(sm, big, ctx)), 2 * 10_000_000 * sz)
            for m in (big, sm):
                m.destroy()
            big = DM.from_torch(ctx, torch.randn(16_000_000, 10, device="cuda", dtype=tdt, generator=gen))
            sm = DM(ctx, 16_000_000, 10, ndt)
            emit("softmax 10 classes", dt, "16000000x10", timed(lambda: K.softmax(sm, big, ctx)), 2 * 160_000_000 * sz)
            for m in (x2, w2, b2, o2, one, pl, w3, b3, h3, big, sm):
                m.destroy()
        # --- DNN training kernels ---------------------------------------------------------------------------------
        if want("train"):
            N = 4096 if dt == "f32" else 2048
            el = N * 64 * 196
            x = DM.from_torch(ctx, torch.randn(N, 64 * 196, device="cuda", dtype=tdt, generator=gen))
            dy = DM.from_torch(ctx, torch.randn(N, 64 * 196, device="cuda", dtype=tdt, generator=gen))
            gam = DM.from_torch(ctx, torch.rand(64, 1, device="cuda", dtype=tdt, generator=gen) + 0.5)
            zer = DM.from_torch(ctx, torch.zeros(64, 1, device="cuda", dtype=tdt))
            res_bn = K.batchNorm2DTrainForward(x, gam, zer, zer, gam, 1e-5, 0.1, ctx)
            emit("batchNorm2DTrainForward 64 channels (statistics pass + normalisation pass)", dt, f"{N}x{64 * 196}",
                 timed(lambda: K.batchNorm2DTrainForward(x, gam, zer, zer, gam, 1e-5, 0.1, ctx)), 2 * el * sz)
            emit("batchNorm2DBackward 64 channels (sums pass + gradient pass)", dt, f"{N}x{64 * 196}",
                 timed(lambda: K.batchNorm2DBackward(res_bn[3], res_bn[4], x, dy, gam, 1e-5, ctx)), 3 * el * sz)
            # the same where a channel's values fit a workgroup's LDS: 32 images of 512 channels, 14 x 14
            ns, cs = 32, 512
            xs = DM.from_torch(ctx, torch.randn(ns, cs * 196, device="cuda", dtype=tdt, generator=gen))
            dys = DM.from_torch(ctx, torch.randn(ns, cs * 196, device="cuda", dtype=tdt, generator=gen))
            gs = DM.from_torch(ctx, torch.rand(cs, 1, device="cuda", dtype=tdt, generator=gen) + 0.5)
            zs = DM.from_torch(ctx, torch.zeros(cs, 1, device="cuda", dtype=tdt))
            rs = K.batchNorm2DTrainForward(xs, gs, zs, zs, gs, 1e-5, 0.1, ctx)
            emit("batchNorm2DTrainForward 512 channels, 14x14 (one read where a channel fits LDS)", dt, f"{ns}x{cs * 196}",
                 timed(lambda: K.batchNorm2DTrainForward(xs, gs, zs, zs, gs, 1e-5, 0.1, ctx)), 2 * ns * cs * 196 * sz)
            emit("batchNorm2DBackward 512 channels, 14x14 (one read where a channel and its gradient fit LDS)", dt, f"{ns}x{cs * 196}",
                 timed(lambda: K.batchNorm2DBackward(rs[3], rs[4], xs, dys, gs, 1e-5, ctx)), 3 * ns * cs * 196 * sz)
            for m_ in (xs, dys, gs, zs, *rs):
                m_.destroy()
            dpool = DM.from_torch(ctx, torch.randn(N, 64 * 49, device="cuda", dtype=tdt, generator=gen))
            dxp = DM(ctx, N, 64 * 196, ndt)
            emit("maxPoolBackward 2x2/2 on 14x14", dt, f"{N}x{64 * 196}",
                 timed(lambda: K.maxPoolBackward(dxp, x, dpool, N, 64, 14, 14, 2, 2, 2, 2, 0, 0, ctx)), 2.25 * el * sz)
            emit("avgPoolBackward 2x2/2 on 14x14", dt, f"{N}x{64 * 196}",
                 timed(lambda: K.avgPoolBackward(dxp, x, dpool, N, 64, 14, 14, 2, 2, 2, 2, 0, 0, ctx)), 1.25 * el * sz)
            Nc = N
            xc = DM.from_torch(ctx, torch.rand(Nc, 32 * 196, device="cuda", dtype=tdt, generator=gen))
            wc = DM.from_torch(ctx, torch.randn(64, 800, device="cuda", dtype=tdt, generator=gen) * 0.05)
            dyc = DM.from_torch(ctx, torch.randn(Nc, 64 * 196, device="cuda", dtype=tdt, generator=gen))
            dxc, dwc = DM(ctx, Nc, 32 * 196, ndt), DM(ctx, 64, 800, ndt)
            fl = 2.0 * Nc * 64 * 196 * 800
            emit("conv2DBackwardData 64->32 ch, 14x14, 5x5 pad 2 (rotated filters + forward convolution of the padded output gradient)", dt, f"batch {Nc}",
                 timed(lambda: K.conv2DBackwardData(wc, dyc, 1, 1, 2, 2, Nc, 32, 14, 14, 64, 32, 5, 5, dxc, ctx)), flops=fl)
            emit("conv2DBackwardFilter 32->64 ch, 14x14, 5x5 pad 2 (image resident in LDS, slabs per workgroup)", dt, f"batch {Nc}",
                 timed(lambda: K.conv2DBackwardFilter(dwc, xc, dyc, 1, 1, 2, 2, Nc, 32, 14, 14, 64, 32, 5, 5, ctx)), flops=fl)
            for m in (x, dy, gam, zer, dpool, dxp, xc, wc, dyc, dxc, dwc, *res_bn):
                m.destroy()
        # --- solve -------------------------------------------------------------------------------------------
        if want("solve"):
            n = 100
            As = DM.from_torch(ctx, torch.rand(n, n, device="cuda", dtype=tdt, generator=gen) + n * torch.eye(n, device="cuda", dtype=tdt))
            bs = DM.from_torch(ctx, torch.rand(n, 1, device="cuda", dtype=tdt, generator=gen))
            xs = DM(ctx, n, 1, ndt)
            us = timed(lambda: K.solve(xs, As, bs, ctx))
            if not args.only or args.only in ("solve",) or args.only in "solve 100x100":
                print(json.dumps({"kernel": "solve 100x100 (latency bound, incl. the singularity flag read-back)", "dtype": dt,
                                  "shape": "100x100", "us": round(us, 1)}), flush=True)
            # normal equations of a 100000 x 100 regression: t(X) X + lambda I and t(X) y from one pass over X
            Xn = DM.from_torch(ctx, torch.rand(100_000, n, device="cuda", dtype=tdt, generator=gen))
            yn = DM.from_torch(ctx, torch.rand(100_000, 1, device="cuda", dtype=tdt, generator=gen))
            An, bn = DM(ctx, n, n, ndt), DM(ctx, n, 1, ndt)
            emit("normalEquations (t(X) X + lambda I, t(X) y; upper tile pairs only)", dt, "100000x100",
                 timed(lambda: K.normalEquations(Xn, yn, 1e-3, ctx, An, bn)), 100_000 * (n + 1) * sz)
            for m_ in (Xn, yn, An, bn):
                m_.destroy()
        ctx.releaseCached()
        torch.cuda.empty_cache()
    ctx.destroy()
    return 0


if __name__ == "__main__":
    sys.exit(main())
