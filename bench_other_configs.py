"""Benchmark lines for BASELINE.json configurations 1, 3, 4 and 5 (`python bench.py --config N`).

Same conventions as bench.py: inputs resident in HBM before the timed region, K timed steps between
synchronisations, one JSON line. `value` is the configuration's own figure of merit (GB/s over canonical
algorithmic bytes for the HBM-bound ones, TFLOP/s for the contractions, images/s for the CNN), next to the
roofline fraction of the dominant kernel and a bounded CPU baseline from the oracle's restatement."""
from __future__ import annotations

import json
import os
import sys
import time

import numpy as np

HBM_PEAK_GBS = 8000.0
MFMA_PEAK = {"f32": 157.3, "f64": 78.6}


CLOCK_WARMUP_S = 0.25


def _timed(torch, fn, steps, warmup):
    """Wall time per step in ms over `steps` steps, after `warmup` untimed ones and as many more untimed ones as it takes
    to fill CLOCK_WARMUP_S: the device needs tens of milliseconds of continuous work to reach its clocks, which steps of
    0.1 ms do not give it in a few dozen repetitions (k-means: 0.26 ms per iteration over the first 50 ms, 0.115 after)."""
    t0 = time.perf_counter()
    done = 0
    while done < warmup or time.perf_counter() - t0 < CLOCK_WARMUP_S:
        fn()
        done += 1
        if done % 16 == 0:
            torch.cuda.synchronize()  # keeps the host no more than 16 steps ahead, so that the clock above means device work
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def _events(torch, fn, reps=30):
    """Average duration of one call of fn on the current stream, with device events (after ten untimed calls)."""
    for _ in range(10):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


def _line(metric_value, unit, ms, args, dtype, workload, roofline, cpu, extra=None):
    cfg = {"workload": workload}
    cfg.update(extra or {})
    return {"metric": "HBM GB/s (% peak) on fused ew+agg pipelines; MatMul/Syrk TFLOP/s (% MFMA peak)",
            "value": round(metric_value, 3), "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": dtype, "data": "synthetic", "config": cfg, "roofline": roofline, "cpu_baseline": cpu}


def measure_contractions(torch, ctx, steps, warmup):
    """The dense-contraction half of the metric at the sizes it is quoted on: MatMul f64 8192^3, MatMul f32 16384^3,
    Syrk f64 t(X) X with X 1,000,000 x 1024. Returns {name: {ms, tflops, pct_of_mfma_peak}}; inputs are generated
    on the device and freed again before the next case."""
    from daphne_amd.kernels import DenseMatrix, matMul, syrk

    gen = torch.Generator(device="cuda").manual_seed(4)
    res = {}
    for name, dt, n, key in (("matmul_f64_8192", torch.float64, 8192, "f64"), ("matmul_f32_16384", torch.float32, 16384, "f32")):
        A = torch.rand(n, n, device="cuda", dtype=dt, generator=gen) * 2 - 1
        B = torch.rand(n, n, device="cuda", dtype=dt, generator=gen) * 2 - 1
        Cm = torch.empty(n, n, device="cuda", dtype=dt)
        dA, dB, dC = (DenseMatrix.from_torch(ctx, t) for t in (A, B, Cm))
        ms = _timed(torch, lambda: matMul(dC, dA, dB, False, False, ctx), steps, warmup)
        res[name] = {"ms": round(ms, 3), "tflops": round(2.0 * n ** 3 / ms / 1e9, 2)}
        res[name]["pct_of_mfma_peak"] = round(100 * res[name]["tflops"] / MFMA_PEAK[key], 1)
        del A, B, Cm, dA, dB, dC
        torch.cuda.empty_cache()
    Xs = torch.rand(1_000_000, 1024, device="cuda", dtype=torch.float64, generator=gen) * 2 - 1
    dX, S = DenseMatrix.from_torch(ctx, Xs), DenseMatrix(ctx, 1024, 1024, np.float64)
    ms_s = _timed(torch, lambda: syrk(S, dX, True, ctx), steps, warmup)
    # the distinct results of t(X) X: n (n + 1) / 2 dot products of length 1e6
    res["syrk_f64_1e6x1024"] = {"ms": round(ms_s, 3), "tflops": round(1024 * 1025 * 1e6 / ms_s / 1e9, 2)}
    res["syrk_f64_1e6x1024"]["pct_of_mfma_peak"] = round(100 * res["syrk_f64_1e6x1024"]["tflops"] / MFMA_PEAK["f64"], 1)
    S.destroy()
    del Xs, dX
    torch.cuda.empty_cache()
    return res


def blas_baseline(n=4096, reps=3):
    """numpy.matmul in double precision on the host: numpy's bundled BLAS is OpenBLAS, the library the reference's
    CPU MatMul calls (src/runtime/local/kernels/MatMul.cpp:24-90, cblas_dgemm). Returns (TFLOP/s, description)."""
    import io
    from contextlib import redirect_stdout

    rng = np.random.default_rng(0)
    a, b = rng.random((n, n)), rng.random((n, n))
    a @ b
    best = float("inf")
    for _ in range(reps):
        t0 = time.perf_counter()
        a @ b
        best = min(best, time.perf_counter() - t0)
    buf = io.StringIO()
    try:
        with redirect_stdout(buf):
            np.show_config()
    except Exception:
        pass
    cfg = buf.getvalue()
    name = "openblas" if "openblas" in cfg.lower() else ("mkl" if "mkl" in cfg.lower() else "BLAS of numpy")
    threads = os.environ.get("OPENBLAS_NUM_THREADS") or os.environ.get("OMP_NUM_THREADS") or str(os.cpu_count())
    return 2.0 * n ** 3 / best / 1e12, f"numpy.matmul f64 {n}^3 ({name}, {threads} threads, best of {reps}: {best:.2f} s)"


def _blas_name():
    import io
    from contextlib import redirect_stdout
    buf = io.StringIO()
    try:
        with redirect_stdout(buf):
            np.show_config()
    except Exception:
        pass
    cfg = buf.getvalue().lower()
    return "OpenBLAS" if "openblas" in cfg else ("MKL" if "mkl" in cfg else "numpy's BLAS")


def _threaded(fn, pieces, threads):
    """fn over the pieces on a pool of host threads (the oracle's kernels and numpy's release the interpreter lock)."""
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(max_workers=threads) as pool:
        return list(pool.map(fn, pieces))


def run(args) -> int:
    import torch

    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests"))
    from daphne_amd.kernels import DenseMatrix, HIPContext, kmeansAssign, kmeansStep, kmeansUpdate, matMul, normalEquations, solve, syrk
    from daphne_amd.workloads import KMeans, lenet_forward, lmds

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    ctx = HIPContext(0)
    gen = torch.Generator(device="cuda").manual_seed(42)
    threads = min(os.cpu_count() or 1, 16)
    orc = None
    if not args.no_cpu:
        import oracle_binding as orc

    if args.config == 1:
        n, m = 100_000, 100
        Xt = torch.rand(n, m, device="cuda", dtype=torch.float64, generator=gen)
        w = torch.randn(m, 1, device="cuda", dtype=torch.float64, generator=gen)
        yt = Xt @ w + 0.1 * torch.randn(n, 1, device="cuda", dtype=torch.float64, generator=gen)
        X, y = DenseMatrix.from_torch(ctx, Xt), DenseMatrix.from_torch(ctx, yt)
        eye = DenseMatrix.from_numpy(ctx, np.eye(m))
        # Solve reports a singular factor to its caller (Solve.h:113-115 throws), so a direct call waits for the device.
        # The steps of the timed region are enqueued back to back like those of every other configuration: with the
        # verdicts deferred (dh_defer_checks) and collected once after the last step. The per-call form is timed beside it.
        ms_immediate = _timed(torch, lambda: lmds(ctx, X, y, 1e-3), args.steps, args.warmup)
        with ctx.deferred_checks():
            ms = _timed(torch, lambda: lmds(ctx, X, y, 1e-3), args.steps, args.warmup)
        # the step's two parts on their own: one pass over X for A and b, then the 100 x 100 solve
        A0, b0 = normalEquations(X, y, 1e-3, ctx)
        w0 = solve(None, A0, b0, ctx)
        t_ne = _events(torch, lambda: normalEquations(X, y, 1e-3, ctx, A0, b0))
        t_solve = _events(torch, lambda: solve(w0, A0, b0, ctx))
        nbytes = (n * m * 8 + m * m * 8) + (n * m * 8 + n * 8 + m * 8) + 3 * m * m * 8
        cpu = None
        if orc:
            # the libraries the reference's CPU kernels call (Syrk.h: cblas_dsyrk, MatMul.cpp: cblas_dgemv, Solve.h:
            # LAPACKE_dgesv) as numpy carries them, all host threads, the whole configuration; best of three
            Xh, yh = Xt.cpu().numpy(), yt.cpu().numpy()
            best = float("inf")
            for _ in range(3):
                t0 = time.perf_counter()
                A = Xh.T @ Xh + np.eye(m) * 1e-3
                b = Xh.T @ yh
                np.linalg.solve(A, b)
                best = min(best, time.perf_counter() - t0)
            t0 = time.perf_counter()
            A = orc.syrk(Xh, True)[1] + np.eye(m) * 1e-3
            b = orc.matmul(Xh, yh, True, False)[1]
            orc.solve(A, b)
            dt = time.perf_counter() - t0
            cpu = {"value": round(nbytes / best / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
                   "sample": f"the whole configuration with numpy's {_blas_name()} / LAPACK (dsyrk or dgemm, dgemv, dgesv), "
                             f"{threads} threads, best of 3 ({best * 1e3:.1f} ms); scalar loops on one thread: {dt:.2f} s = "
                             f"{nbytes / dt / 1e9:.3f} GB/s"}
        ne_bytes = n * m * 8 + n * 8 + m * m * 8 + m * 8
        roof = {"bound": "hbm", "kernel": "ts_sym_kernel<double> + ts_sym_reduce_kernel (t(X) X + lambda I and t(X) y, X read once)",
                "achieved": round(ne_bytes / t_ne / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(ne_bytes / t_ne / 1e6 / HBM_PEAK_GBS, 4), "traffic": None,
                "mfma_tflops": round((m * (m + 1) + 2 * m) * n / t_ne / 1e9, 1)}
        out = _line(nbytes / ms / 1e6, "GB/s", ms, args, "f64",
                    "lmDS normal equations: X 100000x100 f64; A = syrk(X) + 1e-3 I, b = t(X) y, solve (latency bound; steps enqueued "
                    "back to back, the solves' verdicts deferred and collected after the last step)",
                    roof, cpu, {"canonical_bytes_per_step": nbytes, "normal_equations_us": round(t_ne * 1e3, 1),
                                "solve_us": round(t_solve * 1e3, 1), "ms_per_step_verdict_per_call": round(ms_immediate, 4)})
    elif args.config == 3:
        n, f, k = 2_000_000, 64, 16
        centres = torch.randn(k, f, device="cuda", generator=gen) * 5
        Xt = centres[torch.arange(n, device="cuda") % k] + torch.randn(n, f, device="cuda", generator=gen)
        X = DenseMatrix.from_torch(ctx, Xt)
        km = KMeans(ctx, X, k)
        C0 = Xt[torch.arange(k, device="cuda") * 125000].contiguous()
        # two centroid buffers used in turn: a fresh result matrix per iteration would put an allocation and a
        # (synchronising) release between the kernels
        start = DenseMatrix.from_torch(ctx, C0)
        state = {"C": start, "next": 0, "done": 0}
        bufs = [DenseMatrix(ctx, k, f, np.float32), DenseMatrix(ctx, k, f, np.float32)]

        def step(fused=True):  # one Lloyd iteration; runs of ten from the seeded rows, as the configuration has them
            out = bufs[state["next"]]
            state["next"] ^= 1
            state["C"] = km.iterate(state["C"] if state["done"] % 10 else start, out, fused=fused)
            state["done"] += 1

        ms = _timed(torch, step, args.steps, args.warmup)
        t_step = _events(torch, lambda: kmeansStep(km.idx, bufs[state["next"]], X, state["C"], km.xx, km.cc, ctx, km.counts))
        ms_two = _timed(torch, lambda: step("two_passes"), args.steps, args.warmup)
        ms_seq = _timed(torch, lambda: step(False), min(args.steps, 15), args.warmup)
        t_assign = _events(torch, lambda: kmeansAssign(km.idx, X, state["C"], km.xx, km.cc, ctx))
        t_update = _events(torch, lambda: kmeansUpdate(bufs[state["next"]], X, km.idx, k, ctx, km.counts))
        # canonical bytes per iteration: X C^T (read X, write D), D assembly 3 x |D|, idxmin (read D, write idx),
        # one-hot P, P^T X (read P and X), colSums(P)
        D = n * k * 4
        nbytes = (n * f * 4 + D) + 3 * D + (D + n * 8) + D + (D + n * f * 4) + D
        t_gemm = _events(torch, lambda: matMul(km.XC, X, state["C"], False, True, ctx))
        cpu = None
        if orc:
            # one iteration at full size on all host threads: the products by numpy's BLAS (the reference's MatMul calls
            # cblas_sgemm), everything else by the scalar kernels of the port on row pieces, one piece per thread
            Xh = Xt.cpu().numpy()
            Ch = C0.cpu().numpy()
            pieces = [slice(a, min(a + (n + threads - 1) // threads, n)) for a in range(0, n, (n + threads - 1) // threads)]
            xx = np.concatenate(_threaded(lambda sl: orc.agg_row(0, orc.ew_binary(2, Xh[sl], Xh[sl])[1])[1], pieces, threads))

            def assign_piece(sl):
                XC = Xh[sl] @ Ch.T
                Dh = orc.ew_binary(0, orc.ew_binary(0, orc.ew_binary_sca(2, XC, -2.0)[1], xx[sl])[1], cc_row)[1]
                idx = orc.agg_row(4, Dh)[1]
                P = (idx == np.arange(k, dtype=np.uint64)[None, :]).astype(np.float32)
                return P.T @ Xh[sl], orc.agg_col(0, P)[1]

            t0 = time.perf_counter()
            cc_row = np.ascontiguousarray(orc.agg_row(0, orc.ew_binary(2, Ch, Ch)[1])[1].T)
            parts = _threaded(assign_piece, pieces, threads)
            PtX, cnt = sum(p_[0] for p_ in parts), sum(p_[1] for p_ in parts)
            orc.ew_binary(3, PtX, np.ascontiguousarray(cnt.T))
            dt = time.perf_counter() - t0
            cpu = {"value": round(nbytes / dt / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
                   "sample": f"one iteration on all {n} rows, {threads} threads: products by numpy's {_blas_name()} sgemm, the other "
                             f"operators by the port's scalar kernels on row pieces ({dt:.2f} s)"}
        step_bytes = n * f * 4 + n * 4 + n * 8  # X, xx, idx
        step_flops = 2.0 * n * f * k          # X t(C) on the matrix cores; the per-cluster sums are n * f additions on the ordinary ALUs
        roof = {"bound": "hbm", "kernel": "ts_nt_kernel<float,1,true,4,true> + kmeans_finish_kernel (one pass over X: X t(C), distances, "
                                          "row arg-min, per-cluster sums and sizes)",
                "achieved": round(step_bytes / t_step / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(step_bytes / t_step / 1e6 / HBM_PEAK_GBS, 4), "traffic": None,
                "mfma_tflops": round(step_flops / t_step / 1e9, 1)}
        out = _line(nbytes / ms / 1e6, "GB/s", ms, args, "f32",
                    "k-means Lloyd iteration: X 2000000x64 f32 (16 Gaussians), C 16x64; step = one iteration of runs of ten from "
                    "the seeded rows (one pass over X: assignment and update from the same loads)",
                    roof, cpu, {"canonical_bytes_per_step": nbytes, "bytes_per_step_one_pass": step_bytes,
                                "one_pass_gbs": round(step_bytes / ms / 1e6, 1), "step_kernels_ms": round(t_step, 4),
                                "assign_ms": round(t_assign, 4), "update_ms": round(t_update, 4), "xct_ms": round(t_gemm, 4),
                                "ms_per_step_two_passes": round(ms_two, 4), "ms_per_step_operator_sequence": round(ms_seq, 4)})
    elif args.config == 4:
        res = measure_contractions(torch, ctx, args.steps, args.warmup)
        cpu = None
        if orc:
            a = np.random.default_rng(0).random((512, 512))
            t0 = time.perf_counter()
            orc.matmul(a, a)
            dt = time.perf_counter() - t0
            blas_tflops, blas_what = blas_baseline()
            cpu = {"value": round(blas_tflops, 4), "unit": "TFLOP/s", "cores": min(os.cpu_count() or 1, 16), "kind": "port",
                   "sample": f"{blas_what}: the reference's CPU MatMul is a call of this library; beside it the oracle's "
                             f"scalar triple loop at 512^3 on one thread, {2 * 512 ** 3 / dt / 1e12:.5f} TFLOP/s ({dt:.2f} s)"}
        f64 = res["matmul_f64_8192"]["tflops"]
        roof = {"bound": "mfma", "kernel": "gemm_kernel<double,128,128,8,2,2,false,false,0,true>", "achieved": f64,
                "peak": MFMA_PEAK["f64"], "unit": "TFLOP/s", "frac": round(f64 / MFMA_PEAK["f64"], 4), "traffic": None}
        out = _line(f64, "TFLOP/s", res["matmul_f64_8192"]["ms"], args, "f64",
                    "dense contractions: (a) MatMul f64 8192^3 [value], (b) MatMul f32 16384^3, (c) Syrk f64 1000000x1024",
                    roof, cpu, res)
    else:
        N = 4096
        rng = np.random.default_rng(42)
        he = lambda shape, fan: (rng.standard_normal(shape) * np.sqrt(2.0 / fan)).astype(np.float32)
        small = lambda shape: (rng.standard_normal(shape) * 0.1).astype(np.float32)
        Wh = {"w1": he((32, 25), 25), "b1": small((32, 1)), "w2": he((64, 800), 800), "b2": small((64, 1)),
              "w3": he((3136, 512), 3136), "b3": small((1, 512)), "w4": he((512, 10), 512), "b4": small((1, 10))}
        W = {k_: DenseMatrix.from_numpy(ctx, v) for k_, v in Wh.items()}
        xt = torch.rand(N, 784, device="cuda", generator=gen)
        x = DenseMatrix.from_torch(ctx, xt)
        ms = _timed(torch, lambda: lenet_forward(ctx, x, W, N), args.steps, args.warmup)
        # every layer on its own, into a result matrix that is there already (a layer that allocates its result puts
        # a synchronising release of the last one between the kernels, which the events would count)
        from daphne_amd.kernels import affineForward, affineForwardFused, conv2dForwardFused, softmax
        h1, _, _ = conv2dForwardFused(None, x, W["w1"], W["b1"], N, 1, 28, 28, 5, 5, 1, 1, 2, 2, ctx, relu=True, pool=True)
        h2, _, _ = conv2dForwardFused(None, h1, W["w2"], W["b2"], N, 32, 14, 14, 5, 5, 1, 1, 2, 2, ctx, relu=True, pool=True)
        h3 = affineForwardFused(None, h2, W["w3"], W["b3"], ctx)
        h4 = affineForward(None, h3, W["w4"], W["b4"], ctx)
        h5 = softmax(None, h4, ctx)
        layer_ms = {
            "conv1+bias+relu+pool": _events(torch, lambda: conv2dForwardFused(h1, x, W["w1"], W["b1"], N, 1, 28, 28, 5, 5, 1, 1, 2, 2, ctx, relu=True, pool=True)),
            "conv2+bias+relu+pool": _events(torch, lambda: conv2dForwardFused(h2, h1, W["w2"], W["b2"], N, 32, 14, 14, 5, 5, 1, 1, 2, 2, ctx, relu=True, pool=True)),
            "affine1+relu": _events(torch, lambda: affineForwardFused(h3, h2, W["w3"], W["b3"], ctx)),
            "affine2": _events(torch, lambda: affineForward(h4, h3, W["w4"], W["b4"], ctx)),
            "softmax": _events(torch, lambda: softmax(h5, h4, ctx)),
        }
        layer_ms = {k_: round(v, 4) for k_, v in layer_ms.items()}
        flops = {"conv1+bias+relu+pool": 2.0 * N * 32 * 784 * 25, "conv2+bias+relu+pool": 2.0 * N * 64 * 196 * 800,
                 "affine1+relu": 2.0 * N * 3136 * 512, "affine2": 2.0 * N * 512 * 10}
        layer_tflops = {k_: round(flops[k_] / layer_ms[k_] / 1e9, 2) for k_ in flops}
        # the same network with one kernel per operator, for comparison
        ms_unfused = _timed(torch, lambda: lenet_forward(ctx, x, W, N, fused=False), args.steps, args.warmup)
        cpu = None
        if orc:
            # the port's loops (the reference's CPU convolution and pooling are plain loops too, Conv2DForward.h:77-140),
            # images dealt to all host threads; the affine layers by numpy's BLAS as the reference's MatMul would
            nb = 16 * threads
            xh = xt[:nb].cpu().numpy()
            relu = lambda a: orc.ew_binary_sca(14, a, 0.0)[1]

            def forward(sl):
                m_ = sl.stop - sl.start
                h = relu(orc.conv2d(xh[sl], Wh["w1"], Wh["b1"], m_, 1, 28, 28, 5, 5, 1, 1, 2, 2)[1])
                h = orc.maxpool(h, m_, 32, 28, 28, 2, 2, 2, 2, 0, 0)[1]
                h = relu(orc.conv2d(h, Wh["w2"], Wh["b2"], m_, 32, 14, 14, 5, 5, 1, 1, 2, 2)[1])
                h = orc.maxpool(h, m_, 64, 14, 14, 2, 2, 2, 2, 0, 0)[1]
                h = relu(orc.ew_binary(0, h @ Wh["w3"], Wh["b3"])[1])
                return orc.softmax(orc.ew_binary(0, h @ Wh["w4"], Wh["b4"])[1])[1]

            pieces = [slice(a, a + 16) for a in range(0, nb, 16)]
            t0 = time.perf_counter()
            _threaded(forward, pieces, threads)
            dt = time.perf_counter() - t0
            cpu = {"value": round(nb / dt, 2), "unit": "images/s", "cores": threads, "kind": "port",
                   "sample": f"batch {nb} of {N} in pieces of 16 images on {threads} threads: convolution and pooling by the port's "
                             f"loops, affine layers by numpy's {_blas_name()} ({dt:.2f} s)"}
        c2 = layer_tflops["conv2+bias+relu+pool"]
        roof = {"bound": "mfma", "kernel": "conv2d_resident_kernel<float,4,NF,true> (conv2 + ReLU + 2x2 max-pool: 4096x32x14x14, 64 filters 5x5, "
                                           "images resident in LDS)",
                "achieved": c2, "peak": MFMA_PEAK["f32"], "unit": "TFLOP/s", "frac": round(c2 / MFMA_PEAK["f32"], 4), "traffic": None}
        out = _line(N / ms * 1e3, "images/s", ms, args, "f32",
                    "LeNet-style CNN inference, batch 4096, 1x28x28 input, conv-pool-conv-pool-affine-affine-softmax "
                    "(ReLU and pooling in the epilogues of the layers before them)",
                    roof, cpu, {"layer_ms": layer_ms, "layer_tflops": layer_tflops, "total_gflop": 100.6,
                                "ms_per_step_one_kernel_per_operator": round(ms_unfused, 4)})
    print(json.dumps(out))
    return 0
