#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

Workload (BASELINE.json configs[1]): the fused elementwise + aggregation vectorized pipeline
    X 20,000,000 x 64 float32 ~ N(5, 2^2)
    mu = colMeans(X); sd = sqrt(colVars(X)); Z = (X - mu) / sd; r = rowSums(Z * Z); s = sum(r > 64)
One "step" is one pass of that pipeline over X, which is already resident in HBM:
    aggCol(MEAN) -> aggCol(VAR) -> ewUnary(SQRT) on 1 x 64 -> one fused pipeline kernel (reads X, writes r, s).

`value` is GB/s over the canonical algorithmic bytes of the step (each stage: distinct inputs and
outputs once; Z is never materialised): 3 x |X| + |r| + the small vectors. `roofline` is the
fused pipeline kernel alone (its bytes / its own duration, timed with events on the stream it
runs on). `cpu_baseline` times the reference's algorithm for the same pipeline (CPU restatement
in oracle/, same operator-by-operator multithreaded engine) on a bounded row prefix.

After the timed pipeline steps the same run measures the other half of the metric, the dense contractions at the
sizes BASELINE.json quotes (MatMul f64 8192^3, MatMul f32 16384^3, Syrk f64 1e6 x 1024), and reports them in
`config.contractions`; `--no-contractions` skips that.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--rows R] [--no-cpu] [--no-contractions]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0
COUNTER_PROFILE = os.path.join("profiles", "zscore_pipeline_20Mx64_f32_hbm_counters.txt")


def measured_traffic(kernel: str):
    """HBM bytes per launch of `kernel` from the committed counter summary (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE,
    scaled by a copy kernel of known size): the 'read KiB' and 'write KiB' columns of the kernel's row."""
    try:
        with open(os.path.join(ROOT, COUNTER_PROFILE)) as f:
            for line in f:
                cols = line.split()
                if cols and cols[0] == kernel and len(cols) >= 5:
                    return int(round((float(cols[2]) + float(cols[4])) * 1024))
    except (OSError, ValueError):
        pass
    return None



def time_stage_via_wrappers(x_ptr: int, rows: int, cols: int, thr: float, steps: int):
    """ms per run of the fused stage through the generated kernel entry points (tests/cpp/glue_harness.cpp builds the
    run-time objects those take). None if the harness or the kernel library was not built."""
    import ctypes as C

    from daphne_amd import build as b

    harness = os.path.join(ROOT, "tests", "cpp", "build", "libglue_harness.so")
    if not (os.path.exists(harness) and os.path.exists(b.KERNEL_LIB_PATH)):
        return None
    h = C.CDLL(harness)
    h.th_ctx_create.restype = C.c_void_p
    h.th_last_error.restype = C.c_char_p
    h.th_ctx_destroy.argtypes = [C.c_void_p]
    f = h.th_time_zscore_stage_f32
    f.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_float, C.c_int, C.c_int] + [C.POINTER(C.c_double)] * 4
    dctx = h.th_ctx_create()
    if not dctx:
        raise RuntimeError(h.th_last_error().decode())
    out = [C.c_double() for _ in range(4)]
    try:
        if f(dctx, str(b.KERNEL_LIB_PATH).encode(), C.c_void_p(x_ptr), rows, cols, thr, 5, steps, *[C.byref(o) for o in out]) != 0:
            raise RuntimeError(h.th_last_error().decode())
    finally:
        h.th_ctx_destroy(dctx)
    return {"ms_by_operators": out[0].value, "ms_as_one_kernel": out[1].value, "count_by_operators": out[2].value,
            "count_as_one_kernel": out[3].value, "steps": steps}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--config", type=int, default=2, choices=[1, 2, 3, 4, 5],
                    help="which BASELINE.json configuration to run (1-based); the default 2 is the headline "
                         "metric, the others print the same kind of line for their own workload")
    ap.add_argument("--one-pass-stats", action="store_true",
                    help="take colMeans and colVars from one pass over X (dh_agg_col_moments): a shorter step that moves "
                         "10.3 instead of 15.4 GB; `value` is then GB/s over the bytes actually moved")
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--rows", type=int, default=20_000_000)
    ap.add_argument("--cols", type=int, default=64)
    ap.add_argument("--cpu-rows", type=int, default=20_000_000, help="row prefix timed on the host CPU")
    ap.add_argument("--cpu-reps", type=int, default=3, help="repetitions of the CPU baseline (median is reported)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-contractions", action="store_true", help="skip the MatMul / Syrk measurements after the pipeline")
    ap.add_argument("--no-wrappers", action="store_true",
                    help="skip timing the fused stage through the generated HIP_<mnemonic> entry points of libHIPKernels.so")
    ap.add_argument("--contraction-steps", type=int, default=5)
    ap.add_argument("--calib", action="store_true",
                    help="also launch one plain elementwise copy of X (reads |X|, writes |X|): the known-size "
                         "kernel that hardware byte counters are scaled against")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on exactly one GPU; --gpus {args.gpus} is not supported "
              "(the path shards by rows with one small all-reduce, which is documented, not built).", file=sys.stderr)
        return 2

    if args.config != 2:
        import bench_other_configs

        return bench_other_configs.run(args)

    import numpy as np
    import torch

    from daphne_amd.kernels import (AggOpCode, BinaryOpCode, DenseMatrix, HIPContext, UnaryOpCode, aggCol, aggColMoments,
                                    ewUnaryMat)
    from daphne_amd.pipeline import SELF, VectorizedPipeline

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    torch.cuda.set_device(0)
    ctx = HIPContext(0)  # kernels go to the default stream, which is also torch's current stream
    R, Cc = args.rows, args.cols
    gen = torch.Generator(device="cuda").manual_seed(42)
    X_t = torch.empty(R, Cc, device="cuda", dtype=torch.float32)
    X_t.normal_(5.0, 2.0, generator=gen)
    X = DenseMatrix.from_torch(ctx, X_t)

    mu = DenseMatrix(ctx, 1, Cc, np.float32)
    var = DenseMatrix(ctx, 1, Cc, np.float32)
    sd = DenseMatrix(ctx, 1, Cc, np.float32)
    r = DenseMatrix(ctx, R, 1, np.float32)
    thr = float(Cc)

    pipe = VectorizedPipeline(ctx, X)
    pipe.ewBinary(BinaryOpCode.SUB, mu).ewBinary(BinaryOpCode.DIV, sd).ewBinary(BinaryOpCode.MUL, SELF)
    pipe.rowAgg(AggOpCode.SUM)
    pipe.storeRow(r)
    pipe.ewBinary(BinaryOpCode.GT, thr)
    s = pipe.reduceAll(AggOpCode.SUM)

    ev = lambda: torch.cuda.Event(enable_timing=True)
    stage_events = []

    def step(record: bool):
        e = [ev() for _ in range(4)] if record else None
        if record:
            e[0].record()
        if args.one_pass_stats:
            if record:
                e[1].record()
            aggColMoments(X, ctx, stddev=True, res_mean=mu, res_var=sd)
        else:
            aggCol(AggOpCode.MEAN, mu, X, ctx)
            if record:
                e[1].record()
            aggCol(AggOpCode.VAR, var, X, ctx)
            ewUnaryMat(UnaryOpCode.SQRT, sd, var, ctx)  # checks its domain: one tiny device-to-host read
        if record:
            e[2].record()
        pipe.run()
        if record:
            e[3].record()
            stage_events.append(e)

    if args.calib:
        from daphne_amd.kernels import ewBinaryObjSca

        Z = DenseMatrix(ctx, R, Cc, np.float32)
        ewBinaryObjSca(BinaryOpCode.MUL, Z, X, 1.0, ctx)
        ctx.sync()
        Z.destroy()
    for _ in range(args.warmup):
        step(False)
    torch.cuda.synchronize()
    ctx.kernel_timing(True)  # events around the fused stage's body kernel alone, on the context's stream, no waiting
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(True)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    kernel_ms_total, kernel_launches = ctx.kernel_timing_read()
    ctx.kernel_timing(False)

    x_bytes = R * Cc * 4
    vec_bytes = Cc * 4
    bytes_s1 = x_bytes + vec_bytes
    bytes_s2 = x_bytes + vec_bytes + 2 * vec_bytes  # colVars + the sqrt on 1 x C
    bytes_s3 = x_bytes + 2 * vec_bytes + R * 4 + 4  # read X, mu, sd; write r, s
    bytes_step = bytes_s1 + bytes_s2 + bytes_s3
    canonical_bytes = bytes_step
    if args.one_pass_stats:
        bytes_s1 = 0
        bytes_step = bytes_s2 + bytes_s3
    value = bytes_step / (ms_per_step * 1e-3) / 1e9

    ms = lambda a, b: a.elapsed_time(b)
    t_s1 = float(np.mean([ms(e[0], e[1]) for e in stage_events]))
    t_s2 = float(np.mean([ms(e[1], e[2]) for e in stage_events]))
    t_s3 = float(np.mean([ms(e[2], e[3]) for e in stage_events]))
    # the dominant kernel's own duration (the stage's events also cover the two small kernels that fold its partial results)
    kernel_ms = kernel_ms_total / kernel_launches if kernel_launches else t_s3
    achieved = bytes_s3 / (kernel_ms * 1e-3) / 1e9

    s_val = float(s.to_numpy()[0, 0])
    props = ctx.props()
    # how the body ran: 1 = the kernel specialised at run time (what `roofline.kernel` names), 0 = the interpreter
    from daphne_amd import capi

    pipeline_mode = int(capi.lib().dh_vectorized_pipeline_last_mode())

    # The same fused stage the way a DAPHNE program compiled with --hip reaches it: through the generated
    # HIP_<mnemonic> entry points of libHIPKernels.so, as the outlined device body (one entry point per operator) and
    # as HIP_fusedPipeline with the body's text (lowered to the one kernel at run time).
    via_wrappers = None
    if not args.no_wrappers:
        # five untimed runs of each form first: the first fused one compiles its body, and the device takes a few
        # launches to settle after that second of idling
        via_wrappers = time_stage_via_wrappers(int(X_t.data_ptr()), R, Cc, thr, max(1, min(args.steps, 20)))
        if via_wrappers is not None and via_wrappers["count_by_operators"] != via_wrappers["count_as_one_kernel"]:
            print(f"bench.py: the two forms of the fused stage disagree: {via_wrappers}", file=sys.stderr)
            return 4

    xh = None
    if not args.no_cpu:
        xh = X_t[:min(args.cpu_rows, R)].cpu().numpy()

    contractions = None
    if not args.no_contractions:
        import bench_other_configs

        # the pipeline's matrices make room for the contraction operands (X keeps the torch tensor alive)
        r.destroy()
        pipe = X = X_t = None
        torch.cuda.empty_cache()
        contractions = bench_other_configs.measure_contractions(torch, ctx, args.contraction_steps, 1)

    cpu = None
    if not args.no_cpu:
        import oracle_binding as orc

        n_cpu = min(args.cpu_rows, R)
        threads = min(os.cpu_count() or 1, 16)
        runs = []
        for _ in range(max(1, args.cpu_reps)):
            st, mu_c, sd_c, r_c, s_c, secs = orc.zscore_pipeline(xh, threads=threads, thr=thr)
            runs.append(secs.copy())
        runs.sort(key=lambda a: float(a.sum()))
        secs = runs[len(runs) // 2]
        cpu_bytes = 3 * n_cpu * Cc * 4 + n_cpu * 4 + 7 * vec_bytes + 4
        cpu = {
            "value": round(cpu_bytes / float(secs.sum()) / 1e9, 4),
            "unit": "GB/s",
            "cores": threads,
            "kind": "port",
            "sample": (f"first {n_cpu} of {R} rows, {len(runs)} repetitions (median), same pipeline and byte convention; "
                       f"column statistics single-threaded as in the reference ({secs[0]:.2f} s), row-split body on "
                       f"{threads} threads with 96 KiB batches ({secs[1]:.2f} s)"),
        }

    out = {
        "metric": "HBM GB/s (% peak) on fused ew+agg pipelines; MatMul/Syrk TFLOP/s (% MFMA peak)",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"z-score + rowSums + threshold count pipeline, X {R}x{Cc} f32 N(5,2^2) (BASELINE.json configs[1])",
            "rows": R, "cols": Cc,
            "canonical_bytes_per_step": canonical_bytes,
            "bytes_moved_per_step": bytes_step,
            "column_statistics": "one pass (dh_agg_col_moments)" if args.one_pass_stats else "colMeans and colVars as two kernels",
            "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
            "stage_ms": {"colMeans": round(t_s1, 4), "colVars+sqrt": round(t_s2, 4), "fused_pipeline": round(t_s3, 4)},
            "stage_gbs": {"colMeans": round(bytes_s1 / t_s1 / 1e6, 1), "colVars+sqrt": round(bytes_s2 / t_s2 / 1e6, 1),
                          "fused_pipeline": round(bytes_s3 / t_s3 / 1e6, 1)},
            "count_r_gt_thr": s_val,
            "pipeline_mode": "specialised" if pipeline_mode == 1 else "interpreted",
            # the fused stage as a patched DAPHNE dispatches it, through libHIPKernels.so: the outlined body (one entry
            # point per operator, every intermediate in memory) and HIP_fusedPipeline with the body's text (one launch)
            "ms_fused_stage_op_by_op_via_wrappers": None if via_wrappers is None else round(via_wrappers["ms_by_operators"], 4),
            "ms_fused_stage_via_fusedPipeline_wrapper": None if via_wrappers is None else round(via_wrappers["ms_as_one_kernel"], 4),
            "contractions": contractions,
            "device": props["name"], "compute_units": props["compute_units"], "clock_khz": props["clock_khz"],
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "dh_jit_pipeline = dh_pipe::pipeline_body<float,4,1> specialised for the z-score/rowSums/count body",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            # average duration of that kernel over the timed steps: a pair of events around each of its launches
            "kernel_us": round(kernel_ms * 1e3, 1), "launches_timed": int(kernel_launches),
            # HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE at the default shape, read
            # from the committed summary of those runs
            "traffic": measured_traffic("dh_jit_pipeline") if (R, Cc) == (20_000_000, 64) else None,
            "traffic_unit": "bytes per launch",
            "traffic_source": COUNTER_PROFILE,
            "algorithmic_bytes_per_launch": bytes_s3,
        },
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))
    if pipeline_mode != 1:
        print("bench.py: the pipeline body was interpreted, not specialised at run time (" +
              capi.lib().dh_last_error().decode(errors="replace") + "); the line above does not measure the kernel it names",
              file=sys.stderr)
        return 3
    return 0


if __name__ == "__main__":
    sys.exit(main())
