"""Comparison helpers shared by the parity tests.

Tolerances are the ones the build targets: relative error <= 1e-4 for float, <= 1e-10 for
double, bit-exact for indices / integer-valued outputs and for ops that are a single IEEE
operation.
"""
import numpy as np

RTOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-10}


def assert_exact(got, exp):
    got, exp = np.asarray(got), np.asarray(exp)
    assert got.shape == exp.shape, (got.shape, exp.shape)
    same = (got == exp) | (np.isnan(got) & np.isnan(exp)) if got.dtype.kind == "f" else (got == exp)
    if not same.all():
        bad = np.argwhere(~same)[:5]
        raise AssertionError(f"{(~same).sum()} mismatches, first at {bad.tolist()}: got {got[~same][:5]} exp {exp[~same][:5]}")


def variance_floor(x, op_is_stddev=False):
    """Absolute floor for comparing variances (standard deviations) of the values x item by item: the rounding
    noise of sum((x - mean)^2) / n when the true variance is (nearly) zero, 16 eps max|x|^2. It only matters for
    such items; everywhere else the relative bound is the larger one."""
    x = np.asarray(x)
    f = 16 * np.finfo(x.dtype).eps * float(np.max(np.abs(x[np.isfinite(x)]), initial=0.0)) ** 2
    return float(np.sqrt(f)) if op_is_stddev else f


def assert_close(got, exp, rtol=None, elementwise=True, atol=0.0):
    """Relative error check. elementwise: |g-e| <= rtol*|e| + atol per item (plus a tiny absolute floor
    for items that are exactly 0); otherwise norm-wise: max|g-e| <= rtol*max|e|."""
    got, exp = np.asarray(got), np.asarray(exp)
    assert got.shape == exp.shape, (got.shape, exp.shape)
    rtol = RTOL[np.dtype(exp.dtype)] if rtol is None else rtol
    nan_g, nan_e = np.isnan(got), np.isnan(exp)
    assert (nan_g == nan_e).all(), f"NaN pattern differs at {np.argwhere(nan_g != nan_e)[:5].tolist()}"
    inf_e = np.isinf(exp)
    assert (got[inf_e] == exp[inf_e]).all(), "infinities differ"
    m = ~(nan_e | inf_e)
    g, e = got[m].astype(np.float64), exp[m].astype(np.float64)
    if g.size == 0:
        return
    err = np.abs(g - e)
    if elementwise:
        tiny = np.finfo(exp.dtype).tiny if exp.dtype.kind == "f" else 0.0
        bound = rtol * np.abs(e) + 16 * tiny + atol
    else:
        bound = np.full_like(e, rtol * np.abs(e).max())
    bad = err > bound
    if bad.any():
        i = np.argmax(err - bound)
        raise AssertionError(f"{bad.sum()} of {bad.size} items out of tolerance {rtol}: worst got {g[i]!r} exp {e[i]!r} "
                             f"rel {err[i] / max(abs(e[i]), 1e-300):.3e}")
