"""ctypes binding of oracle/liboracle.so - the CPU restatement of the reference's kernels.

Test infrastructure only. Builds the library with `make -C oracle` if it is missing.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

ORACLE_DIR = Path(__file__).resolve().parent.parent / "oracle"
LIB = ORACLE_DIR / "liboracle.so"

ST_OK, ST_RUNTIME, ST_INVALID, ST_DOMAIN = 0, 1, 2, 3
_SUF = {np.dtype(np.float32): "f32", np.dtype(np.float64): "f64", np.dtype(np.int64): "si64", np.dtype(np.uint64): "ui64",
        np.dtype(np.int32): "si32", np.dtype(np.uint32): "ui32"}
_CT = {np.dtype(np.float32): C.c_float, np.dtype(np.float64): C.c_double, np.dtype(np.int64): C.c_int64,
       np.dtype(np.uint64): C.c_uint64, np.dtype(np.int32): C.c_int32, np.dtype(np.uint32): C.c_uint32}
_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB.exists():
            subprocess.run(["make", "-C", str(ORACLE_DIR)], check=True, capture_output=True)
        _lib = C.CDLL(str(LIB))
    return _lib


def _p(a):
    return C.c_void_p(a.ctypes.data) if a is not None else None


def _f(name, dt):
    return getattr(lib(), f"oracle_{name}_{_SUF[np.dtype(dt)]}")


def _sc(dt, v):
    dt = np.dtype(dt)
    return _CT[dt](int(v) if dt.kind in "iu" else v)


def _ld(a):
    """Leading dimension (elements) of a 2-D row-major array or view."""
    if a.size == 0:
        return max(a.shape[1], 1)
    assert a.ndim == 2 and (a.shape[1] <= 1 or a.strides[1] == a.itemsize)
    return a.strides[0] // a.itemsize if a.shape[0] > 1 else max(a.shape[1], 1)


sz = C.c_size_t


def ew_binary(op, lhs, rhs):
    res = np.empty(lhs.shape, lhs.dtype)
    st = _f("ew_binary", lhs.dtype)(int(op), _p(res), sz(_ld(res)), _p(lhs), sz(lhs.shape[0]), sz(lhs.shape[1]),
                                    sz(_ld(lhs)), _p(rhs), sz(rhs.shape[0]), sz(rhs.shape[1]), sz(_ld(rhs)))
    return st, res


def ew_binary_sca(op, lhs, s):
    res = np.empty(lhs.shape, lhs.dtype)
    st = _f("ew_binary_sca", lhs.dtype)(int(op), _p(res), sz(_ld(res)), _p(lhs), sz(lhs.shape[0]), sz(lhs.shape[1]),
                                        sz(_ld(lhs)), _sc(lhs.dtype, s))
    return st, res


def ew_unary(op, arg):
    res = np.empty(arg.shape, arg.dtype)
    st = _f("ew_unary", arg.dtype)(int(op), _p(res), sz(_ld(res)), _p(arg), sz(arg.shape[0]), sz(arg.shape[1]),
                                   sz(_ld(arg)))
    return st, res


def agg_all(op, arg):
    out = np.empty(1, arg.dtype)
    st = _f("agg_all", arg.dtype)(int(op), _p(arg), sz(arg.shape[0]), sz(arg.shape[1]), sz(_ld(arg)), _p(out))
    return st, out[0]


def agg_row(op, arg):
    if int(op) in (4, 5):
        res = np.empty((arg.shape[0], 1), np.uint64)
        st = _f("agg_row_idx", arg.dtype)(int(op), _p(res), sz(1), _p(arg), sz(arg.shape[0]), sz(arg.shape[1]),
                                          sz(_ld(arg)))
        return st, res
    res = np.empty((arg.shape[0], 1), arg.dtype)
    st = _f("agg_row", arg.dtype)(int(op), _p(res), sz(1), _p(arg), sz(arg.shape[0]), sz(arg.shape[1]), sz(_ld(arg)))
    return st, res


def agg_col(op, arg):
    if int(op) in (4, 5):
        res = np.empty((1, arg.shape[1]), np.uint64)
        st = _f("agg_col_idx", arg.dtype)(int(op), _p(res), _p(arg), sz(arg.shape[0]), sz(arg.shape[1]), sz(_ld(arg)))
        return st, res
    res = np.empty((1, arg.shape[1]), arg.dtype)
    st = _f("agg_col", arg.dtype)(int(op), _p(res), _p(arg), sz(arg.shape[0]), sz(arg.shape[1]), sz(_ld(arg)))
    return st, res


def matmul(lhs, rhs, ta=False, tb=False):
    nr1 = lhs.shape[1] if ta else lhs.shape[0]
    nc2 = rhs.shape[0] if tb else rhs.shape[1]
    res = np.empty((nr1, nc2), lhs.dtype)
    st = _f("matmul", lhs.dtype)(_p(res), sz(max(nc2, 1)), _p(lhs), sz(lhs.shape[0]), sz(lhs.shape[1]), sz(_ld(lhs)),
                                 _p(rhs), sz(rhs.shape[0]), sz(rhs.shape[1]), sz(_ld(rhs)), int(ta), int(tb))
    return st, res


def syrk(arg, trans_left=True):
    n = arg.shape[1] if trans_left else arg.shape[0]
    res = np.empty((n, n), arg.dtype)
    st = _f("syrk", arg.dtype)(_p(res), sz(n), _p(arg), sz(arg.shape[0]), sz(arg.shape[1]), sz(_ld(arg)),
                               int(trans_left))
    return st, res


def solve(A, b):
    A = np.ascontiguousarray(A)
    b = np.ascontiguousarray(b).reshape(-1)
    x = np.empty(b.shape, A.dtype)
    st = _f("solve", A.dtype)(_p(x), _p(A), sz(A.shape[0]), _p(b))
    return st, x.reshape(-1, 1)


def conv2d(data, filt, bias, N, Cc, H, W, Hf, Wf, sh, sw, ph, pw):
    F = filt.shape[0]
    P = (H + 2 * ph - Hf) // sh + 1
    Q = (W + 2 * pw - Wf) // sw + 1
    res = np.empty((N, F * P * Q), data.dtype)
    rh, rw = sz(), sz()
    st = _f("conv2d_forward", data.dtype)(_p(res), C.byref(rh), C.byref(rw), _p(data), _p(filt), _p(bias), sz(N),
                                          sz(Cc), sz(H), sz(W), sz(F), sz(Hf), sz(Wf), sz(sh), sz(sw), sz(ph), sz(pw))
    return st, res, rh.value, rw.value


def maxpool(data, N, Cc, H, W, ph, pw, sh, sw, padh, padw):
    P = (H + 2 * padh - ph) // sw + 1
    Q = (W + 2 * padw - pw) // sh + 1
    res = np.empty((N, Cc * P * Q), data.dtype)
    rh, rw = sz(), sz()
    st = _f("maxpool_forward", data.dtype)(_p(res), C.byref(rh), C.byref(rw), _p(data), sz(N), sz(Cc), sz(H), sz(W),
                                           sz(ph), sz(pw), sz(sh), sz(sw), sz(padh), sz(padw))
    return st, res, rh.value, rw.value


def bias_add(data, bias):
    res = np.empty(data.shape, data.dtype)
    st = _f("bias_add", data.dtype)(_p(res), _p(data), sz(data.shape[0]), sz(data.shape[1]), _p(bias), sz(bias.size))
    return st, res


def batchnorm(data, gamma, beta, mean, var, eps, stat_index=0):
    res = np.empty(data.shape, data.dtype)
    st = _f("batchnorm_inference", data.dtype)(_p(res), _p(data), sz(data.shape[0]), sz(data.shape[1]), _p(gamma),
                                               _p(beta), _p(mean), _p(var), sz(gamma.shape[0]), _sc(data.dtype, eps),
                                               int(stat_index))
    return st, res


def softmax(arg):
    res = np.empty(arg.shape, arg.dtype)
    st = _f("softmax", arg.dtype)(_p(res), sz(_ld(res)), _p(arg), sz(arg.shape[0]), sz(arg.shape[1]), sz(_ld(arg)))
    return st, res

def avgpool(data, N, Cc, H, W, ph, pw, sh, sw, padh, padw):
    P = (H + 2 * padh - ph) // sw + 1
    Q = (W + 2 * padw - pw) // sh + 1
    res = np.empty((N, Cc * P * Q), data.dtype)
    rh, rw = sz(), sz()
    st = _f("avgpool_forward", data.dtype)(_p(res), C.byref(rh), C.byref(rw), _p(data), sz(N), sz(Cc), sz(H), sz(W),
                                           sz(ph), sz(pw), sz(sh), sz(sw), sz(padh), sz(padw))
    return st, res, rh.value, rw.value


def relu(arg):
    res = np.empty(arg.shape, arg.dtype)
    st = _f("relu_forward", arg.dtype)(_p(res), sz(_ld(res)), _p(arg), sz(arg.shape[0]), sz(arg.shape[1]), sz(_ld(arg)))
    return st, res


def fill(value, rows, cols, dt):
    res = np.empty((rows, cols), dt)
    st = _f("fill", dt)(_p(res), sz(max(cols, 1)), _sc(dt, value), sz(rows), sz(cols))
    return st, res


def col_bind(lhs, rhs):
    res = np.empty((lhs.shape[0], lhs.shape[1] + rhs.shape[1]), lhs.dtype)
    st = _f("col_bind", lhs.dtype)(_p(res), sz(_ld(res)), _p(lhs), sz(lhs.shape[0]), sz(lhs.shape[1]), sz(_ld(lhs)),
                                   _p(rhs), sz(rhs.shape[0]), sz(rhs.shape[1]), sz(_ld(rhs)))
    return st, res


def extract_col(arg, sel):
    sel = np.ascontiguousarray(sel, dtype=np.int64)
    res = np.empty((arg.shape[0], sel.shape[0]), arg.dtype)
    st = _f("extract_col", arg.dtype)(_p(res), sz(_ld(res)), _p(arg), sz(arg.shape[0]), sz(arg.shape[1]), sz(_ld(arg)),
                                      _p(sel), sz(sel.shape[0]), sz(sel.shape[1] if sel.ndim == 2 else 1))
    return st, res


def transpose(arg):
    res = np.empty((arg.shape[1], arg.shape[0]), arg.dtype)
    st = _f("transpose", arg.dtype)(_p(res), sz(_ld(res)), _p(arg), sz(arg.shape[0]), sz(arg.shape[1]), sz(_ld(arg)))
    return st, res


def gemv(mat, vec):
    """Gemv.h:51-77: t(mat) @ vec, through the same restatement as MatMul with transa."""
    return matmul(mat, vec, True, False)


def zscore_pipeline(X, threads=4, thr=64.0):
    """Reference-style execution of the z-score / row-sum / threshold-count pipeline (float32):
    column statistics as single kernel calls, the row-split body on `threads` workers."""
    assert X.dtype == np.float32 and X.flags.c_contiguous
    rows, cols = X.shape
    mu, sd = np.empty((1, cols), np.float32), np.empty((1, cols), np.float32)
    r, s = np.empty((rows, 1), np.float32), np.empty(1, np.float32)
    secs = np.zeros(2, np.float64)
    st = lib().oracle_zscore_pipeline_f32(_p(X), sz(rows), sz(cols), C.c_int(threads), C.c_float(thr), _p(mu), _p(sd),
                                          _p(r), _p(s), _p(secs))
    return st, mu, sd, r, s[0], secs


# -- DNN training kernels (oracle/dnn_training_cpu.cpp) ---------------------------------------
def batchnorm_train_forward(x, gamma, beta, ema_mean, ema_var, eps, mu):
    dt = x.dtype
    C = gamma.size
    res = np.empty_like(x)
    outs = [np.empty((C, 1), dt) for _ in range(4)]  # new_ema_mean, new_ema_var, mean, inv_var
    st = _f("batchnorm_train_forward", dt)(_p(res), _p(outs[0]), _p(outs[1]), _p(outs[2]), _p(outs[3]), _p(x), sz(x.shape[0]),
                                           sz(x.shape[1]), _p(gamma), _p(beta), _p(ema_mean), _p(ema_var), sz(C),
                                           _sc(dt, eps), _sc(dt, mu))
    return st, res, outs[0], outs[1], outs[2], outs[3]


def batchnorm_backward(mean, inv_var, x, dout, gamma):
    dt = x.dtype
    C = gamma.size
    dX, dG, dB = np.empty_like(x), np.empty((C, 1), dt), np.empty((C, 1), dt)
    st = _f("batchnorm_backward", dt)(_p(dX), _p(dG), _p(dB), _p(mean), _p(inv_var), _p(x), _p(dout), sz(x.shape[0]),
                                      sz(x.shape[1]), _p(gamma), sz(C))
    return st, dX, dG, dB


def _pool_backward(name, x, dout, N, C, H, W, ph, pw, sh, sw, padh, padw):
    res = np.empty((N, C * H * W), x.dtype)
    st = _f(name, x.dtype)(_p(res), _p(x), _p(dout), sz(N), sz(C), sz(H), sz(W), sz(ph), sz(pw), sz(sh), sz(sw), sz(padh),
                           sz(padw))
    return st, res


def maxpool_backward(x, dout, N, C, H, W, ph, pw, sh, sw, padh, padw):
    return _pool_backward("maxpool_backward", x, dout, N, C, H, W, ph, pw, sh, sw, padh, padw)


def avgpool_backward(x, dout, N, C, H, W, ph, pw, sh, sw, padh, padw):
    return _pool_backward("avgpool_backward", x, dout, N, C, H, W, ph, pw, sh, sw, padh, padw)


def conv2d_backward_data(filt, dy, N, C, H, W, F, Hf, Wf, sh, sw, padh, padw):
    dX = np.empty((N, C * H * W), filt.dtype)
    st = _f("conv2d_backward_data", filt.dtype)(_p(dX), _p(filt), _p(dy), sz(N), sz(C), sz(H), sz(W), sz(F), sz(Hf), sz(Wf),
                                                sz(sh), sz(sw), sz(padh), sz(padw))
    return st, dX


def conv2d_backward_filter(x, dy, N, C, H, W, F, Hf, Wf, sh, sw, padh, padw):
    dW = np.empty((F, C * Hf * Wf), x.dtype)
    st = _f("conv2d_backward_filter", x.dtype)(_p(dW), _p(x), _p(dy), sz(N), sz(C), sz(H), sz(W), sz(F), sz(Hf), sz(Wf),
                                               sz(sh), sz(sw), sz(padh), sz(padw))
    return st, dW
