"""Python mirror of the reference's kernel interface for the device path.

Function names, argument order and error behaviour follow the reference's kernel convenience
functions (``ewBinaryMat(opCode, res, lhs, rhs, ctx)``, ``aggRow(opCode, res, arg, ctx)``,
``matMul(res, lhs, rhs, transa, transb, ctx)`` ...; reference: src/runtime/local/kernels/*.h and
src/runtime/local/kernels/CUDA/*.h). ``res=None`` makes the kernel allocate the result, a
``DenseMatrix`` passed as ``res`` is written in place - like ``DT *&res`` in the reference.

Everything here only marshals pointers and shapes into the C ABI of libdaphne_hip.so; all
arithmetic happens in the HIP kernels. There is no CPU fallback.
"""
from __future__ import annotations

import ctypes as C
import enum
from typing import Optional

import numpy as np

from . import capi


class BinaryOpCode(enum.IntEnum):  # runtime/local/kernels/BinaryOpCode.h:29-55
    ADD = 0; SUB = 1; MUL = 2; DIV = 3; POW = 4; MOD = 5; LOG = 6; EQ = 7; NEQ = 8; LT = 9; LE = 10
    GT = 11; GE = 12; MIN = 13; MAX = 14; AND = 15; OR = 16; BITWISE_AND = 17; CONCAT = 18


class UnaryOpCode(enum.IntEnum):  # runtime/local/kernels/UnaryOpCode.h:28-55
    MINUS = 0; ABS = 1; SIGN = 2; SQRT = 3; EXP = 4; LN = 5; SIN = 6; COS = 7; TAN = 8; ASIN = 9
    ACOS = 10; ATAN = 11; SINH = 12; COSH = 13; TANH = 14; FLOOR = 15; CEIL = 16; ROUND = 17
    ISNAN = 18; UPPER = 19; LOWER = 20


class AggOpCode(enum.IntEnum):  # runtime/local/kernels/AggOpCode.h:25-35
    SUM = 0; PROD = 1; MIN = 2; MAX = 3; IDXMIN = 4; IDXMAX = 5; MEAN = 6; STDDEV = 7; VAR = 8


_SUFFIX = {np.dtype(np.float32): "f32", np.dtype(np.float64): "f64", np.dtype(np.int64): "si64",
           np.dtype(np.uint64): "ui64", np.dtype(np.int32): "si32", np.dtype(np.uint32): "ui32"}
_CTYPE = {np.dtype(np.float32): C.c_float, np.dtype(np.float64): C.c_double, np.dtype(np.int64): C.c_int64,
          np.dtype(np.uint64): C.c_uint64, np.dtype(np.int32): C.c_int32, np.dtype(np.uint32): C.c_uint32}


class HIPContext:
    """Device context + allocator; the counterpart of the reference's CUDAContext
    (src/runtime/local/context/CUDAContext.h:29-114)."""

    def __init__(self, device: int = 0):
        self._h = C.c_void_p()
        capi.check(capi.lib().dh_ctx_create(device, C.byref(self._h)))

    # CUDAContext::getMemBudget
    def getMemBudget(self) -> int:
        return capi.lib().dh_ctx_mem_budget(self._h)

    def memInUse(self) -> int:
        return capi.lib().dh_ctx_mem_in_use(self._h)

    def memCached(self) -> int:
        return capi.lib().dh_ctx_mem_cached(self._h)

    def releaseCached(self) -> None:
        capi.check(capi.lib().dh_ctx_release_cached(self._h))

    def props(self) -> dict:
        cus, khz, total = C.c_int(), C.c_int(), C.c_size_t()
        name = C.create_string_buffer(256)
        capi.check(capi.lib().dh_ctx_props(self._h, C.byref(cus), C.byref(khz), C.byref(total), name, 256))
        return {"compute_units": cus.value, "clock_khz": khz.value, "total_mem": total.value,
                "name": name.value.decode()}

    def malloc(self, nbytes: int, zero: bool = False) -> int:
        p = C.c_void_p()
        capi.check(capi.lib().dh_malloc(self._h, nbytes, int(zero), C.byref(p)))
        return p.value or 0

    def free(self, ptr: int) -> None:
        capi.check(capi.lib().dh_free(self._h, ptr))

    def set_stream(self, stream_handle: int) -> None:
        capi.check(capi.lib().dh_ctx_set_stream(self._h, stream_handle))

    def sync(self) -> None:
        capi.check(capi.lib().dh_sync(self._h))

    def deferred_checks(self):
        """Context manager: inside it, kernels that validate their arguments on the device (integer DIV / MOD,
        SQRT / LN / ASIN / ACOS, ExtractCol positions) do not wait for their verdict; the first failure is raised
        when the block ends (or by check_deferred() inside it)."""
        ctx = self

        class _Deferred:
            def __enter__(self_inner):
                capi.check(capi.lib().dh_defer_checks(ctx._h, 1))
                return ctx

            def __exit__(self_inner, exc_type, exc, tb):
                capi.check(capi.lib().dh_defer_checks(ctx._h, 0))
                if exc_type is None:
                    ctx.check_deferred()
                else:  # do not let a pending verdict leak into later calls
                    capi.lib().dh_check_deferred(ctx._h)
                return False

        return _Deferred()

    def check_deferred(self) -> None:
        capi.check(capi.lib().dh_check_deferred(self._h))

    def set_pipeline_mode(self, mode: int) -> None:
        """1: fused pipeline bodies are specialised at run time, 0: interpreted, -1: as the environment says."""
        capi.check(capi.lib().dh_ctx_set_pipeline_mode(self._h, mode))

    def timer_start(self) -> None:
        capi.check(capi.lib().dh_timer_start(self._h))

    def timer_stop_ms(self) -> float:
        ms = C.c_float()
        capi.check(capi.lib().dh_timer_stop_ms(self._h, C.byref(ms)))
        return ms.value

    def kernel_timing(self, on: bool) -> None:
        """Switches the stopwatch on single kernels on or off (dh_kernel_timing): while it is on, a fused pipeline
        records the duration of its body kernel alone."""
        capi.check(capi.lib().dh_kernel_timing(self._h, 1 if on else 0))

    def kernel_timing_read(self):
        """(sum of the timed kernels' durations in ms, their number) since the stopwatch was switched on or last read."""
        total, n = C.c_double(), C.c_size_t()
        capi.check(capi.lib().dh_kernel_timing_read(self._h, C.byref(total), C.byref(n)))
        return total.value, n.value

    def destroy(self) -> None:
        if self._h:
            capi.lib().dh_ctx_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class DenseMatrix:
    """Row-major dense matrix resident in device memory: pointer, numRows, numCols, rowSkip
    (reference: src/runtime/local/datastructures/DenseMatrix.h:42-56). Views share the buffer."""

    def __init__(self, ctx: HIPContext, rows: int, cols: int, dtype, ptr: Optional[int] = None,
                 row_skip: Optional[int] = None, zero: bool = False, keepalive=None):
        self.ctx = ctx
        self.rows, self.cols = int(rows), int(cols)
        self.dtype = np.dtype(dtype)
        self.row_skip = int(row_skip if row_skip is not None else cols)
        self._owned = ptr is None
        self._keepalive = keepalive
        if ptr is None:
            ptr = ctx.malloc(max(1, self.rows * self.row_skip) * self.dtype.itemsize, zero)
        self.ptr = ptr

    # -- construction -------------------------------------------------------------------
    @staticmethod
    def from_numpy(ctx: HIPContext, a) -> "DenseMatrix":
        a = np.ascontiguousarray(a)
        if a.ndim == 1:
            a = a.reshape(-1, 1)
        m = DenseMatrix(ctx, a.shape[0], a.shape[1], a.dtype)
        if a.size:
            capi.check(capi.lib().dh_h2d(ctx._h, m.ptr, a.ctypes.data, a.nbytes))
        return m

    @staticmethod
    def from_torch(ctx: HIPContext, t) -> "DenseMatrix":
        """Wraps a 2-D row-major torch tensor already resident on the device (no copy)."""
        import torch

        assert t.is_cuda and t.dim() == 2 and t.stride(1) == 1
        dt = {torch.float32: np.float32, torch.float64: np.float64, torch.int64: np.int64,
              torch.uint64: np.uint64, torch.int32: np.int32, torch.uint32: np.uint32}[t.dtype]
        return DenseMatrix(ctx, t.shape[0], t.shape[1], dt, ptr=t.data_ptr(), row_skip=t.stride(0) if t.shape[0] > 1 else t.shape[1],
                           keepalive=t)

    # -- reference accessors --------------------------------------------------------------
    def getNumRows(self) -> int:
        return self.rows

    def getNumCols(self) -> int:
        return self.cols

    def getRowSkip(self) -> int:
        return self.row_skip

    def getNumItems(self) -> int:
        return self.rows * self.cols

    def to_numpy(self) -> np.ndarray:
        buf = np.empty((self.rows, self.row_skip), dtype=self.dtype)
        if buf.size:
            n = ((self.rows - 1) * self.row_skip + self.cols) * self.dtype.itemsize
            capi.check(capi.lib().dh_d2h(self.ctx._h, buf.ctypes.data, self.ptr, n))
        return np.ascontiguousarray(buf[:, : self.cols])

    def slice(self, r0: int, r1: int, c0: int = 0, c1: Optional[int] = None) -> "DenseMatrix":
        """View of rows [r0, r1) and columns [c0, c1) (DenseMatrix::slice of the reference)."""
        c1 = self.cols if c1 is None else c1
        off = (r0 * self.row_skip + c0) * self.dtype.itemsize
        return DenseMatrix(self.ctx, r1 - r0, c1 - c0, self.dtype, ptr=self.ptr + off, row_skip=self.row_skip,
                           keepalive=self)

    def destroy(self) -> None:
        if self._owned and self.ptr:
            self.ctx.free(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            if self._owned and self.ptr and self.ctx._h:
                self.destroy()
        except Exception:
            pass


def _fn(name: str, dtype):
    try:
        suf = _SUFFIX[np.dtype(dtype)]
    except KeyError:
        raise capi.DaphneHipError(capi.DH_ERR_RUNTIME, f"{name}: unsupported value type {dtype}")
    fn = getattr(capi.lib(), f"{name}_{suf}", None)
    if fn is None:  # e.g. MatMul or the unary operators on integers: not instantiated, as in the reference
        raise capi.DaphneHipError(capi.DH_ERR_RUNTIME, f"{name}: not instantiated for the value type {np.dtype(dtype)}")
    return fn


def _same_dtype(*ms):
    d = ms[0].dtype
    for m in ms[1:]:
        if m is not None and m.dtype != d:
            raise capi.DaphneHipError(capi.DH_ERR_RUNTIME, "mixed value types are not instantiated for the device kernels")
    return d


# ------------------------------------------------------------------------------------------
# elementwise
# ------------------------------------------------------------------------------------------
def ewBinaryMat(opCode, res, lhs: DenseMatrix, rhs: DenseMatrix, ctx: HIPContext) -> DenseMatrix:
    """CUDA::ewBinaryMat (kernels/CUDA/EwBinaryMat.h:40-47)."""
    dt = _same_dtype(lhs, rhs, res)
    if res is None:
        res = DenseMatrix(ctx, lhs.rows, lhs.cols, dt)
    capi.check(_fn("dh_ew_binary", dt)(ctx._h, int(opCode), res.ptr, res.row_skip, lhs.ptr, lhs.rows, lhs.cols,
                                       lhs.row_skip, rhs.ptr, rhs.rows, rhs.cols, rhs.row_skip))
    return res


def ewBinaryObjSca(opCode, res, lhs: DenseMatrix, rhs: float, ctx: HIPContext) -> DenseMatrix:
    """CUDA::ewBinaryObjSca (kernels/CUDA/EwBinaryObjSca.h:52-60)."""
    dt = _same_dtype(lhs, res)
    if res is None:
        res = DenseMatrix(ctx, lhs.rows, lhs.cols, dt)
    capi.check(_fn("dh_ew_binary_sca", dt)(ctx._h, int(opCode), res.ptr, res.row_skip, lhs.ptr, lhs.rows, lhs.cols,
                                           lhs.row_skip, rhs if dt.kind in "iu" else float(rhs)))
    return res


def ewUnaryMat(opCode, res, arg: DenseMatrix, ctx: HIPContext) -> DenseMatrix:
    """ewUnaryMat (kernels/EwUnaryMat.h:43-45)."""
    dt = _same_dtype(arg, res)
    if res is None:
        res = DenseMatrix(ctx, arg.rows, arg.cols, dt)
    capi.check(_fn("dh_ew_unary", dt)(ctx._h, int(opCode), res.ptr, res.row_skip, arg.ptr, arg.rows, arg.cols,
                                      arg.row_skip))
    return res


# ------------------------------------------------------------------------------------------
# aggregations
# ------------------------------------------------------------------------------------------
def aggAll(opCode, arg: DenseMatrix, ctx: HIPContext) -> float:
    """CUDA::aggAll (kernels/CUDA/AggAll.h:44-50): returns the scalar."""
    out = _CTYPE[arg.dtype]()
    capi.check(_fn("dh_agg_all", arg.dtype)(ctx._h, int(opCode), arg.ptr, arg.rows, arg.cols, arg.row_skip,
                                            C.byref(out)))
    return arg.dtype.type(out.value)


def aggRow(opCode, res, arg: DenseMatrix, ctx: HIPContext) -> DenseMatrix:
    """CUDA::aggRow (kernels/CUDA/AggRow.h:46-52); IDXMIN / IDXMAX give a DenseMatrix<size_t>
    (kernels/AggRow.h:71-94)."""
    if int(opCode) in (AggOpCode.IDXMIN, AggOpCode.IDXMAX):
        if res is None:
            res = DenseMatrix(ctx, arg.rows, 1, np.uint64)
        capi.check(_fn("dh_agg_row_idx", arg.dtype)(ctx._h, int(opCode), res.ptr, res.row_skip, arg.ptr, arg.rows,
                                                    arg.cols, arg.row_skip))
        return res
    if res is None:
        res = DenseMatrix(ctx, arg.rows, 1, arg.dtype)
    capi.check(_fn("dh_agg_row", arg.dtype)(ctx._h, int(opCode), res.ptr, res.row_skip, arg.ptr, arg.rows, arg.cols,
                                            arg.row_skip))
    return res


def aggCol(opCode, res, arg: DenseMatrix, ctx: HIPContext) -> DenseMatrix:
    """CUDA::aggCol (kernels/CUDA/AggCol.h:46-52)."""
    if int(opCode) in (AggOpCode.IDXMIN, AggOpCode.IDXMAX):
        if res is None:
            res = DenseMatrix(ctx, 1, arg.cols, np.uint64)
        capi.check(_fn("dh_agg_col_idx", arg.dtype)(ctx._h, int(opCode), res.ptr, arg.ptr, arg.rows, arg.cols,
                                                    arg.row_skip))
        return res
    if res is None:
        res = DenseMatrix(ctx, 1, arg.cols, arg.dtype)
    capi.check(_fn("dh_agg_col", arg.dtype)(ctx._h, int(opCode), res.ptr, arg.ptr, arg.rows, arg.cols, arg.row_skip))
    return res


def aggColMoments(arg: DenseMatrix, ctx: HIPContext, stddev: bool = False, res_mean=None, res_var=None):
    """aggCol(MEAN) and aggCol(VAR | STDDEV) of the same matrix from one pass over it. Returns (mean, var)."""
    if res_mean is None:
        res_mean = DenseMatrix(ctx, 1, arg.cols, arg.dtype)
    if res_var is None:
        res_var = DenseMatrix(ctx, 1, arg.cols, arg.dtype)
    capi.check(_fn("dh_agg_col_moments", arg.dtype)(ctx._h, res_mean.ptr, res_var.ptr, int(stddev), arg.ptr, arg.rows,
                                                    arg.cols, arg.row_skip))
    return res_mean, res_var


# ------------------------------------------------------------------------------------------
# contractions
# ------------------------------------------------------------------------------------------
def matMul(res, lhs: DenseMatrix, rhs: DenseMatrix, transa: bool, transb: bool, ctx: HIPContext) -> DenseMatrix:
    """CUDA::matMul (kernels/CUDA/MatMul.h:45-51)."""
    dt = _same_dtype(lhs, rhs, res)
    nr1 = lhs.cols if transa else lhs.rows
    nc2 = rhs.rows if transb else rhs.cols
    if res is None:
        res = DenseMatrix(ctx, nr1, nc2, dt)
    capi.check(_fn("dh_matmul", dt)(ctx._h, res.ptr, res.row_skip, lhs.ptr, lhs.rows, lhs.cols, lhs.row_skip,
                                    rhs.ptr, rhs.rows, rhs.cols, rhs.row_skip, int(transa), int(transb)))
    return res


def syrk(res, arg: DenseMatrix, transLeft: bool, ctx: HIPContext) -> DenseMatrix:
    """syrk (kernels/Syrk.h:38-40; device version kernels/CUDA/Syrk.h:40-46)."""
    n = arg.cols if transLeft else arg.rows
    if res is None:
        res = DenseMatrix(ctx, n, n, arg.dtype)
    capi.check(_fn("dh_syrk", arg.dtype)(ctx._h, res.ptr, res.row_skip, arg.ptr, arg.rows, arg.cols, arg.row_skip,
                                         int(transLeft)))
    return res


def normalEquations(X: DenseMatrix, y: DenseMatrix, lam: float, ctx: HIPContext, A: Optional[DenseMatrix] = None,
                    b: Optional[DenseMatrix] = None):
    """A = t(X) X + lam I and b = t(X) y from one pass over X (dh_normal_equations_*): the operator sequence
    syrk + ewMul + ewAdd + matMul of scripts/algorithms/lmDS_.daph:60-75. Returns (A, b)."""
    dt = _same_dtype(X, y, A)
    if y.rows != X.rows or y.cols != 1:
        raise capi.DaphneHipError(1, "normalEquations: y must be a column vector with as many rows as X")
    if A is None:
        A = DenseMatrix(ctx, X.cols, X.cols, dt)
    if b is None:
        b = DenseMatrix(ctx, X.cols, 1, dt)
    capi.check(_fn("dh_normal_equations", dt)(ctx._h, A.ptr, A.row_skip, b.ptr, b.row_skip, X.ptr, X.rows, X.cols, X.row_skip,
                                              y.ptr, y.row_skip, lam))
    return A, b


def kmeansAssign(idx, X: DenseMatrix, C: DenseMatrix, xx: DenseMatrix, cc: DenseMatrix, ctx: HIPContext) -> DenseMatrix:
    """idx = idxminRow((X @ t(C)) * -2 + xx + t(cc)) in one pass over X (dh_kmeans_assign_*): the operator sequence
    MatMul, EwBinaryObjSca MUL, EwBinaryMat ADD twice, AggRow IDXMIN of test/api/cli/algorithms/kmeans.daphne:14-16.
    xx holds one value per row of X, cc one per row of C; idx is rows x 1, uint64."""
    dt = _same_dtype(X, C, xx, cc)
    if C.cols != X.cols or xx.getNumItems() != X.rows or cc.getNumItems() != C.rows:
        raise capi.DaphneHipError(1, "kmeansAssign: C must have X's columns, xx one value per row of X, cc one per centroid")
    if idx is None:
        idx = DenseMatrix(ctx, X.rows, 1, np.uint64)
    capi.check(_fn("dh_kmeans_assign", dt)(ctx._h, idx.ptr, X.ptr, X.rows, X.cols, X.row_skip, C.ptr, C.rows, C.row_skip, xx.ptr,
                                           cc.ptr))
    return idx


def kmeansUpdate(C_new, X: DenseMatrix, idx: DenseMatrix, k: int, ctx: HIPContext, counts: Optional[DenseMatrix] = None):
    """C_new = (t(P) @ X) / t(colSums(P)) for P = one-hot(idx), in one pass over X (dh_kmeans_update_*): the comparison,
    MatMul, AggCol SUM and EwBinaryMat DIV of test/api/cli/algorithms/kmeans.daphne:17-21. Returns (C_new, counts)."""
    dt = X.dtype
    if idx.getNumItems() != X.rows:
        raise capi.DaphneHipError(1, "kmeansUpdate: idx must hold one value per row of X")
    if C_new is None:
        C_new = DenseMatrix(ctx, k, X.cols, dt)
    if counts is None:
        counts = DenseMatrix(ctx, 1, k, dt)
    capi.check(_fn("dh_kmeans_update", dt)(ctx._h, C_new.ptr, C_new.row_skip, counts.ptr, X.ptr, X.rows, X.cols, X.row_skip, idx.ptr, k))
    return C_new, counts


def kmeansStep(idx, C_new, X: DenseMatrix, C: DenseMatrix, xx: DenseMatrix, cc: DenseMatrix, ctx: HIPContext,
               counts: Optional[DenseMatrix] = None):
    """kmeansAssign and kmeansUpdate as one call (dh_kmeans_step_*): one pass over X where the library has a kernel for
    it (up to 64 features, in double up to 16 centroids), the two passes elsewhere. Returns (idx, C_new, counts)."""
    dt = _same_dtype(X, C, xx, cc)
    k = C.rows
    if C.cols != X.cols or xx.getNumItems() != X.rows or cc.getNumItems() != k:
        raise capi.DaphneHipError(1, "kmeansStep: C must have X's columns, xx one value per row of X, cc one per centroid")
    if idx is None:
        idx = DenseMatrix(ctx, X.rows, 1, np.uint64)
    if C_new is None:
        C_new = DenseMatrix(ctx, k, X.cols, dt)
    if counts is None:
        counts = DenseMatrix(ctx, 1, k, dt)
    capi.check(_fn("dh_kmeans_step", dt)(ctx._h, idx.ptr, C_new.ptr, C_new.row_skip, counts.ptr, X.ptr, X.rows, X.cols, X.row_skip,
                                         C.ptr, k, C.row_skip, xx.ptr, cc.ptr))
    return idx, C_new, counts


def solve(res, lhs: DenseMatrix, rhs: DenseMatrix, ctx: HIPContext) -> DenseMatrix:
    """CUDA::solve (kernels/CUDA/Solve.h; CPU kernels/Solve.h:86-116): A x = b by LU."""
    dt = _same_dtype(lhs, rhs, res)
    if lhs.rows != rhs.rows:
        raise capi.DaphneHipError(1, "#rows of lhs and #rows of rhs must be the same")
    if lhs.rows != lhs.cols:
        raise capi.DaphneHipError(1, "#rows and #cols of lhs must be the same")
    if lhs.row_skip != lhs.cols:
        raise capi.DaphneHipError(1, "#cols of lhs must match row skip")
    if rhs.cols != 1:
        raise capi.DaphneHipError(1, "#cols of rhs must be 1")
    if res is None:
        res = DenseMatrix(ctx, lhs.rows, 1, dt)
    capi.check(_fn("dh_solve", dt)(ctx._h, res.ptr, lhs.ptr, lhs.rows, lhs.row_skip, rhs.ptr))
    return res


# ------------------------------------------------------------------------------------------
# DNN
# ------------------------------------------------------------------------------------------
def conv2dForward(res, data: DenseMatrix, filter: DenseMatrix, bias, batch_size, num_channels, img_h, img_w,
                  filter_h, filter_w, stride_h, stride_w, pad_h, pad_w, ctx: HIPContext):
    """CUDA::Convolution::Forward::apply (kernels/CUDA/Convolution.h:33-38). Returns
    (res, res_h, res_w)."""
    dt = _same_dtype(data, filter, bias, res)
    F = filter.rows
    P = (img_h + 2 * pad_h - filter_h) // stride_h + 1 if img_h + 2 * pad_h >= filter_h else 0
    Q = (img_w + 2 * pad_w - filter_w) // stride_w + 1 if img_w + 2 * pad_w >= filter_w else 0
    if res is None:
        res = DenseMatrix(ctx, batch_size, F * P * Q, dt)
    rh, rw = C.c_size_t(), C.c_size_t()
    capi.check(_fn("dh_conv2d_forward", dt)(ctx._h, res.ptr, C.byref(rh), C.byref(rw), data.ptr, filter.ptr,
                                            filter.rows, filter.cols, bias.ptr if bias is not None else None,
                                            batch_size, num_channels, img_h, img_w, filter_h, filter_w, stride_h,
                                            stride_w, pad_h, pad_w))
    return res, rh.value, rw.value


EPILOGUE_RELU, EPILOGUE_MAXPOOL_2X2 = 1, 2  # enum dh_epilogue


def conv2dForwardFused(res, data: DenseMatrix, filter: DenseMatrix, bias, batch_size, num_channels, img_h, img_w,
                       filter_h, filter_w, stride_h, stride_w, pad_h, pad_w, ctx: HIPContext, relu=True, pool=False):
    """conv2dForward with reluForward and / or maxPoolForward (2 x 2 window, stride 2, no padding) folded into the
    store (dh_conv2d_forward_fused_*): the results of the separate kernels, bit for bit. Returns (res, res_h, res_w),
    the extents being the pooled ones with pool=True."""
    dt = _same_dtype(data, filter, bias, res)
    F = filter.rows
    P = (img_h + 2 * pad_h - filter_h) // stride_h + 1 if img_h + 2 * pad_h >= filter_h else 0
    Q = (img_w + 2 * pad_w - filter_w) // stride_w + 1 if img_w + 2 * pad_w >= filter_w else 0
    if pool:
        P, Q = ((P - 2) // 2 + 1 if P >= 2 else 0), ((Q - 2) // 2 + 1 if Q >= 2 else 0)
    if res is None:
        res = DenseMatrix(ctx, batch_size, F * P * Q, dt)
    rh, rw = C.c_size_t(), C.c_size_t()
    flags = (EPILOGUE_RELU if relu else 0) | (EPILOGUE_MAXPOOL_2X2 if pool else 0)
    capi.check(_fn("dh_conv2d_forward_fused", dt)(ctx._h, res.ptr, C.byref(rh), C.byref(rw), data.ptr, filter.ptr,
                                                  filter.rows, filter.cols, bias.ptr if bias is not None else None,
                                                  batch_size, num_channels, img_h, img_w, filter_h, filter_w, stride_h,
                                                  stride_w, pad_h, pad_w, flags))
    return res, rh.value, rw.value


def maxPoolForward(res, data: DenseMatrix, batch_size, num_channels, img_h, img_w, pool_h, pool_w, stride_h,
                   stride_w, pad_h, pad_w, ctx: HIPContext):
    """CUDA::NN::Pooling::Forward<MAX>::apply (kernels/CUDA/Pooling.h:31-35; CPU
    kernels/MaxPoolForward.h:35-44). Returns (res, res_h, res_w)."""
    dt = data.dtype
    P = (img_h + 2 * pad_h - pool_h) // stride_w + 1 if img_h + 2 * pad_h >= pool_h else 0
    Q = (img_w + 2 * pad_w - pool_w) // stride_h + 1 if img_w + 2 * pad_w >= pool_w else 0
    if res is None:
        res = DenseMatrix(ctx, batch_size, num_channels * P * Q, dt)
    rh, rw = C.c_size_t(), C.c_size_t()
    capi.check(_fn("dh_maxpool_forward", dt)(ctx._h, res.ptr, C.byref(rh), C.byref(rw), data.ptr, batch_size,
                                             num_channels, img_h, img_w, pool_h, pool_w, stride_h, stride_w, pad_h,
                                             pad_w))
    return res, rh.value, rw.value


def affineForward(res, data: DenseMatrix, weights: DenseMatrix, bias, ctx: HIPContext) -> DenseMatrix:
    """CUDA::NN::Affine::Forward::apply (kernels/CUDA/Affine.h:24-26)."""
    dt = _same_dtype(data, weights, bias, res)
    if res is None:
        res = DenseMatrix(ctx, data.rows, weights.cols, dt)
    capi.check(_fn("dh_affine_forward", dt)(ctx._h, res.ptr, data.ptr, data.rows, data.cols, weights.ptr,
                                            weights.rows, weights.cols, bias.ptr if bias is not None else None,
                                            bias.rows if bias is not None else 0,
                                            bias.cols if bias is not None else 0))
    return res


def affineForwardFused(res, data: DenseMatrix, weights: DenseMatrix, bias, ctx: HIPContext, relu=True) -> DenseMatrix:
    """affineForward followed by reluForward in one pass (dh_affine_forward_fused_*), same result bit for bit."""
    dt = _same_dtype(data, weights, bias, res)
    if res is None:
        res = DenseMatrix(ctx, data.rows, weights.cols, dt)
    capi.check(_fn("dh_affine_forward_fused", dt)(ctx._h, res.ptr, data.ptr, data.rows, data.cols, weights.ptr,
                                                  weights.rows, weights.cols, bias.ptr if bias is not None else None,
                                                  bias.rows if bias is not None else 0,
                                                  bias.cols if bias is not None else 0, EPILOGUE_RELU if relu else 0))
    return res


def biasAdd(res, data: DenseMatrix, bias: DenseMatrix, ctx: HIPContext) -> DenseMatrix:
    """CUDA::BiasAdd::apply (kernels/CUDA/BiasAdd.h:26-28; CPU kernels/BiasAdd.h:34-52)."""
    dt = _same_dtype(data, bias, res)
    if res is None:
        res = DenseMatrix(ctx, data.rows, data.cols, dt)
    capi.check(_fn("dh_bias_add", dt)(ctx._h, res.ptr, data.ptr, data.rows, data.cols, bias.ptr, bias.getNumItems()))
    return res


def batchNormInferenceForward(res, data, gamma, beta, ema_mean, ema_var, eps, ctx: HIPContext,
                              stat_index: int = 0) -> DenseMatrix:
    """CUDA::BatchNormInferenceForward::apply (kernels/CUDA/BatchNorm.h:26-29)."""
    dt = _same_dtype(data, gamma, beta, ema_mean, ema_var, res)
    if res is None:
        res = DenseMatrix(ctx, data.rows, data.cols, dt)
    capi.check(_fn("dh_batchnorm_inference", dt)(ctx._h, res.ptr, data.ptr, data.rows, data.cols, gamma.ptr, beta.ptr,
                                                 ema_mean.ptr, ema_var.ptr, gamma.rows, float(eps), stat_index))
    return res


def softmax(res, arg: DenseMatrix, ctx: HIPContext) -> DenseMatrix:
    """CUDA::Softmax::apply (kernels/CUDA/Softmax.h:32-34; CPU kernels/Softmax.h:22-58)."""
    if res is None:
        res = DenseMatrix(ctx, arg.rows, arg.cols, arg.dtype)
    capi.check(_fn("dh_softmax", arg.dtype)(ctx._h, res.ptr, res.row_skip, arg.ptr, arg.rows, arg.cols, arg.row_skip))
    return res


def avgPoolForward(res, data: DenseMatrix, batch_size, num_channels, img_h, img_w, pool_h, pool_w, stride_h,
                   stride_w, pad_h, pad_w, ctx: HIPContext):
    """CUDA::NN::Pooling::Forward<AVG>::apply (kernels/CUDA/Pooling.h:31-35; CPU kernels/AvgPoolForward.h,
    Pooling.cpp:28-107). Returns (res, res_h, res_w)."""
    dt = data.dtype
    P = (img_h + 2 * pad_h - pool_h) // stride_w + 1 if img_h + 2 * pad_h >= pool_h else 0
    Q = (img_w + 2 * pad_w - pool_w) // stride_h + 1 if img_w + 2 * pad_w >= pool_w else 0
    if res is None:
        res = DenseMatrix(ctx, batch_size, num_channels * P * Q, dt)
    rh, rw = C.c_size_t(), C.c_size_t()
    capi.check(_fn("dh_avgpool_forward", dt)(ctx._h, res.ptr, C.byref(rh), C.byref(rw), data.ptr, batch_size,
                                             num_channels, img_h, img_w, pool_h, pool_w, stride_h, stride_w, pad_h,
                                             pad_w))
    return res, rh.value, rw.value


def reluForward(res, data: DenseMatrix, ctx: HIPContext) -> DenseMatrix:
    """CUDA::NN::Activation::Forward<ReLU>::apply (kernels/CUDA/Activation.h:24-33)."""
    if res is None:
        res = DenseMatrix(ctx, data.rows, data.cols, data.dtype)
    capi.check(_fn("dh_relu_forward", data.dtype)(ctx._h, res.ptr, res.row_skip, data.ptr, data.rows, data.cols,
                                                  data.row_skip))
    return res


def fill(res, arg, numRows: int, numCols: int, ctx: HIPContext, dtype=np.float64) -> DenseMatrix:
    """CUDA::Fill::apply (kernels/CUDA/Fill.h:30-47)."""
    if res is None:
        res = DenseMatrix(ctx, numRows, numCols, dtype)
    capi.check(_fn("dh_fill", res.dtype)(ctx._h, res.ptr, res.row_skip, arg, numRows, numCols))
    return res


def colBind(res, lhs: DenseMatrix, rhs: DenseMatrix, ctx: HIPContext) -> DenseMatrix:
    """CUDA::ColBind::apply (kernels/CUDA/ColBind.h:26-34; CPU kernels/ColBind.h:58-91)."""
    dt = _same_dtype(lhs, rhs, res)
    if res is None:
        res = DenseMatrix(ctx, lhs.rows, lhs.cols + rhs.cols, dt)
    capi.check(_fn("dh_col_bind", dt)(ctx._h, res.ptr, res.row_skip, lhs.ptr, lhs.rows, lhs.cols, lhs.row_skip, rhs.ptr,
                                      rhs.rows, rhs.cols, rhs.row_skip))
    return res


def extractCol(res, arg: DenseMatrix, sel: DenseMatrix, ctx: HIPContext) -> DenseMatrix:
    """CUDA::ExtractCol::apply (kernels/CUDA/ExtractCol.h:26-35; CPU kernels/ExtractCol.h:74-114). `sel` is an
    int64 column of positions."""
    if sel.dtype != np.dtype(np.int64):
        raise TypeError("extractCol: positions must be int64")
    if res is None:
        res = DenseMatrix(ctx, arg.rows, sel.rows, arg.dtype)
    capi.check(_fn("dh_extract_col", arg.dtype)(ctx._h, res.ptr, res.row_skip, arg.ptr, arg.rows, arg.cols, arg.row_skip,
                                                sel.ptr, sel.rows, sel.cols, sel.row_skip))
    return res


def transpose(res, arg: DenseMatrix, ctx: HIPContext) -> DenseMatrix:
    """CUDA::Transpose::apply (kernels/CUDA/Transpose.h:33-39; CPU kernels/Transpose.h:51-76)."""
    if res is None:
        res = DenseMatrix(ctx, arg.cols, arg.rows, arg.dtype)
    capi.check(_fn("dh_transpose", arg.dtype)(ctx._h, res.ptr, res.row_skip, arg.ptr, arg.rows, arg.cols, arg.row_skip))
    return res


def gemv(res, mat: DenseMatrix, vec: DenseMatrix, ctx: HIPContext) -> DenseMatrix:
    """CUDA::Gemv::apply (kernels/CUDA/Gemv.h:34-40; CPU kernels/Gemv.h:51-77): res = t(mat) @ vec."""
    dt = _same_dtype(mat, vec, res)
    if res is None:
        res = DenseMatrix(ctx, mat.cols, 1, dt)
    capi.check(_fn("dh_gemv", dt)(ctx._h, res.ptr, res.row_skip, mat.ptr, mat.rows, mat.cols, mat.row_skip, vec.ptr,
                                  vec.rows, vec.row_skip))
    return res


# ------------------------------------------------------------------------------------------
# DNN training kernels
# ------------------------------------------------------------------------------------------
def batchNorm2DTrainForward(in_: DenseMatrix, gamma: DenseMatrix, beta: DenseMatrix, emaMean: DenseMatrix, emaVar: DenseMatrix,
                            eps: float, mu: float, ctx: HIPContext):
    """BatchNorm2DTrainForward::apply (kernels/BatchNorm2DTrainForward.h:66-118). Returns (res, new_emaMean, new_emaVar,
    mean, invVar); the four statistics are C x 1 (the reference returns C x C matrices with the first C values set)."""
    dt = _same_dtype(in_, gamma, beta, emaMean, emaVar)
    C = gamma.rows * gamma.cols
    res = DenseMatrix(ctx, in_.rows, in_.cols, dt)
    outs = [DenseMatrix(ctx, C, 1, dt) for _ in range(4)]
    capi.check(_fn("dh_batchnorm_train_forward", dt)(ctx._h, res.ptr, outs[0].ptr, outs[1].ptr, outs[2].ptr, outs[3].ptr, in_.ptr,
                                                     in_.rows, in_.cols, gamma.ptr, beta.ptr, emaMean.ptr, emaVar.ptr, C, eps, mu))
    return (res, *outs)


def batchNorm2DBackward(mean: DenseMatrix, invVar: DenseMatrix, in_: DenseMatrix, dout: DenseMatrix, gamma: DenseMatrix,
                        eps: float, ctx: HIPContext):
    """BatchNorm2DBackward::apply (kernels/BatchNorm2DBackward.h:63-120). Returns (dX, dGamma, dBeta)."""
    dt = _same_dtype(in_, dout, gamma, mean, invVar)
    C = gamma.rows * gamma.cols
    dX, dG, dB = DenseMatrix(ctx, in_.rows, in_.cols, dt), DenseMatrix(ctx, C, 1, dt), DenseMatrix(ctx, C, 1, dt)
    capi.check(_fn("dh_batchnorm_backward", dt)(ctx._h, dX.ptr, dG.ptr, dB.ptr, mean.ptr, invVar.ptr, in_.ptr, dout.ptr, in_.rows,
                                                in_.cols, gamma.ptr, C, eps))
    return dX, dG, dB


def _poolBackward(name, res, input_, dOut, N, C, H, W, ph, pw, sh, sw, padh, padw, ctx):
    dt = _same_dtype(input_, dOut, res)
    if res is None:
        res = DenseMatrix(ctx, N, C * H * W, dt)
    capi.check(_fn(name, dt)(ctx._h, res.ptr, input_.ptr, dOut.ptr, N, C, H, W, ph, pw, sh, sw, padh, padw))
    return res


def maxPoolBackward(res, input_: DenseMatrix, dOut: DenseMatrix, batch_size, num_channels, img_h, img_w, pool_h, pool_w,
                    stride_h, stride_w, pad_h, pad_w, ctx: HIPContext) -> DenseMatrix:
    """MaxPoolBackward::apply (kernels/MaxPoolBackward.h:35-82), same argument order."""
    return _poolBackward("dh_maxpool_backward", res, input_, dOut, batch_size, num_channels, img_h, img_w, pool_h, pool_w,
                         stride_h, stride_w, pad_h, pad_w, ctx)


def avgPoolBackward(res, input_: DenseMatrix, dOut: DenseMatrix, batch_size, num_channels, img_h, img_w, pool_h, pool_w,
                    stride_h, stride_w, pad_h, pad_w, ctx: HIPContext) -> DenseMatrix:
    """AvgPoolBackward::apply (kernels/AvgPoolBackward.h:35-77), same argument order."""
    return _poolBackward("dh_avgpool_backward", res, input_, dOut, batch_size, num_channels, img_h, img_w, pool_h, pool_w,
                         stride_h, stride_w, pad_h, pad_w, ctx)


def conv2DBackwardData(filter_: DenseMatrix, output: DenseMatrix, stride_h, stride_w, pad_h, pad_w, input_batch_size,
                       input_num_channels, input_h, input_w, filter_num_filters, filter_num_channels, filter_h, filter_w,
                       data, ctx: HIPContext) -> DenseMatrix:
    """Conv2DBackwardData::apply (kernels/Conv2DBackwardData.h:88-100), same argument order (`output` is the gradient
    w.r.t. the convolution's output, `data` the result)."""
    dt = _same_dtype(filter_, output, data)
    if data is None:
        data = DenseMatrix(ctx, input_batch_size, input_num_channels * input_h * input_w, dt)
    capi.check(_fn("dh_conv2d_backward_data", dt)(ctx._h, data.ptr, filter_.ptr, output.ptr, input_batch_size, input_num_channels,
                                                  input_h, input_w, filter_num_filters, filter_h, filter_w, stride_h, stride_w,
                                                  pad_h, pad_w))
    return data


def conv2DBackwardFilter(dFilter, input_: DenseMatrix, output: DenseMatrix, stride_h, stride_w, pad_h, pad_w, input_batch_size,
                         input_num_channels, input_h, input_w, filter_num_filters, filter_num_channels, filter_h, filter_w,
                         ctx: HIPContext) -> DenseMatrix:
    """Conv2DBackwardFilter::apply (kernels/Conv2DBackwardFilter.h:68-76), same argument order."""
    dt = _same_dtype(input_, output, dFilter)
    if dFilter is None:
        dFilter = DenseMatrix(ctx, filter_num_filters, filter_num_channels * filter_h * filter_w, dt)
    capi.check(_fn("dh_conv2d_backward_filter", dt)(ctx._h, dFilter.ptr, input_.ptr, output.ptr, input_batch_size,
                                                    input_num_channels, input_h, input_w, filter_num_filters, filter_h, filter_w,
                                                    stride_h, stride_w, pad_h, pad_w))
    return dFilter
