"""Host-side builder for the fused vectorized pipeline (dh_vectorized_pipeline_*).

Mirrors what the reference's compiler does when it outlines the body of a VectorizedPipelineOp
(src/compiler/lowering/LowerToLLVMPass.cpp:654-726) and hands it to
VectorizedPipeline<DenseMatrix<VT>>::apply (src/runtime/local/kernels/VectorizedPipeline.h:35-69):
the body is a chain of row-split operators; here it is recorded as an instruction list and run as
one device kernel. Only marshalling happens in Python.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Union

import numpy as np

from . import capi
from .kernels import AggOpCode, DenseMatrix, HIPContext

MAX_INSTR = 16
MAX_OPERANDS = 4

KIND_EW_BINARY, KIND_EW_UNARY, KIND_ROW_AGG, KIND_STORE_TILE, KIND_STORE_ROW, KIND_STORE_ROW_IDX, KIND_REDUCE_ALL = range(7)
OPD_SCALAR, OPD_SELF, OPD_ROWVEC, OPD_COLVEC, OPD_MATRIX, OPD_ROWREG = range(6)


class PipeInstr(C.Structure):
    _fields_ = [("kind", C.c_int32), ("op", C.c_int32), ("domain", C.c_int32), ("operand", C.c_int32),
                ("index", C.c_int32), ("swap", C.c_int32), ("scalar", C.c_double)]


class PipeIO(C.Structure):
    _fields_ = [
        ("x", C.c_void_p), ("ld_x", C.c_size_t),
        ("matrix", C.c_void_p * MAX_OPERANDS), ("ld_matrix", C.c_size_t * MAX_OPERANDS),
        ("rowvec", C.c_void_p * MAX_OPERANDS),
        ("colvec", C.c_void_p * MAX_OPERANDS), ("ld_colvec", C.c_size_t * MAX_OPERANDS),
        ("out_tile", C.c_void_p * MAX_OPERANDS), ("ld_out_tile", C.c_size_t * MAX_OPERANDS),
        ("out_row", C.c_void_p * MAX_OPERANDS), ("ld_out_row", C.c_size_t * MAX_OPERANDS),
        ("out_all", C.c_void_p * 2),
    ]


SELF = "self"
ROWREG = "rowreg"


class VectorizedPipeline:
    """Records a pipeline body over the rows of ``x`` and runs it fused on the device."""

    def __init__(self, ctx: HIPContext, x: DenseMatrix):
        if x.dtype not in (np.dtype(np.float32), np.dtype(np.float64)):
            raise capi.DaphneHipError(1, "vectorizedPipeline: unsupported value type")
        self.ctx, self.x = ctx, x
        self.instrs: list[PipeInstr] = []
        self.io = PipeIO()
        self.io.x, self.io.ld_x = x.ptr, x.row_skip
        self._n = {"matrix": 0, "rowvec": 0, "colvec": 0, "out_tile": 0, "out_row": 0, "out_all": 0}
        self._keep: list = [x]
        self._scalars: list[DenseMatrix] = []
        self.domain = 0
        self._call = None

    def _slot(self, what: str, limit: int = MAX_OPERANDS) -> int:
        i = self._n[what]
        if i >= limit:
            raise capi.DaphneHipError(1, f"vectorizedPipeline: more than {limit} {what} slots")
        self._n[what] = i + 1
        return i

    def _push(self, **kw) -> None:
        if len(self.instrs) >= MAX_INSTR:
            raise capi.DaphneHipError(1, f"vectorizedPipeline: more than {MAX_INSTR} instructions")
        self.instrs.append(PipeInstr(**kw))
        self._call = None

    # -- operators --------------------------------------------------------------------------
    def ewBinary(self, op, operand: Union[float, str, DenseMatrix], swap: bool = False) -> "VectorizedPipeline":
        kw = dict(kind=KIND_EW_BINARY, op=int(op), domain=self.domain, swap=int(swap))
        if isinstance(operand, DenseMatrix):
            m = operand
            if m.dtype != self.x.dtype:
                raise capi.DaphneHipError(1, "vectorizedPipeline: mixed value types")
            self._keep.append(m)
            if m.rows == self.x.rows and m.cols == self.x.cols and self.domain == 0:
                i = self._slot("matrix")
                self.io.matrix[i], self.io.ld_matrix[i] = m.ptr, m.row_skip
                kw.update(operand=OPD_MATRIX, index=i)
            elif m.rows == 1 and m.cols == self.x.cols and self.domain == 0:
                i = self._slot("rowvec")
                self.io.rowvec[i] = m.ptr
                kw.update(operand=OPD_ROWVEC, index=i)
            elif m.rows == self.x.rows and m.cols == 1:
                i = self._slot("colvec")
                self.io.colvec[i], self.io.ld_colvec[i] = m.ptr, m.row_skip
                kw.update(operand=OPD_COLVEC, index=i)
            else:
                raise capi.DaphneHipError(1, "EwBinaryMat(Dense) - lhs and rhs must either have the same dimensions, or "
                                             "one of them must be a row/column vector with the width/height of the other")
        elif operand == SELF:
            kw.update(operand=OPD_SELF)
        elif operand == ROWREG:
            kw.update(operand=OPD_ROWREG)
        else:
            kw.update(operand=OPD_SCALAR, scalar=float(operand))
        self._push(**kw)
        return self

    def ewUnary(self, op) -> "VectorizedPipeline":
        self._push(kind=KIND_EW_UNARY, op=int(op), domain=self.domain)
        return self

    def rowAgg(self, op) -> "VectorizedPipeline":
        """r = agg(t); following elementwise instructions work on r until toTile()."""
        self._push(kind=KIND_ROW_AGG, op=int(op))
        self.domain = 1
        return self

    def toTile(self) -> "VectorizedPipeline":
        self.domain = 0
        return self

    # -- outputs ----------------------------------------------------------------------------
    def storeTile(self, res: Optional[DenseMatrix] = None) -> DenseMatrix:
        if res is None:
            res = DenseMatrix(self.ctx, self.x.rows, self.x.cols, self.x.dtype)
        i = self._slot("out_tile")
        self.io.out_tile[i], self.io.ld_out_tile[i] = res.ptr, res.row_skip
        self._keep.append(res)
        self._push(kind=KIND_STORE_TILE, index=i)
        return res

    def storeRow(self, res: Optional[DenseMatrix] = None, as_index: bool = False) -> DenseMatrix:
        if res is None:
            res = DenseMatrix(self.ctx, self.x.rows, 1, np.uint64 if as_index else self.x.dtype)
        i = self._slot("out_row")
        self.io.out_row[i], self.io.ld_out_row[i] = res.ptr, res.row_skip
        self._keep.append(res)
        self._push(kind=KIND_STORE_ROW_IDX if as_index else KIND_STORE_ROW, index=i)
        return res

    def reduceAll(self, op) -> DenseMatrix:
        """Combine r (after rowAgg) or every item of t over all rows; returns a 1x1 device matrix."""
        i = self._slot("out_all", 2)
        res = DenseMatrix(self.ctx, 1, 1, self.x.dtype)
        self.io.out_all[i] = res.ptr
        self._keep.append(res)
        self._push(kind=KIND_REDUCE_ALL, op=int(op), domain=self.domain, index=i)
        return res

    def run(self) -> None:
        # the marshalled call is built once per recorded body (recording an operator drops it)
        call = self._call
        if call is None or call[0] != len(self.instrs):
            arr = (PipeInstr * max(1, len(self.instrs)))(*self.instrs)
            suf = "f32" if self.x.dtype == np.float32 else "f64"
            fn = getattr(capi.lib(), f"dh_vectorized_pipeline_{suf}")
            fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_size_t, C.c_size_t]
            call = self._call = (len(self.instrs), fn, arr, C.cast(arr, C.c_void_p), C.cast(C.pointer(self.io), C.c_void_p))
        _, fn, _, arr_p, io_p = call
        capi.check(fn(self.ctx._h, arr_p, len(self.instrs), io_p, self.x.rows, self.x.cols))
