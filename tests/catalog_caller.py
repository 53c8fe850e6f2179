"""Calls the generated entry points of libHIPKernels.so the way a DAPHNE program does: by the function name the
kernel catalog lists, with pointers to run-time objects, a dispatch id and the DaphneContext last.

The run-time objects (DaphneContext, DenseMatrix<T>) are made and read back through tests/cpp/glue_harness.cpp; the
ctypes signature of each entry point is derived from the parameter list the generator produced it with.
Test infrastructure only.
"""
from __future__ import annotations

import ctypes as C
import importlib.util
import json
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT / "tests"))

SUFFIX = {np.dtype(np.float32): "f32", np.dtype(np.float64): "f64", np.dtype(np.int64): "si64", np.dtype(np.uint64): "ui64",
          np.dtype(np.int32): "si32", np.dtype(np.uint32): "ui32"}
CPP_VT = {"float": np.float32, "double": np.float64, "int64_t": np.int64, "uint64_t": np.uint64, "size_t": np.uint64,
          "int32_t": np.int32, "uint32_t": np.uint32}
SCALAR_CT = {"float": C.c_float, "double": C.c_double, "int64_t": C.c_int64, "uint64_t": C.c_uint64, "size_t": C.c_size_t,
             "int32_t": C.c_int32, "uint32_t": C.c_uint32, "bool": C.c_bool}


def _load_generator():
    from daphne_amd import build as b

    spec = importlib.util.spec_from_file_location("genHIPKernelInst", b.KERNEL_GENERATOR)
    mod = sys.modules.get("genHIPKernelInst")
    if mod is None:
        mod = importlib.util.module_from_spec(spec)
        sys.modules["genHIPKernelInst"] = mod
        spec.loader.exec_module(mod)
    return mod


class Matrix:
    """A DenseMatrix<T> of the C++ layer, owned by Python."""

    def __init__(self, rt: "Runtime", handle: int, dtype, owned: bool = True):
        self.rt, self.h, self.dtype, self.owned = rt, handle, np.dtype(dtype), owned

    def _f(self, name):
        return getattr(self.rt.harness, f"th_mat_{name}_{SUFFIX[self.dtype]}")

    @property
    def shape(self):
        return int(self._f("rows")(self.h)), int(self._f("cols")(self.h))

    def where(self) -> int:
        """bit 0: the host copy is current, bit 1: the device copy is."""
        return int(self._f("where")(self.h))

    def to_numpy(self) -> np.ndarray:
        out = np.empty(self.shape, self.dtype)
        if self._f("to_host")(self.h, C.c_void_p(out.ctypes.data)) != 0:
            raise RuntimeError(self.rt.harness.th_last_error().decode())
        return out

    def slice(self, rl, ru, cl, cu) -> "Matrix":
        h = self._f("slice")(self.h, rl, ru, cl, cu)
        if not h:
            raise RuntimeError(self.rt.harness.th_last_error().decode())
        return Matrix(self.rt, h, self.dtype)

    def destroy(self):
        if self.h and self.owned:
            self._f("destroy")(self.h)
        self.h = None


class Runtime:
    """A DaphneContext with a HIP context, the kernel library and its catalog."""

    def __init__(self):
        from daphne_amd import build as b

        import cpp_build

        if not (b.KERNEL_LIB_PATH.exists() and b.KERNEL_CATALOG_PATH.exists()):
            b.build_kernel_library(verbose=False)
        if not cpp_build.HARNESS_LIB.exists():
            cpp_build.build_harness()
        self.harness = C.CDLL(str(cpp_build.HARNESS_LIB))
        self.catalog = json.loads(b.KERNEL_CATALOG_PATH.read_text())
        # the catalog names the library relative to its own directory (KernelCatalogParser.cpp:131)
        self.libs = {}
        for rec in self.catalog:
            p = b.KERNEL_CATALOG_PATH.parent / rec["libPath"]
            if p not in self.libs:
                self.libs[p] = C.CDLL(str(p))
            rec["_lib"] = self.libs[p]
        gen = _load_generator()
        self.wrappers = {w.func_name: w for w in gen.generate(json.loads(b.KERNEL_SPEC.read_text()), "HIP")}
        h = self.harness
        h.th_last_error.restype = C.c_char_p
        h.th_ctx_create.restype = C.c_void_p
        h.th_ctx_create_bare.restype = C.c_void_p
        h.th_ctx_uses_hip.argtypes = [C.c_void_p]
        h.th_ctx_destroy.argtypes = [C.c_void_p]
        h.th_register_kernel.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.c_int, C.c_int]
        h.th_set_statistics.argtypes = [C.c_void_p, C.c_int]
        h.th_kernel_calls.argtypes = [C.c_void_p, C.c_int]
        h.th_kernel_calls.restype = C.c_uint64
        h.th_set_vect.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64]
        h.th_device_allocations.argtypes = [C.c_void_p]
        h.th_device_allocations.restype = C.c_size_t
        for suf in SUFFIX.values():
            f = lambda n: getattr(h, f"th_mat_{n}_{suf}")  # noqa: E731
            f("from_host").argtypes = [C.c_size_t, C.c_size_t, C.c_void_p]
            f("from_host").restype = C.c_void_p
            for n in ("rows", "cols"):
                f(n).argtypes = [C.c_void_p]
                f(n).restype = C.c_size_t
            f("where").argtypes = [C.c_void_p]
            f("to_host").argtypes = [C.c_void_p, C.c_void_p]
            f("slice").argtypes = [C.c_void_p] + [C.c_size_t] * 4
            f("slice").restype = C.c_void_p
            f("destroy").argtypes = [C.c_void_p]
        for suf in ("f32", "f64"):
            fn = getattr(h, f"th_run_fused_pipeline_{suf}")
            fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_int), C.POINTER(C.c_int),
                           C.POINTER(C.c_int64), C.c_size_t, C.POINTER(C.c_void_p), C.POINTER(C.c_int), C.POINTER(C.c_int),
                           C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.c_size_t]
        self.ctx = h.th_ctx_create()
        if not self.ctx:
            raise RuntimeError("no DaphneContext with a HIP context: " + h.th_last_error().decode())

    def close(self):
        if self.ctx:
            self.harness.th_ctx_destroy(self.ctx)
            self.ctx = None

    def matrix(self, a: np.ndarray) -> Matrix:
        a = np.ascontiguousarray(a)
        assert a.ndim == 2
        h = getattr(self.harness, f"th_mat_from_host_{SUFFIX[a.dtype]}")(a.shape[0], a.shape[1], C.c_void_p(a.ctypes.data))
        return Matrix(self, h, a.dtype)

    def find(self, mnemonic: str, res_types: list[str], arg_types: list[str]) -> dict:
        """The catalog lookup of RewriteToCallKernelOpPass.cpp:403-415: op mnemonic, result and argument types, backend."""
        hits = [r for r in self.catalog if r["opMnemonic"] == mnemonic and r["backend"] == "HIP" and
                r["resTypes"] == res_types and r["argTypes"] == arg_types]
        if len(hits) != 1:
            raise LookupError(f"{len(hits)} kernels for {mnemonic} {res_types} <- {arg_types}")
        return hits[0]

    def call(self, func_name: str, *args, kid: int | None = None):
        """Calls the entry point. `args` are the kernel's inputs in order (Matrix, None for a null matrix pointer, or
        Python scalars); results are created by the kernel and returned in the order of the parameter list: Matrix for a
        data object, a number for a scalar result."""
        w = self.wrappers[func_name]
        rec = next(r for r in self.catalog if r["kernelFuncName"] == func_name)
        fn = getattr(rec["_lib"], func_name)
        argtypes, values, outs, keep = [], [], [], []
        inputs = list(args)
        for p in w.params:
            t = p.type.replace("const ", "").strip()
            if t.startswith("DenseMatrix<"):
                vt = CPP_VT[t[len("DenseMatrix<"):t.index(">")]]
                if t.endswith("**") and p.type.startswith("const "):
                    # an input handed over by reference (conv2DBackwardData's `output`, a quirk kept from the
                    # reference's kernels.json): a pointer to the pointer
                    m = inputs.pop(0)
                    slot = C.c_void_p(m.h)
                    keep.append(slot)
                    argtypes.append(C.POINTER(C.c_void_p))
                    values.append(C.byref(slot))
                elif t.endswith("**"):
                    if p.is_output:
                        slot = C.c_void_p(None)
                        outs.append(("matrix", slot, vt))
                        argtypes.append(C.POINTER(C.c_void_p))
                        values.append(C.byref(slot))
                    else:
                        raise NotImplementedError(p.type)
                else:
                    m = inputs.pop(0)
                    argtypes.append(C.c_void_p)
                    values.append(m.h if m is not None else None)
            elif t.endswith("*"):  # a scalar result through a pointer
                ct = SCALAR_CT[t[:-1].strip()]
                slot = ct()
                outs.append(("scalar", slot, None))
                argtypes.append(C.POINTER(ct))
                values.append(C.byref(slot))
            elif p.is_output:  # a by-value "result" (the reference's generator drops the reference): ignored
                argtypes.append(SCALAR_CT[t])
                values.append(0)
            else:
                argtypes.append(SCALAR_CT[t])
                values.append(inputs.pop(0))
        assert not inputs, f"{len(inputs)} arguments too many for {func_name}"
        if w.has_kid:
            argtypes.append(C.c_int)
            values.append(self.register(func_name) if kid is None else kid)
        if w.has_ctx:
            argtypes.append(C.c_void_p)
            values.append(self.ctx)
        fn.argtypes, fn.restype = argtypes, None
        fn(*values)
        res = []
        for kind, slot, vt in outs:
            res.append(Matrix(self, slot.value, vt) if kind == "matrix" else slot.value)
        return res[0] if len(res) == 1 else tuple(res)

    def register(self, name: str, file: str = "test.daphne", line: int = 1, col: int = 1) -> int:
        return self.harness.th_register_kernel(self.ctx, name.encode(), file.encode(), line, col)
