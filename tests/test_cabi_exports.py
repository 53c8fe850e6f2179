"""CPU: the built library loads, exports every entry point the public header declares, reports
errors instead of crashing when there is no device, and the run-time specialisation of pipeline
bodies compiles (hiprtc needs no GPU to compile)."""
import ctypes as C
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = (ROOT / "include" / "daphne_hip.h").read_text()


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    text = re.sub(r"#define[^\n]*(\\\n[^\n]*)*", "", text)
    names = set(re.findall(r"\b(dh_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_header_declares_the_kernel_set():
    names = declared_functions()
    for stem in ("dh_ew_binary", "dh_ew_binary_sca", "dh_ew_unary", "dh_agg_all", "dh_agg_row", "dh_agg_row_idx",
                 "dh_agg_col", "dh_agg_col_idx", "dh_matmul", "dh_syrk", "dh_solve", "dh_conv2d_forward",
                 "dh_maxpool_forward", "dh_affine_forward", "dh_bias_add", "dh_batchnorm_inference", "dh_softmax",
                 "dh_vectorized_pipeline"):
        for suf in ("f32", "f64"):
            assert f"{stem}_{suf}" in names, f"{stem}_{suf} is not declared"
    for fn in ("dh_ctx_create", "dh_ctx_destroy", "dh_malloc", "dh_free", "dh_h2d", "dh_d2h", "dh_d2d", "dh_sync",
               "dh_last_error", "dh_ctx_mem_budget"):
        assert fn in names


def test_library_exports_every_declared_symbol():
    from daphne_amd import capi

    lib = capi.lib()
    missing = [n for n in declared_functions() if not hasattr(lib, n)]
    assert not missing, f"declared in include/daphne_hip.h but not exported: {missing}"


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from daphne_amd import capi

    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", tmp_path / "libdaphne_hip.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        capi.lib()


def test_context_creation_without_device_reports_an_error():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a device is present")
    from daphne_amd import capi

    lib = capi.lib()
    h = C.c_void_p()
    st = lib.dh_ctx_create(0, C.byref(h))
    assert st != capi.DH_OK and not h.value
    assert lib.dh_last_error()
    with pytest.raises(capi.DaphneHipError):
        capi.check(st)
    # null context: every kernel entry point refuses instead of dereferencing it
    assert lib.dh_ew_binary_f32(None, 0, None, 0, None, 1, 1, 1, None, 1, 1, 1) == capi.DH_ERR_RUNTIME
    assert lib.dh_matmul_f64(None, None, 1, None, 1, 1, 1, None, 1, 1, 1, 0, 0) == capi.DH_ERR_RUNTIME


def test_pipeline_body_specialisation_compiles():
    from daphne_amd import capi
    from daphne_amd.pipeline import (KIND_EW_BINARY, KIND_EW_UNARY, KIND_REDUCE_ALL, KIND_ROW_AGG, KIND_STORE_ROW,
                                     KIND_STORE_ROW_IDX, KIND_STORE_TILE, OPD_COLVEC, OPD_MATRIX, OPD_ROWREG,
                                     OPD_ROWVEC, OPD_SCALAR, OPD_SELF, PipeInstr)

    lib = capi.lib()
    lib.dh_vectorized_pipeline_compile_check.argtypes = [C.c_int, C.c_size_t, C.c_int, C.c_void_p, C.c_int]
    zscore = [PipeInstr(kind=KIND_EW_BINARY, op=1, operand=OPD_ROWVEC, index=0),
              PipeInstr(kind=KIND_EW_BINARY, op=3, operand=OPD_ROWVEC, index=1),
              PipeInstr(kind=KIND_EW_BINARY, op=2, operand=OPD_SELF),
              PipeInstr(kind=KIND_ROW_AGG, op=0), PipeInstr(kind=KIND_STORE_ROW, index=0),
              PipeInstr(kind=KIND_EW_BINARY, op=11, domain=1, operand=OPD_SCALAR, scalar=64.0),
              PipeInstr(kind=KIND_REDUCE_ALL, op=0, domain=1, index=0)]
    every_kind = [PipeInstr(kind=KIND_EW_BINARY, op=4, operand=OPD_MATRIX, index=0, swap=1),
                  PipeInstr(kind=KIND_EW_BINARY, op=0, operand=OPD_COLVEC, index=0),
                  PipeInstr(kind=KIND_EW_UNARY, op=3), PipeInstr(kind=KIND_STORE_TILE, index=0),
                  PipeInstr(kind=KIND_ROW_AGG, op=4), PipeInstr(kind=KIND_STORE_ROW_IDX, index=0),
                  PipeInstr(kind=KIND_ROW_AGG, op=8), PipeInstr(kind=KIND_EW_BINARY, op=3, operand=OPD_ROWREG),
                  PipeInstr(kind=KIND_REDUCE_ALL, op=3, domain=0, index=1)]
    for prog, vt, cols, vectorised in ((zscore, 0, 64, 1), (every_kind, 1, 100, 1), (every_kind, 0, 7, 0)):
        arr = (PipeInstr * len(prog))(*prog)
        st = lib.dh_vectorized_pipeline_compile_check(vt, cols, vectorised, C.cast(arr, C.c_void_p), len(prog))
        assert st == capi.DH_OK, lib.dh_last_error().decode()
