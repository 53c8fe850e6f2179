"""ctypes binding of libdaphne_hip.so (the C ABI declared in include/daphne_hip.h).

Loading fails loudly when the library has not been built: there is no CPU fallback.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libdaphne_hip.so"

DH_OK, DH_ERR_RUNTIME, DH_ERR_INVALID_ARG, DH_ERR_DOMAIN, DH_ERR_HIP, DH_ERR_OOM, DH_ERR_OUT_OF_RANGE = range(7)

sz = C.c_size_t
vp = C.c_void_p
i32 = C.c_int


class DaphneHipError(RuntimeError):
    """std::runtime_error of the reference (bad shapes, unknown op codes, HIP failures)."""

    def __init__(self, status: int, msg: str):
        super().__init__(msg)
        self.status = status


class DaphneHipInvalidArgument(DaphneHipError, ValueError):
    """std::invalid_argument of the reference."""


class DaphneHipDomainError(DaphneHipError, ArithmeticError):
    """std::domain_error of the reference (sqrt/ln/asin/acos outside their domain)."""


class DaphneHipOutOfRange(DaphneHipError, IndexError):
    """std::out_of_range of the reference (ExtractCol position outside the matrix)."""


_lib = None


def _signatures(lib: C.CDLL) -> None:
    ctxp = vp
    lib.dh_last_error.restype = C.c_char_p
    lib.dh_last_error.argtypes = []
    lib.dh_ctx_create.argtypes = [i32, C.POINTER(vp)]
    lib.dh_ctx_destroy.argtypes = [ctxp]
    lib.dh_ctx_mem_budget.argtypes = [ctxp]
    lib.dh_ctx_mem_budget.restype = sz
    lib.dh_ctx_mem_in_use.argtypes = [ctxp]
    lib.dh_ctx_mem_in_use.restype = sz
    lib.dh_ctx_mem_cached.argtypes = [ctxp]
    lib.dh_ctx_mem_cached.restype = sz
    lib.dh_ctx_release_cached.argtypes = [ctxp]
    lib.dh_ctx_device.argtypes = [ctxp]
    lib.dh_ctx_props.argtypes = [ctxp, C.POINTER(i32), C.POINTER(i32), C.POINTER(sz), C.c_char_p, sz]
    lib.dh_device_memory.argtypes = [i32, C.POINTER(sz), C.POINTER(sz)]
    lib.dh_ctx_set_stream.argtypes = [ctxp, vp]
    lib.dh_ctx_get_stream.argtypes = [ctxp]
    lib.dh_ctx_get_stream.restype = vp
    lib.dh_sync.argtypes = [ctxp]
    lib.dh_defer_checks.argtypes = [ctxp, i32]
    lib.dh_check_deferred.argtypes = [ctxp]
    lib.dh_malloc.argtypes = [ctxp, sz, i32, C.POINTER(vp)]
    lib.dh_free.argtypes = [ctxp, vp]
    lib.dh_h2d.argtypes = [ctxp, vp, vp, sz]
    lib.dh_d2h.argtypes = [ctxp, vp, vp, sz]
    lib.dh_d2d.argtypes = [ctxp, vp, vp, sz]
    lib.dh_d2d_2d.argtypes = [ctxp, vp, sz, vp, sz, sz, sz]
    lib.dh_d2h_2d.argtypes = [ctxp, vp, sz, vp, sz, sz, sz]
    lib.dh_timer_start.argtypes = [ctxp]
    lib.dh_ctx_set_pipeline_mode.argtypes = [ctxp, i32]
    lib.dh_ctx_get_pipeline_mode.argtypes = [ctxp]
    lib.dh_vectorized_pipeline_last_mode.argtypes = []
    lib.dh_vectorized_pipeline_cache_size.argtypes = []
    lib.dh_vectorized_pipeline_cache_size.restype = sz
    lib.dh_vectorized_pipeline_set_cache_limit.argtypes = [sz]
    lib.dh_vectorized_pipeline_set_cache_limit.restype = sz
    lib.dh_agg_col_noalloc_f32.argtypes = [ctxp, i32, vp, vp, sz, sz, sz]
    lib.dh_agg_col_noalloc_scratch_bytes.argtypes = []
    lib.dh_agg_col_noalloc_scratch_bytes.restype = sz
    lib.dh_timer_stop_ms.argtypes = [ctxp, C.POINTER(C.c_float)]
    lib.dh_kernel_timing.argtypes = [ctxp, i32]
    lib.dh_kernel_timing_read.argtypes = [ctxp, C.POINTER(C.c_double), C.POINTER(sz)]
    for suf, ct in (("f32", C.c_float), ("f64", C.c_double)):
        f = lambda name: getattr(lib, f"{name}_{suf}")
        f("dh_ew_binary").argtypes = [ctxp, i32, vp, sz, vp, sz, sz, sz, vp, sz, sz, sz]
        f("dh_ew_binary_sca").argtypes = [ctxp, i32, vp, sz, vp, sz, sz, sz, ct]
        f("dh_ew_unary").argtypes = [ctxp, i32, vp, sz, vp, sz, sz, sz]
        f("dh_agg_all").argtypes = [ctxp, i32, vp, sz, sz, sz, C.POINTER(ct)]
        f("dh_agg_all_dev").argtypes = [ctxp, i32, vp, sz, sz, sz, vp]
        f("dh_agg_row").argtypes = [ctxp, i32, vp, sz, vp, sz, sz, sz]
        f("dh_agg_row_idx").argtypes = [ctxp, i32, vp, sz, vp, sz, sz, sz]
        f("dh_agg_col").argtypes = [ctxp, i32, vp, vp, sz, sz, sz]
        f("dh_agg_col_idx").argtypes = [ctxp, i32, vp, vp, sz, sz, sz]
        for name, at in _LATE_SIGNATURES.items():
            fn = getattr(lib, f"{name}_{suf}", None)
            if fn is not None:
                fn.argtypes = [ct if a == "T" else a for a in at]
    # integer value types: elementwise for all four, aggregations and data reorganisation for 64-bit ones
    for suf, ct in (("si64", C.c_int64), ("ui64", C.c_uint64), ("si32", C.c_int32), ("ui32", C.c_uint32)):
        getattr(lib, f"dh_ew_binary_{suf}").argtypes = [ctxp, i32, vp, sz, vp, sz, sz, sz, vp, sz, sz, sz]
        getattr(lib, f"dh_ew_binary_sca_{suf}").argtypes = [ctxp, i32, vp, sz, vp, sz, sz, sz, ct]
    lib.dh_agg_all_si64.argtypes = [ctxp, i32, vp, sz, sz, sz, C.POINTER(C.c_int64)]
    lib.dh_agg_row_si64.argtypes = [ctxp, i32, vp, sz, vp, sz, sz, sz]
    lib.dh_agg_row_idx_si64.argtypes = [ctxp, i32, vp, sz, vp, sz, sz, sz]
    lib.dh_agg_col_si64.argtypes = [ctxp, i32, vp, vp, sz, sz, sz]
    lib.dh_agg_col_idx_si64.argtypes = [ctxp, i32, vp, vp, sz, sz, sz]
    lib.dh_fill_si64.argtypes = [ctxp, vp, sz, C.c_int64, sz, sz]
    lib.dh_fill_ui64.argtypes = [ctxp, vp, sz, C.c_uint64, sz, sz]
    lib.dh_col_bind_si64.argtypes = _LATE_SIGNATURES["dh_col_bind"]
    lib.dh_extract_col_si64.argtypes = _LATE_SIGNATURES["dh_extract_col"]
    lib.dh_transpose_si64.argtypes = _LATE_SIGNATURES["dh_transpose"]


# Entry points added after the first kernels; bound when the library exports them.
_LATE_SIGNATURES: dict[str, list] = {
    "dh_matmul": [vp, vp, sz, vp, sz, sz, sz, vp, sz, sz, sz, i32, i32],
    "dh_syrk": [vp, vp, sz, vp, sz, sz, sz, i32],
    "dh_solve": [vp, vp, vp, sz, sz, vp],
    "dh_normal_equations": [vp, vp, sz, vp, sz, vp, sz, sz, sz, vp, sz, "T"],
    "dh_kmeans_assign": [vp, vp, vp, sz, sz, sz, vp, sz, sz, vp, vp],
    "dh_kmeans_update": [vp, vp, sz, vp, vp, sz, sz, sz, vp, sz],
    "dh_kmeans_step": [vp, vp, vp, sz, vp, vp, sz, sz, sz, vp, sz, sz, vp, vp],
    "dh_conv2d_forward": [vp, vp, C.POINTER(sz), C.POINTER(sz), vp, vp, sz, sz, vp, sz, sz, sz, sz, sz, sz, sz, sz, sz, sz],
    "dh_conv2d_forward_fused": [vp, vp, C.POINTER(sz), C.POINTER(sz), vp, vp, sz, sz, vp, sz, sz, sz, sz, sz, sz, sz, sz, sz, sz,
                                C.c_uint],
    "dh_maxpool_forward": [vp, vp, C.POINTER(sz), C.POINTER(sz), vp, sz, sz, sz, sz, sz, sz, sz, sz, sz, sz],
    "dh_affine_forward": [vp, vp, vp, sz, sz, vp, sz, sz, vp, sz, sz],
    "dh_affine_forward_fused": [vp, vp, vp, sz, sz, vp, sz, sz, vp, sz, sz, C.c_uint],
    "dh_bias_add": [vp, vp, vp, sz, sz, vp, sz],
    "dh_batchnorm_inference": [vp, vp, vp, sz, sz, vp, vp, vp, vp, sz, "T", i32],
    "dh_softmax": [vp, vp, sz, vp, sz, sz, sz],
    "dh_agg_col_moments": [vp, vp, vp, i32, vp, sz, sz, sz],
    "dh_avgpool_forward": [vp, vp, C.POINTER(sz), C.POINTER(sz), vp, sz, sz, sz, sz, sz, sz, sz, sz, sz, sz],
    "dh_relu_forward": [vp, vp, sz, vp, sz, sz, sz],
    "dh_fill": [vp, vp, sz, "T", sz, sz],
    "dh_col_bind": [vp, vp, sz, vp, sz, sz, sz, vp, sz, sz, sz],
    "dh_extract_col": [vp, vp, sz, vp, sz, sz, sz, vp, sz, sz, sz],
    "dh_transpose": [vp, vp, sz, vp, sz, sz, sz],
    "dh_gemv": [vp, vp, sz, vp, sz, sz, sz, vp, sz, sz],
    "dh_batchnorm_train_forward": [vp, vp, vp, vp, vp, vp, vp, sz, sz, vp, vp, vp, vp, sz, "T", "T"],
    "dh_batchnorm_backward": [vp, vp, vp, vp, vp, vp, vp, vp, sz, sz, vp, sz, "T"],
    "dh_maxpool_backward": [vp, vp, vp, vp, sz, sz, sz, sz, sz, sz, sz, sz, sz, sz],
    "dh_avgpool_backward": [vp, vp, vp, vp, sz, sz, sz, sz, sz, sz, sz, sz, sz, sz],
    "dh_conv2d_backward_data": [vp, vp, vp, vp, sz, sz, sz, sz, sz, sz, sz, sz, sz, sz, sz],
    "dh_conv2d_backward_filter": [vp, vp, vp, vp, sz, sz, sz, sz, sz, sz, sz, sz, sz, sz, sz],
}


def lib() -> C.CDLL:
    """Returns the loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m daphne_amd.build` "
                "(there is no CPU fallback for the device kernels)"
            )
        _lib = C.CDLL(str(LIB_PATH))
        _signatures(_lib)
    return _lib


def check(status: int) -> None:
    """Turns a dh_status into the exception type the reference would throw."""
    if status == DH_OK:
        return
    msg = lib().dh_last_error().decode("utf-8", "replace")
    if status == DH_ERR_INVALID_ARG:
        raise DaphneHipInvalidArgument(status, msg)
    if status == DH_ERR_OUT_OF_RANGE:
        raise DaphneHipOutOfRange(status, msg)
    if status == DH_ERR_DOMAIN:
        raise DaphneHipDomainError(status, msg)
    raise DaphneHipError(status, msg)
