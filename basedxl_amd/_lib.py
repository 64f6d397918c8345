"""ctypes binding of libcascmm.so (the C ABI declared in include/cascmm.h).

There is no second code path: if the shared library is missing or cannot be loaded the
import of the operator fails with an error that says how to build it.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_int, c_int32, c_int64, c_size_t, c_void_p, POINTER

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcascmm.so")

# enums of include/cascmm.h
DT_F32, DT_F16, DT_BF16 = 0, 1, 2
FMT_BF16, FMT_FP16, FMT_FP8 = 0, 1, 2
PROD_TRI, PROD_FULL = 0, 1
ERR_BAD_FORMAT = -4   # CASCMM_ERR_BAD_FORMAT: no kernel for this (dtype, format, terms, products, shape)

FMT_BY_NAME = {"bf16": FMT_BF16, "fp16": FMT_FP16, "fp8": FMT_FP8}
PROD_BY_NAME = {"tri": PROD_TRI, "full": PROD_FULL}

_GEMM_ARGS = [c_void_p, c_void_p, c_void_p, c_void_p,  # A B C bias
              c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,  # M N K lda ldb ldc
              c_int, c_int, c_int, c_int,  # dtype fmt terms products
              c_void_p, c_void_p, c_size_t, c_void_p]  # tensor_exps workspace workspace_bytes stream

#: every exported symbol with its signature; tests check that the library exports each one
SIGNATURES = {
    "cascmm_gemm": (c_int, _GEMM_ARGS),
    "cascmm_gemm_variant": (c_int, _GEMM_ARGS + [c_int]),
    "cascmm_gemm_noalloc": (c_int, _GEMM_ARGS[:15] + [c_void_p]),
    "cascmm_init": (c_int, []),
    "cascmm_gemm_grouped": (c_int, [c_int, c_void_p, c_void_p, c_void_p, c_void_p] + _GEMM_ARGS[4:] + [c_int]),
    "cascmm_prepared_bytes": (c_size_t, [c_int64, c_int64, c_int, c_int]),
    "cascmm_prepare_weight": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_void_p, c_void_p,
                                      c_size_t, c_void_p]),
    "cascmm_gemm_prepared": (c_int, [c_int, c_void_p, c_void_p, c_void_p, c_void_p] + [c_int64] * 5 + [c_int] * 4
                             + [c_void_p, c_void_p, c_size_t, c_void_p, c_int]),
    "cascmm_prepare_weight_glu": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_void_p, c_void_p,
                                          c_size_t, c_void_p]),
    "cascmm_gemm_prepared_glu": (c_int, [c_int, c_void_p, c_void_p, c_void_p, c_void_p] + [c_int64] * 5 + [c_int] * 4
                                 + [c_void_p, c_void_p, c_int]),
    "cascmm_select_variant_prepared": (c_int, [c_int] + [c_int64] * 5 + [c_int] * 4),
    "cascmm_select_variant_glu": (c_int, [c_int64] * 6 + [c_int] * 4),
    "cascmm_gemm_glu": (c_int, [c_void_p] * 4 + [c_int64] * 6 + [c_int] * 4 + [c_void_p, c_int]),
    "cascmm_left_slots_bytes": (c_size_t, [c_int64, c_int64]),
    "cascmm_prepare_left": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "cascmm_prepare_weight_chained": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "cascmm_gemm_glu_chained": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_size_t, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                        c_int64, c_void_p]),
    "cascmm_chained_supported": (c_int, [c_int64, c_int64, c_int64]),
    "cascmm_gemm_chained": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "cascmm_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int]),
    "cascmm_select_variant": (c_int, [c_int64] * 6 + [c_int] * 4),
    "cascmm_select_variant_grouped": (c_int, [c_int] + [c_int64] * 6 + [c_int] * 4),
    "cascmm_variant_count": (c_int, []),
    "cascmm_variant_name": (c_char_p, [c_int]),
    "cascmm_variant_kernel": (c_char_p, [c_int]),
    "cascmm_probe_mfma": (c_int, [c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "cascmm_probe_stream": (c_int, [c_void_p, c_void_p, c_size_t, c_int, c_void_p, c_size_t, c_void_p]),
    "cascmm_tensor_exp": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p, c_void_p]),
    "cascmm_tensor_exps": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "cascmm_gemm_fp8_autoscale": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p] + [c_int64] * 6 + [c_int, c_int]
                                  + [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "cascmm_split_terms": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_void_p]),
    "cascmm_selftest": (c_int, []),
    "cascmm_strerror": (c_char_p, [c_int]),
    "cascmm_version": (c_int, []),
}


class CascmmError(RuntimeError):
    """A cascmm_* call returned a non-zero status."""

    def __init__(self, status: int, where: str):
        self.status = status
        msg = lib().cascmm_strerror(status)
        super().__init__(f"{where} failed: {msg.decode() if msg else 'unknown'} (status {status})")


_lib = None


def lib() -> ctypes.CDLL:
    """The loaded library (loaded once)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: the HIP extension is not built. "
                "Run `python -m basedxl_amd.build` (needs hipcc, targets gfx950). "
                "There is no CPU or PyTorch fallback for cascaded_lowp_matmul.")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(status: int, where: str) -> None:
    if status != 0:
        raise CascmmError(status, where)


def variant_names() -> list:
    l = lib()
    return [l.cascmm_variant_name(i).decode() for i in range(l.cascmm_variant_count())]
