"""Loader for the HIP library behind the C ABI declared in ``include/llmc_amd.h``.

The library is the only compute path of this package: there is no CPU or eager
fallback, and a missing library raises at first use.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libllmc_amd.so")
CSRC_DIR = os.path.join(os.path.dirname(_HERE), "csrc")

_lib = None


class LibraryMissing(RuntimeError):
    pass


def build(jobs: int = 8) -> str:
    """Compile every kernel for gfx950 (cross-compiles without a GPU)."""
    import subprocess

    subprocess.check_call(["make", "-C", CSRC_DIR, f"-j{jobs}", "-B"])
    global _lib
    _lib = None
    return LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LibraryMissing(
                f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
                "(there is no fallback path)"
            )
        _lib = ctypes.CDLL(LIB_PATH)
        _declare(_lib)
    return _lib


_P = ctypes.c_void_p
_I64 = ctypes.c_int64
_I32 = ctypes.c_int32
_F32 = ctypes.c_float

# name -> argtypes; every function returns int
SIGNATURES = {
    "llmc_version": [],
    "llmc_hessian_workspace_bytes": [_I64, _I64],
    "llmc_hessian_accumulate_grouped": [_P, _I64, _P, _I64, _P, _I32, _I64, _I32, _F32, _I32, _P],
    "llmc_gptq_hinv_grouped_workspace_bytes": [_I64, _I64],
    "llmc_gptq_hinv_grouped": [_P, _I64, _I32, _I64, _P, _P, _F32, _I32, _P, _P, _I64, _P, _I64, _P, _P],
    "llmc_gptq_quantize_grouped_workspace_bytes": [_I64, _I64, _I64, _I32],
    "llmc_gptq_quantize_grouped": [_P, _I32, _I32, _I64, _I64, _I64, _P, _I64, _I64, _P, _P, _P, _I32, _P, _P, _P, _I64,
                                   _I64, _I32, _I32, _I32, _I32, _P, _I64, _P, _P, _I64, _P],
    "llmc_sparsegpt_workspace_bytes": [_I64, _I64, _I32],
    "llmc_sparsegpt_sparsify": [_P, _I32, _I64, _I64, _I64, _P, _I64, _P, ctypes.c_double, _I32, _I32, _I32, _I32, _I32,
                                _P, _I64, _P, _P, _I64, _P],
    "llmc_hessian_accumulate_segments": [_P, _I64, _P, _I32, _I64, _I64, _I64, _I64, _I32, _F32, _I32, _P, _I64, _P],
    "llmc_hessian_accumulate": [_P, _I64, _P, _I64, _I64, _I64, _I32, _F32, _I32, _P, _I64, _P],
    "llmc_minmax_groups": [_P, _I32, _I64, _I64, _I64, _I64, _P, _P, _P, _I64, _P],
    "llmc_minmax_blocks": [_P, _I32, _I64, _I64, _I64, _I32, _I32, _P, _P, _P],
    "llmc_minmax_strided": [_P, _I32, _I64, _I64, _I64, _I64, _I64, _P, _P, _P],
    "llmc_absmax_accumulate": [_P, _P, _I64, _I32, _P, _P],
    "llmc_generate_gparam": [_P, _I32, _P, _P],
    "llmc_calculate_qparams": [_P, _P, _I64, _I32, _I32, _I32, _I32, _I32, _P, _P, _I32, _P, _P, _P],
    "llmc_quantize": [_P, _I32, _I64, _I64, _I64, _P, _I32, _P, _P, _P, _I32, _I32, _I64, _I64, _I64,
                      _I32, _P, _I32, _I64, _P],
    "llmc_dynamic_per_token_quantize": [_P, _I32, _I64, _I64, _I64, _I32, _I32, _I32, _P, _I64, _P, _P],
}
SIGNATURES.update({
    "llmc_gptq_hinv_workspace_bytes": [_I64],
    "llmc_gptq_hinv": [_P, _I64, _I64, _P, _F32, _F32, _I32, _P, _P, _I64, _P, _P],
    "llmc_gptq_factor_form": [_I64, _I32],
    "llmc_gptq_quantize_workspace_bytes": [_I64, _I64, _I32],
    "llmc_gptq_quantize": [_P, _I32, _I64, _I64, _I64, _P, _I64, _P, _P, _P, _I32, _P, _P, _P, _I64, _I64,
                           _I32, _I32, _I32, _I32, _P, _I64, _P, _P, _I64, _P],
})
_F64 = ctypes.c_double
SIGNATURES.update({
    "llmc_mse_workspace_bytes": [_I64],
    "llmc_mse_observe_groups": [_P, _I32, _I64, _I64, _I64, _I64, _I32, _I32, _I32, _I32, _I32, _F64, _I32, _F32,
                                _F32, _P, _P, _P, _I64, _P],
    "llmc_sumsq_workspace_bytes": [_I64],
    "llmc_sgemm": [_P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I64, _F32, _F32, _I32, _I32, _P],
    "llmc_sumsq_accumulate": [_P, _I32, _I64, _I64, _I64, _P, _P, _I64, _P],
    "llmc_sumsq_accumulate_noalloc": [_P, _I32, _I64, _I64, _I64, _P, _P],
    "llmc_imatrix_observe_groups": [_P, _I32, _I64, _I64, _I64, _I64, _I32, _I32, _I32, _I32, _I32, _F64, _I32, _F32,
                                    _F32, _P, _P, _P, _P, _I64, _P],
    "llmc_imatrix_observe_strided": [_P, _I32, _I64, _I64, _I64, _I64, _I64, _I32, _I32, _I32, _I32, _I32, _F64, _I32,
                                     _F32, _F32, _P, _P, _P, _I64, _P],
    "llmc_imatrix_observe_blocks": [_P, _I32, _I64, _I64, _I64, _I32, _I32, _I32, _I32, _I32, _I32, _I32, _F64, _I32,
                                    _F32, _F32, _P, _P, _P, _I64, _P],
    "llmc_mse_observe_strided": [_P, _I32, _I64, _I64, _I64, _I64, _I64, _I32, _I32, _I32, _I32, _I32, _F64, _I32,
                                 _F32, _F32, _P, _P, _P, _I64, _P],
    "llmc_mse_observe_blocks": [_P, _I32, _I64, _I64, _I64, _I32, _I32, _I32, _I32, _I32, _I32, _I32, _F64, _I32,
                                _F32, _F32, _P, _P, _P, _I64, _P],
})
SIGNATURES["llmc_diag_argsort_desc"] = [_P, _I64, _I32, _I64, _P, _P]
SIGNATURES["llmc_grouped_linear"] = [_P, _I32, _I64, _P, _I64, _I32, _I32, _P, _I64, _P, _I32, _I64, _I64, _P]
# functions whose return type is not int
RESTYPES = {
    "llmc_hessian_workspace_bytes": ctypes.c_int64,
    "llmc_minmax_workspace_bytes": ctypes.c_int64,
    "llmc_gptq_hinv_workspace_bytes": ctypes.c_int64,
    "llmc_mse_workspace_bytes": ctypes.c_int64,
    "llmc_gptq_quantize_workspace_bytes": ctypes.c_int64,
    "llmc_sparsegpt_workspace_bytes": ctypes.c_int64,
    "llmc_gptq_quantize_grouped_workspace_bytes": ctypes.c_int64,
    "llmc_gptq_hinv_grouped_workspace_bytes": ctypes.c_int64,
    "llmc_sumsq_workspace_bytes": ctypes.c_int64,
}
SIGNATURES["llmc_minmax_workspace_bytes"] = []


def _declare(l: ctypes.CDLL) -> None:
    for name, argtypes in SIGNATURES.items():
        fn = getattr(l, name)
        fn.argtypes = argtypes
        fn.restype = RESTYPES.get(name, ctypes.c_int)


def check(rc: int, what: str) -> None:
    if rc == 0:
        return
    if rc < 0:
        raise ValueError(f"{what}: argument {-rc} rejected")
    if rc >= 1000:
        raise RuntimeError(f"{what}: HIP error {rc - 1000}")
    raise RuntimeError(f"{what}: info={rc}")
