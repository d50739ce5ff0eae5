"""ctypes binding of libtokenweave_amd.so (the C ABI in include/tokenweave_amd.h).

There is no fallback: if the HIP library has not been built, every op raises.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtokenweave_amd.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

TW_OK = 0
TW_ERR_INVALID_ARGUMENT = -1
TW_ERR_ALIGNMENT = -2
TW_ERR_DTYPE = -3
TW_ERR_LAUNCH = -4

TW_DTYPE_BF16 = 0
TW_DTYPE_F16 = 1
TW_DTYPE_F32 = 2
TW_MAX_PARTIALS = 16
TW_SPLIT_MAX_TOKENS = 256
TW_SPLIT_WORKSPACE_BYTES = TW_SPLIT_MAX_TOKENS * 384

_vp, _i64, _u64, _f32, _ci = (ctypes.c_void_p, ctypes.c_int64, ctypes.c_uint64,
                              ctypes.c_float, ctypes.c_int)

# name -> argtypes; the order is the order of include/tokenweave_amd.h
PROTOTYPES = {
    "tw_version": [],
    "tw_last_error": [],
    "tw_num_compute_units": [],
    "tw_fused_add_rms_norm": [_vp, _vp, _vp, _i64, _i64, _f32, _ci, _vp],
    "tw_rms_norm": [_vp, _vp, _vp, _i64, _i64, _f32, _ci, _vp],
    "tw_rms_norm_inplace": [_vp, _vp, _vp, _i64, _i64, _f32, _ci, _vp],
    "tw_fused_add_rms_norm_cta": [_vp, _vp, _vp, _i64, _i64, _ci, _f32, _vp],
    "tw_reduce_add_rms_norm": [ctypes.POINTER(_vp), _ci, _vp, _vp, _vp, _i64, _i64, _ci, _f32, _vp],
    "tw_fused_rs_ln_cta": [_vp, _vp, _vp, _u64, _i64, _ci, _ci, _ci, _f32, _i64, _i64, _vp],
    "tw_fused_rs_ln_ag_cta": [_vp, _vp, _vp, _u64, _i64, _ci, _ci, _ci, _f32, _i64, _i64, _vp],
    "tw_reduce_add_rms_norm_ws": [ctypes.POINTER(_vp), _ci, _vp, _vp, _vp, _i64, _i64, _ci, _f32, _vp, _i64,
                                  _vp],
    "tw_fused_rs_ln_ag_cta_ws": [_vp, _vp, _vp, _u64, _i64, _ci, _ci, _ci, _f32, _i64, _i64, _vp, _i64, _vp],
    "tw_reduce_add_rms_norm_noalloc": [ctypes.POINTER(_vp), _ci, _vp, _vp, _vp, _i64, _i64, _ci, _f32, _vp],
    "tw_split_segments": [_i64, _i64, _ci],
    "tw_gemm_bf16_nt": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _ci, _vp],
    "tw_gemm_bf16_nt_bias": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _ci, _vp],
    "tw_gemm_bf16_nt_partials": [ctypes.POINTER(_vp), ctypes.POINTER(_vp), ctypes.POINTER(_vp), _ci, _i64, _i64,
                                 _i64, _i64, _ci, _vp],
    "tw_rms_norm_static_fp8_quant": [_vp, _vp, _vp, _vp, _i64, _i64, _f32, _ci, _vp],
    "tw_fused_add_rms_norm_static_fp8_quant": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _f32, _ci, _vp],
    "tw_reduce_add_rms_norm_static_fp8_quant": [ctypes.POINTER(_vp), _ci, _vp, _vp, _vp, _vp, _i64, _i64,
                                                _ci, _f32, _vp],
    "tw_rms_norm_dynamic_per_token_quant": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _f32, _ci, _ci, _vp],
    "tw_reduce_add_rms_norm_dynamic_per_token_quant": [ctypes.POINTER(_vp), _ci, _vp, _vp, _vp, _vp, _vp,
                                                       _i64, _i64, _ci, _f32, _ci, _vp],
    "tw_gemm_bf16_nt_partials_bias": [ctypes.POINTER(_vp), ctypes.POINTER(_vp), ctypes.POINTER(_vp),
                                      ctypes.POINTER(_vp), _ci, _i64, _i64, _i64, _i64, _ci, _vp],
}

_lib = None


def build(verbose: bool = False) -> str:
    """Compile the HIP sources for gfx950 with hipcc (cross-compiles without a GPU)."""
    global _lib
    proc = subprocess.run(["make", "-B", "-C", CSRC_DIR], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True)
    if verbose or proc.returncode != 0:
        print(proc.stdout)
    if proc.returncode != 0:
        raise RuntimeError("hipcc build of libtokenweave_amd.so failed:\n" + proc.stdout)
    _lib = None
    return LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {CSRC_DIR}` "
                "(tokenweave_amd has no non-HIP fallback)")
        L = ctypes.CDLL(LIB_PATH)
        for name, argtypes in PROTOTYPES.items():
            fn = getattr(L, name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_char_p if name == "tw_last_error" else _ci
        _lib = L
    return _lib


def last_error() -> str:
    return lib().tw_last_error().decode("utf-8", "replace")


def check(rc: int) -> None:
    """Turn a TW_ERR_* return code into the exception the reference would raise."""
    if rc == TW_OK:
        return
    msg = last_error()
    if rc == TW_ERR_DTYPE:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)
