"""TEST INFRASTRUCTURE ONLY: loader for the CPU parity checker.

Only tests, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg
import this module.  ``tokenweave_amd`` (the product) never does.

Three independent statements of the same path live here:

* ``libtw_oracle.so`` (``tw_oracle.c``) — C restatement of the reference's CPU
  path ``csrc/cpu/layernorm.cpp:44-88`` extended to P partial buffers;
* ``_ref/libtw_ref.so`` — the reference's own ``csrc/cpu/layernorm.cpp`` compiled
  from its sources (P=1 only, truncating fp32->bf16 as in its non-AVX512-BF16
  builds);
* ``forward_native_np`` — numpy fp32 restatement of ``RMSNorm.forward_native``
  (``vllm/model_executor/layers/layernorm.py:173-210``), the oracle of the
  reference's own unit test ``tests/kernels/test_layernorm.py:48``.

All arrays are ``numpy.uint16`` holding bf16 bit patterns, C-contiguous.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(_HERE, "libtw_oracle.so")
REF_SO = os.path.join(_HERE, "_ref", "libtw_ref.so")

ROUND_RNE = 0
ROUND_TRUNC = 1

_u16p = ctypes.POINTER(ctypes.c_uint16)
_lib = None
_ref = None


def build(force: bool = False) -> None:
    """Compile tw_oracle.c (and oracle/_ref when the reference tree is present)."""
    args = ["make", "-C", _HERE]
    if force:
        args.append("-B")
    subprocess.run(args, check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_SO):
            build()
        L = ctypes.CDLL(ORACLE_SO)
        i64, f32, ci = ctypes.c_int64, ctypes.c_float, ctypes.c_int
        L.tw_oracle_fused_add_rms_norm.argtypes = [_u16p, _u16p, _u16p, i64, i64, f32, ci]
        L.tw_oracle_reduce_add_rms_norm.argtypes = [
            ctypes.POINTER(_u16p), ci, _u16p, _u16p, _u16p, i64, i64, f32, ci]
        L.tw_oracle_rms_norm.argtypes = [_u16p, _u16p, _u16p, i64, i64, f32, ci]
        L.tw_oracle_rms_norm_inplace.argtypes = [_u16p, _u16p, _u16p, i64, i64, f32, ci]
        L.tw_oracle_gemm_bf16_nt.argtypes = [_u16p, _u16p, _u16p, i64, i64, i64, ci]
        L.tw_oracle_static_fp8_quant.argtypes = [ctypes.POINTER(ctypes.c_uint8), _u16p, i64, f32]
        L.tw_oracle_static_fp8_quant.restype = ci
        L.tw_oracle_rms_norm_dynamic_per_token_quant.argtypes = [
            ctypes.POINTER(ctypes.c_uint8), ctypes.POINTER(ctypes.c_float), ctypes.POINTER(_u16p), ci,
            _u16p, _u16p, ctypes.POINTER(ctypes.c_float), i64, i64, f32, ci]
        L.tw_oracle_rms_norm_dynamic_per_token_quant.restype = ci
        for name in ("fused_add_rms_norm", "reduce_add_rms_norm", "rms_norm",
                     "rms_norm_inplace", "gemm_bf16_nt"):
            getattr(L, "tw_oracle_" + name).restype = ci
        _lib = L
    return _lib


def have_ref() -> bool:
    return os.path.exists(REF_SO)


def ref() -> ctypes.CDLL:
    """The reference's own layernorm.cpp; needs libtorch (present in the image)."""
    global _ref
    if _ref is None:
        import torch  # noqa: F401  (loads libtorch_cpu/libc10 so the .so resolves)
        R = ctypes.CDLL(REF_SO)
        i64, f64 = ctypes.c_int64, ctypes.c_double
        R.tw_ref_fused_add_rms_norm.argtypes = [_u16p, _u16p, _u16p, i64, i64, f64]
        R.tw_ref_rms_norm.argtypes = [_u16p, _u16p, _u16p, i64, i64, f64]
        R.tw_ref_fused_add_rms_norm.restype = ctypes.c_int
        R.tw_ref_rms_norm.restype = ctypes.c_int
        _ref = R
    return _ref


def _p(a: np.ndarray):
    assert a.dtype == np.uint16 and a.flags["C_CONTIGUOUS"], (a.dtype, a.flags)
    return a.ctypes.data_as(_u16p)


def _th(x: np.ndarray):
    H = x.shape[-1]
    return x.size // H if H else 0, H


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what}: oracle rejected the arguments (rc={rc})")


# ----------------------------------------------------------------------------
# C restatement
# ----------------------------------------------------------------------------
def fused_add_rms_norm(x, r, w, eps, mode=ROUND_RNE):
    """In place: r <- x + r, x <- norm(r) * w.  Returns (x, r)."""
    T, H = _th(x)
    _check(lib().tw_oracle_fused_add_rms_norm(_p(x), _p(r), _p(w), T, H, eps, mode),
           "fused_add_rms_norm")
    return x, r


def reduce_add_rms_norm(partials, r, w, eps, y=None, mode=ROUND_RNE):
    """r <- sum_p partials[p] + r (in place); returns (y, r).  y may alias a partial."""
    P = len(partials)
    T, H = _th(r)
    if y is None:
        y = np.empty_like(r)
    arr = (_u16p * P)(*[_p(a) for a in partials])
    _check(lib().tw_oracle_reduce_add_rms_norm(arr, P, _p(y), _p(r), _p(w), T, H, eps, mode),
           "reduce_add_rms_norm")
    return y, r


def rms_norm(x, w, eps, out=None, mode=ROUND_RNE):
    T, H = _th(x)
    if out is None:
        out = np.empty_like(x)
    _check(lib().tw_oracle_rms_norm(_p(out), _p(x), _p(w), T, H, eps, mode), "rms_norm")
    return out


def rms_norm_inplace(out, x, w, eps, mode=ROUND_RNE):
    """out <- x, x <- norm(x) * w.  Returns x."""
    T, H = _th(x)
    _check(lib().tw_oracle_rms_norm_inplace(_p(out), _p(x), _p(w), T, H, eps, mode),
           "rms_norm_inplace")
    return x


def gemm_bf16_nt(a, b, mode=ROUND_RNE):
    """out[M,N] = a[M,K] @ b[N,K]^T, fp32 accumulate, bf16 out."""
    M, K = a.shape
    N, K2 = b.shape
    assert K == K2
    out = np.empty((M, N), np.uint16)
    _check(lib().tw_oracle_gemm_bf16_nt(_p(out), _p(a), _p(b), M, N, K, mode), "gemm")
    return out


def static_fp8_quant(y, scale):
    """bf16 bit patterns -> e4m3fn codes (uint8): fp8_rne(clamp(f32(y) * (1/scale), +-448))."""
    assert y.dtype == np.uint16 and y.flags["C_CONTIGUOUS"]
    out = np.empty(y.shape, np.uint8)
    _check(lib().tw_oracle_static_fp8_quant(out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)),
                                            _p(y), y.size, scale), "static_fp8_quant")
    return out


QUANT_FP8 = 0
QUANT_INT8 = 1


def rms_norm_dynamic_per_token_quant(partials, w, eps, qkind, scale_ub=None, r=None):
    """Fused (P-partial) add + RMSNorm + dynamic per-token quantisation.

    partials: list of [T, H] bf16 bit patterns; r (optional) is updated in place.
    Returns (codes uint8 [T, H] — e4m3fn bytes or int8 two's complement, scales f32 [T, 1])."""
    P = len(partials)
    T, H = _th(partials[0])
    out = np.empty(partials[0].shape, np.uint8)
    scales = np.empty((T, 1), np.float32)
    arr = (_u16p * P)(*[_p(a) for a in partials])
    ub = None
    if scale_ub is not None:
        ub = ctypes.pointer(ctypes.c_float(float(scale_ub)))
    _check(lib().tw_oracle_rms_norm_dynamic_per_token_quant(
        out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)),
        scales.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), arr, P,
        _p(r) if r is not None else None, _p(w), ub, T, H, eps, qkind),
        "rms_norm_dynamic_per_token_quant")
    return out, scales


# ----------------------------------------------------------------------------
# the reference's own compiled CPU path (P = 1)
# ----------------------------------------------------------------------------
def ref_fused_add_rms_norm(x, r, w, eps):
    T, H = _th(x)
    _check(ref().tw_ref_fused_add_rms_norm(_p(x), _p(r), _p(w), T, H, eps), "ref fused_add")
    return x, r


def ref_rms_norm(x, w, eps):
    T, H = _th(x)
    out = np.empty_like(x)
    _check(ref().tw_ref_rms_norm(_p(out), _p(x), _p(w), T, H, eps), "ref rms_norm")
    return out


# ----------------------------------------------------------------------------
# bf16 <-> fp32 in numpy, and the forward_native restatement
# ----------------------------------------------------------------------------
def bf16_to_f32(a: np.ndarray) -> np.ndarray:
    return (a.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(f: np.ndarray, mode=ROUND_RNE) -> np.ndarray:
    u = np.ascontiguousarray(f, dtype=np.float32).view(np.uint32)
    if mode == ROUND_TRUNC:
        return (u >> 16).astype(np.uint16)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    rounded = (u + (0x7FFF + ((u >> 16) & 1))) >> 16
    return np.where(nan, (u >> 16) | 0x40, rounded).astype(np.uint16)


def forward_native_np(x, r, w, eps):
    """RMSNorm.forward_native (layernorm.py:173-210) on bf16 bit patterns.

    Not in place.  Differs from the CPU path in where it rounds: y is
    bf16(s * rsqrt(var + eps)) then a bf16 * bf16 weight multiply (two
    roundings), and the mean is numpy's pairwise fp32 mean.
    Returns y, or (y, r') when r is given.
    """
    s = bf16_to_f32(x)
    r_new = None
    if r is not None:
        s = s + bf16_to_f32(r)
        r_new = f32_to_bf16(s)
    var = np.mean(s * s, axis=-1, keepdims=True, dtype=np.float32)
    inv = (np.float32(1.0) / np.sqrt(var + np.float32(eps))).astype(np.float32)
    n = f32_to_bf16(s * inv)
    y = f32_to_bf16(bf16_to_f32(n) * bf16_to_f32(w))
    return y if r is None else (y, r_new)


def reduce_add_rms_norm_f64(partials, r, w, eps):
    """High-precision witness: everything in float64, no intermediate rounding.

    Returns (y_f64, s_f64): the normalised output and the pre-norm sum, both
    unrounded, for tolerance checks against any bf16 implementation."""
    s = np.zeros(r.shape, np.float64)
    for p in partials:
        s += bf16_to_f32(p).astype(np.float64)
    s += bf16_to_f32(r).astype(np.float64)
    inv = 1.0 / np.sqrt(np.mean(s * s, axis=-1, keepdims=True) + float(eps))
    return s * inv * bf16_to_f32(w).astype(np.float64), s
