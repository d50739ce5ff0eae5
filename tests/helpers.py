"""Shared by the tests: torch <-> bf16 bit patterns, ulp distance, comparisons."""
import numpy as np
import torch

RTOL, ATOL = 1.6e-2, 1e-2   # tolerance of the path on bf16 outputs and on the residual


def to_bits(t: torch.Tensor) -> np.ndarray:
    """bf16 torch tensor (any device) -> C-contiguous uint16 numpy array."""
    assert t.dtype == torch.bfloat16
    return np.ascontiguousarray(t.detach().contiguous().cpu().view(torch.int16).numpy().view(np.uint16))


def from_bits(a: np.ndarray, device="cpu") -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).to(device)


def bits_to_f32(a: np.ndarray) -> np.ndarray:
    return (a.astype(np.uint32) << 16).view(np.float32)


def ulp_distance(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Distance in bf16 units of last place between two bit-pattern arrays
    (sign-magnitude mapped to a monotone integer line)."""
    def key(u):
        i = u.astype(np.int32)
        return np.where(i & 0x8000, -(i & 0x7FFF), i & 0x7FFF)
    return np.abs(key(a) - key(b))


def assert_close_bits(got: np.ndarray, want: np.ndarray, what: str, rtol=RTOL, atol=ATOL):
    g, w = bits_to_f32(got).astype(np.float64), bits_to_f32(want).astype(np.float64)
    bad = ~(np.abs(g - w) <= atol + rtol * np.abs(w))
    bad |= np.isnan(g) != np.isnan(w)
    assert not bad.any(), (
        f"{what}: {int(bad.sum())} of {bad.size} elements outside rtol={rtol} atol={atol}; "
        f"worst |diff|={np.nanmax(np.abs(g - w)):.4g}")


def assert_parity(y_got, r_got, y_want, r_want, what: str, max_y_ulp=1, max_y_mismatch=2e-3):
    """The bar of the path plus the tighter facts this implementation guarantees:
    the residual (fixed-order fp32 sum, one RNE rounding) is bit-exact; y differs from
    the checker only through the summation order of the mean of squares, i.e. by at
    most one bf16 ulp on a small fraction of elements."""
    assert_close_bits(y_got, y_want, what + " y")
    assert_close_bits(r_got, r_want, what + " residual")
    assert np.array_equal(r_got, r_want), f"{what}: residual differs in {(r_got != r_want).sum()} elements"
    d = ulp_distance(y_got, y_want)
    assert d.max() <= max_y_ulp, f"{what}: y off by {d.max()} ulp"
    frac = float((d != 0).mean())
    assert frac <= max_y_mismatch, f"{what}: {frac:.2%} of y elements differ by an ulp"


def bench_lib():
    """benchlib/libtw_bench.so (measurement and test-only kernels), or a skip when it has
    not been built.  Its error text comes from twb_last_error()."""
    import ctypes
    import os

    import pytest
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "benchlib", "libtw_bench.so")
    if not os.path.exists(path):
        pytest.skip(f"{path} has not been built (make -C benchlib)")
    L = ctypes.CDLL(path)
    vp, i64, ci, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
    L.twb_last_error.restype = ctypes.c_char_p
    L.twb_reduce_add_rms_norm_split_spread.argtypes = [ctypes.POINTER(vp), ci, vp, vp, vp, i64, i64, f32, ci, vp, vp]
    return L
