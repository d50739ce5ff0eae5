"""tw_reduce_add_rms_norm_noalloc — the split-row op on the library's static device
workspace — against tw_reduce_add_rms_norm_ws with a caller's workspace: bit for bit,
through the C ABI, on two calls in a row, the second on a smaller batch."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import to_bits
from tokenweave_amd import _lib
from tokenweave_amd import workloads as wl

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def call(entry, inp, extra):
    """Runs `entry` on clones of the inputs; returns (y bits, residual bits)."""
    cfg = inp.cfg
    parts = [p.clone() for p in inp.partials]
    res = inp.residual.clone()
    ptrs = (ctypes.c_void_p * cfg.P)(*[p.data_ptr() for p in parts])
    sp = torch.cuda.current_stream().cuda_stream
    rc = entry(ptrs, cfg.P, parts[0].data_ptr(), res.data_ptr(), inp.weight.data_ptr(), cfg.T, cfg.H, 0,
               cfg.eps, *extra, sp)
    assert rc == _lib.TW_OK, _lib.last_error()
    torch.cuda.synchronize()
    return to_bits(parts[0]), to_bits(res)


def test_no_alloc_entry_point_matches_the_workspace_entry_point():
    L = _lib.lib()
    torch.cuda.set_device(0)
    ws = torch.zeros(_lib.TW_SPLIT_WORKSPACE_BYTES, dtype=torch.uint8, device=DEV)
    for T, H, seed in ((32, 8192, 71), (8, 8192, 72), (40, 16384, 73), (3, 8200, 74), (200, 8192, 75)):
        print(f"[case] no-alloc T={T} H={H} segs={L.tw_split_segments(T, H, 0)}", flush=True)
        cfg = wl.NormConfig("noalloc", P=8, T=T, H=H, eps=1e-5, seed=seed, partial_std=8 ** -0.5)
        inp = wl.make_norm_inputs(cfg, DEV)
        before = torch.cuda.memory_allocated()
        y_n, r_n = call(L.tw_reduce_add_rms_norm_noalloc, inp, ())
        assert torch.cuda.memory_allocated() == before
        y_w, r_w = call(L.tw_reduce_add_rms_norm_ws, inp, (ws.data_ptr(), ws.numel()))
        assert np.array_equal(y_n, y_w), f"T={T} H={H}: y differs in {(y_n != y_w).sum()} elements"
        assert np.array_equal(r_n, r_w), f"T={T} H={H}: residual differs in {(r_n != r_w).sum()} elements"
    # the first two cases took the split-row kernel (the static workspace was in use)
    assert L.tw_split_segments(32, 8192, 0) > 1 and L.tw_split_segments(8, 8192, 0) > 1


def test_no_alloc_entry_point_refuses_more_rows_than_its_workspace_holds():
    L = _lib.lib()
    torch.cuda.set_device(0)
    T, H = _lib.TW_SPLIT_MAX_TOKENS + 1, 1024
    x = torch.zeros((T, H), dtype=torch.bfloat16, device=DEV)
    r = torch.zeros_like(x)
    w = torch.ones(H, dtype=torch.bfloat16, device=DEV)
    ptrs = (ctypes.c_void_p * 1)(x.data_ptr())
    rc = L.tw_reduce_add_rms_norm_noalloc(ptrs, 1, x.data_ptr(), r.data_ptr(), w.data_ptr(), T, H, 0, 1e-5, None)
    assert rc == _lib.TW_ERR_INVALID_ARGUMENT
    assert "exceeds" in _lib.last_error() and str(_lib.TW_SPLIT_MAX_TOKENS) in _lib.last_error()
    torch.cuda.synchronize()
