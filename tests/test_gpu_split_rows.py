"""The split-row kernel (several workgroups per token row, for decode-size batches)
against the one-workgroup-per-row kernel — bit for bit — and against the CPU checker,
through the C ABI."""
import ctypes

import numpy as np
import pytest
import torch

import tokenweave_amd as tw
from helpers import assert_parity, to_bits
from tokenweave_amd import _custom_ops as ops
from tokenweave_amd import _lib
from tokenweave_amd import workloads as wl

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make(P, T, H, seed=11):
    cfg = wl.NormConfig("split", P=P, T=T, H=H, eps=1e-5, seed=seed, partial_std=P ** -0.5)
    return cfg, wl.make_norm_inputs(cfg, DEV)


def run(inp, split, alias=0):
    parts = [p.clone() for p in inp.partials]
    res = inp.residual.clone()
    out = parts[alias] if alias is not None else torch.empty_like(res)
    ops.reduce_add_rms_norm(parts, out, res, inp.weight, inp.cfg.eps, None, split=split)
    torch.cuda.synchronize()
    return to_bits(out), to_bits(res)


@pytest.mark.parametrize("H", [6144, 8192])
@pytest.mark.parametrize("P", [1, 8])
@pytest.mark.parametrize("T", [1, 8, 32])
def test_decode_sizes_bit_identical_and_oracle_parity(oracle, T, P, H):
    """The decode sizes of the Llama-70B shard (hidden size 8192) take the split-row kernel;
    at hidden size 6144 the row is too short for the split to pay and the same entry point
    runs one workgroup per row."""
    print(f"[case] split T={T} P={P} H={H} segs={ops.split_segments(T, H)}", flush=True)
    assert (ops.split_segments(T, H) > 1) == (H == 8192)
    cfg, inp = make(P, T, H)
    y_s, r_s = run(inp, True)
    y_1, r_1 = run(inp, False)
    assert np.array_equal(y_s, y_1) and np.array_equal(r_s, r_1)
    y_w, r_w = oracle.reduce_add_rms_norm([to_bits(p) for p in inp.partials], to_bits(inp.residual),
                                          to_bits(inp.weight), cfg.eps)
    assert_parity(y_s, r_s, y_w, r_w, f"split T={T} P={P} H={H}")


@pytest.mark.parametrize("T,P,H", [(2, 2, 8192), (3, 3, 8200), (7, 5, 12288), (9, 16, 8192), (48, 8, 8192),
                                   (40, 4, 16384), (5, 7, 32768), (33, 8, 10240), (1, 8, 8192), (47, 2, 16392)])
def test_other_shapes_bit_identical(T, P, H):
    """Ragged last chunks (H = 8200: 1025 vectors, H = 16392: 2049), the longest rows of the
    vector kernel, run-time P, the largest row count that is split, eight-chunk segments."""
    print(f"[case] split T={T} P={P} H={H} segs={ops.split_segments(T, H)}", flush=True)
    assert ops.split_segments(T, H) > 1
    cfg, inp = make(P, T, H, seed=23)
    y_s, r_s = run(inp, True, alias=P - 1)
    y_1, r_1 = run(inp, False, alias=P - 1)
    assert np.array_equal(y_s, y_1) and np.array_equal(r_s, r_1)


@pytest.mark.parametrize("T,P,H", [(64, 8, 8192), (256, 8, 8192), (3, 3, 1032), (8, 2, 4096)])
def test_shapes_that_are_not_split_run_the_row_kernel(T, P, H):
    """More rows than pay, or rows too short to cut: the workspace entry point is the plain op."""
    assert ops.split_segments(T, H) == 1
    cfg, inp = make(P, T, H, seed=29)
    y_s, r_s = run(inp, True)
    y_1, r_1 = run(inp, False)
    assert np.array_equal(y_s, y_1) and np.array_equal(r_s, r_1)


def test_output_to_a_separate_buffer_and_repeated_calls_share_one_workspace():
    cfg, inp = make(8, 8, 8192, seed=31)
    want = run(inp, False, alias=None)
    for _ in range(5):
        got = run(inp, True, alias=None)
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
    # a larger, then a smaller batch through the same workspace
    for T in (32, 3):
        assert ops.split_segments(T, 8192) > 1
        cfg, inp = make(8, T, 8192, seed=32 + T)
        got, want = run(inp, True), run(inp, False)
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])


def test_reference_call_site_takes_the_split_kernel(oracle):
    """fused_allreduce_layernorm -> RMSNorm(fused_ar=True) -> fused_rs_ln_ag_cta with
    MAX_CTAS = 0 on a decode batch: same bits as the capped (one workgroup per row) call."""
    ws, rank, T, H = 8, 5, 16, 8192
    cfg, inp = make(ws, T, H, seed=41)
    layer = tw.RMSNorm(H, eps=cfg.eps, dtype=torch.bfloat16).to(DEV)
    layer.weight.data.copy_(inp.weight)
    outs = []
    for cap in (0, T):
        buf = tw.PartialsBuffer(ws, T, H, rank=rank, device=DEV)
        buf.storage.copy_(inp.staging)
        res = inp.residual.clone()
        y, r = layer(buf.hidden_states(T), res, MAX_CTAS=cap, fused_ar=True, symm_mem_hdl=buf, rank=rank,
                     world_size=ws, offset=0)
        torch.cuda.synchronize()
        outs.append((to_bits(y), to_bits(r)))
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])
    y_w, r_w = oracle.reduce_add_rms_norm([to_bits(p) for p in inp.partials], to_bits(inp.residual),
                                          to_bits(inp.weight), cfg.eps)
    assert_parity(outs[0][0], outs[0][1], y_w, r_w, "call site, split")


def test_graph_capture_and_replay_of_the_split_kernel():
    cfg, inp = make(8, 8, 8192, seed=51)
    want = run(inp, False, alias=None)
    parts = [p.clone() for p in inp.partials]
    res0 = inp.residual.clone()
    res = res0.clone()
    out = torch.empty_like(res)
    op = ops.bind_reduce_add_rms_norm(parts, out, res, inp.weight, cfg.eps, None, split=True)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        op()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        op()
    for _ in range(4):
        res.copy_(res0)
        out.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(to_bits(out), want[0]) and np.array_equal(to_bits(res), want[1])


def test_workspace_argument_checks():
    L = _lib.lib()
    cfg, inp = make(2, 4, 1024, seed=61)
    ptrs = (ctypes.c_void_p * 2)(*[p.data_ptr() for p in inp.partials])
    ws = torch.zeros(_lib.TW_SPLIT_WORKSPACE_BYTES + 256, dtype=torch.uint8, device=DEV)
    args = (ptrs, 2, inp.partials[0].data_ptr(), inp.residual.data_ptr(), inp.weight.data_ptr(), 4, 1024, 0, 1e-5)
    assert L.tw_reduce_add_rms_norm_ws(*args, ws.data_ptr(), 1024, None) == _lib.TW_ERR_INVALID_ARGUMENT
    assert "workspace" in _lib.last_error()
    assert L.tw_reduce_add_rms_norm_ws(*args, ws.data_ptr() + 16, _lib.TW_SPLIT_WORKSPACE_BYTES, None) == \
        _lib.TW_ERR_ALIGNMENT
    # no workspace: the plain op
    assert L.tw_reduce_add_rms_norm_ws(*args, None, 0, None) == _lib.TW_OK
    torch.cuda.synchronize()
    # a grid cap is honoured by not splitting
    assert ops.split_segments(8, 8192, 8) == 1
    assert ops.split_segments(4096, 8192) == 1
