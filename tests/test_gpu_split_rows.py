"""The split-row kernel (several workgroups per token row, for decode-size batches)
against the one-workgroup-per-row kernel — bit for bit — and against the CPU checker,
through the C ABI."""
import ctypes

import numpy as np
import pytest
import torch

import tokenweave_amd as tw
from helpers import assert_parity, bench_lib, to_bits
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


def run_spread(L, inp, seg_waves, ws, alias=0):
    """The split-row kernel with the segments of a row on consecutive workgroups, i.e. on
    different XCDs (the measurement library's form; the product keeps a row on one XCD)."""
    cfg = inp.cfg
    parts = [p.clone() for p in inp.partials]
    res = inp.residual.clone()
    out = parts[alias] if alias is not None else torch.empty_like(res)
    ptrs = (ctypes.c_void_p * cfg.P)(*[p.data_ptr() for p in parts])
    rc = L.twb_reduce_add_rms_norm_split_spread(ptrs, cfg.P, out.data_ptr(), res.data_ptr(), inp.weight.data_ptr(),
                                                cfg.T, cfg.H, cfg.eps, seg_waves, ws.data_ptr(),
                                                torch.cuda.current_stream().cuda_stream)
    assert rc == 0, L.twb_last_error().decode()
    torch.cuda.synchronize()
    return to_bits(out), to_bits(res)


@pytest.mark.parametrize("seg_waves", [4, 8])
@pytest.mark.parametrize("T,P,H", [(1, 8, 8192), (8, 8, 8192), (32, 8, 8192), (32, 1, 8192), (48, 8, 8192),
                                   (3, 3, 8200), (7, 5, 12288), (9, 16, 8192), (40, 4, 16384), (5, 7, 32768),
                                   (47, 2, 16392), (256, 8, 8192), (2, 2, 1024)])
def test_segments_spread_over_xcds_bit_identical(T, P, H, seg_waves):
    """The hand-over between the segment workgroups of a row does not depend on their
    sharing an XCD: with the segments of every row spread over the XCDs the results are the
    one-workgroup kernel's, bit for bit, five launches in a row on one workspace."""
    L = bench_lib()
    if (H // 8 + 63) // 64 <= seg_waves:
        pytest.skip("the row is a single segment of this size")
    print(f"[case] spread split T={T} P={P} H={H} waves per segment={seg_waves}", flush=True)
    cfg, inp = make(P, T, H, seed=71)
    want = run(inp, False, alias=P - 1)
    ws = torch.zeros(_lib.TW_SPLIT_WORKSPACE_BYTES, dtype=torch.uint8, device=DEV)
    for i in range(5):
        got = run_spread(L, inp, seg_waves, ws, alias=P - 1)
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1]), f"launch {i}"
    assert int(ws.view(torch.int32).view(-1, 96)[:, 64].abs().max()) == 0, "an arrival counter was left non-zero"


@pytest.mark.parametrize("form,launches", [("product", 3072), ("spread", 1536)])
def test_soak_alternating_decode_shapes_on_one_workspace(form, launches):
    """A few thousand back-to-back launches of the split-row kernel on ONE workspace,
    alternating between the decode shapes (1 .. 48 rows, hidden size 8192 / 16384, one and
    eight partials), every result compared with the one-workgroup kernel's bits on the GPU.
    The launches of a block of 128 are not separated by host synchronisation (the next
    launch follows as closely as the queue allows, which is when a stale value left by the
    previous one would be seen); the run stops at the first block that holds a mismatch and
    names its first launch."""
    L = bench_lib() if form == "spread" else None
    shapes = [(T, P, H) for H in (8192, 16384) for P in (1, 8) for T in (1, 8, 32, 48)]
    ws = torch.zeros(_lib.TW_SPLIT_WORKSPACE_BYTES, dtype=torch.uint8, device=DEV)
    cases = []
    for i, (T, P, H) in enumerate(shapes):
        assert ops.split_segments(T, H) > 1
        cfg, inp = make(P, T, H, seed=300 + i)
        y_w, r_w = run(inp, False, alias=None)
        res = inp.residual.clone()
        out = torch.empty_like(res)
        ptrs = (ctypes.c_void_p * P)(*[p.data_ptr() for p in inp.partials])
        cases.append(dict(cfg=cfg, inp=inp, res=res, out=out, ptrs=ptrs,
                          y_want=torch.from_numpy(y_w.view(np.int16)).to(DEV),
                          r_want=torch.from_numpy(r_w.view(np.int16)).to(DEV)))
    lib = _lib.lib()
    sp = torch.cuda.current_stream().cuda_stream
    block = 128
    flags = torch.zeros(block, dtype=torch.int32, device=DEV)
    rng = np.random.default_rng(5)
    order = rng.integers(0, len(cases), size=launches)
    for b0 in range(0, launches, block):
        flags.zero_()
        for j, ci in enumerate(order[b0:b0 + block]):
            c = cases[ci]
            cfg = c["cfg"]
            c["res"].copy_(c["inp"].residual)
            if form == "spread":
                rc = L.twb_reduce_add_rms_norm_split_spread(c["ptrs"], cfg.P, c["out"].data_ptr(),
                                                            c["res"].data_ptr(), c["inp"].weight.data_ptr(), cfg.T,
                                                            cfg.H, cfg.eps, 4 if ci % 2 else 8, ws.data_ptr(), sp)
                assert rc == 0, L.twb_last_error().decode()
            else:
                rc = lib.tw_reduce_add_rms_norm_ws(c["ptrs"], cfg.P, c["out"].data_ptr(), c["res"].data_ptr(),
                                                   c["inp"].weight.data_ptr(), cfg.T, cfg.H, 0, cfg.eps,
                                                   ws.data_ptr(), ws.numel(), sp)
                assert rc == 0, _lib.last_error()
            bad = (c["out"].view(torch.int16) != c["y_want"]).any() | (c["res"].view(torch.int16) != c["r_want"]).any()
            flags[j] = bad.to(torch.int32)
        f = flags.cpu().numpy()
        if f.any():
            j = int(np.flatnonzero(f)[0])
            T, P, H = shapes[order[b0 + j]]
            pytest.fail(f"{form}: launch {b0 + j} (T={T} P={P} H={H}) differs from the one-workgroup kernel; "
                        f"{int(f.sum())} of the block's {len(f)} launches differ")
    assert int(ws.view(torch.int32).view(-1, 96)[:, 64].abs().max()) == 0, "an arrival counter was left non-zero"


# ---------------------------------------------------------------------------
# mixed launch: a few more rows than compute units
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("H", [8192, 6144, 4608, 2048])
@pytest.mark.parametrize("P", [1, 8, 3])
@pytest.mark.parametrize("extra", [1, 8, 13, 32, 47, 64])
def test_mixed_launch_bit_identical(extra, P, H):
    """C + extra rows (extra <= C / 4) on a GPU with C compute units: the workspace entry
    point gives the first C rows a workgroup each and cuts the excess rows into quarters, a
    workgroup each.  Same bits as one workgroup per row, twice in a row on one workspace."""
    cus = ops.num_compute_units(DEV)
    T = cus + extra
    segs = ops.split_segments(T, H)
    print(f"[case] mixed T={T} P={P} H={H} segments per excess row={segs}", flush=True)
    assert segs == (2 if H == 4608 else 4)   # rows of 9 chunks on 3 waves are halved, not quartered
    cfg, inp = make(P, T, H, seed=80 + extra)
    want = run(inp, False, alias=P - 1)
    for i in range(2):
        got = run(inp, True, alias=P - 1)
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1]), f"call {i}"


def test_mixed_launch_limits_and_oracle_parity(oracle):
    cus = ops.num_compute_units(DEV)
    assert ops.split_segments(cus, 8192) == 1                    # exactly one row per unit: nothing to balance
    assert ops.split_segments(cus + cus // 4 + 1, 8192) == 1     # quarters would queue two deep on a unit
    assert ops.split_segments(cus + 8, 8192, MAX_CTAS=64) == 1   # a grid cap is honoured by not cutting rows
    assert ops.split_segments(cus + 8, 16384) == 1               # rows of more than 1024 vectors: other shape
    assert ops.split_segments(cus + 8, 8200) == 1
    T = cus + 45
    cfg, inp = make(8, T, 8192, seed=97)
    y, r = run(inp, None)                                        # the default route of the public op
    y_w, r_w = oracle.reduce_add_rms_norm([to_bits(p) for p in inp.partials], to_bits(inp.residual),
                                          to_bits(inp.weight), cfg.eps)
    assert_parity(y, r, y_w, r_w, f"mixed T={T}")


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
