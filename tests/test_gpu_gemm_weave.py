"""The weave configuration on a real GPU: the bf16 MFMA GEMM that produces a
rank's partial sum, and the two-stream step that overlaps it with the fused norm.

GEMM parity is against fp32 arithmetic on the CPU at rtol 1.6e-2 / atol 1e-2 (no
reference test pins torch.matmul's accumulation order for this call)."""
import numpy as np
import pytest
import torch

import tokenweave_amd as tw
from helpers import ATOL, RTOL, to_bits
from tokenweave_amd import _custom_ops as ops
from tokenweave_amd import workloads as wl

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def cpu_gemm(a, b):
    return (a.float().cpu() @ b.float().cpu().t())


def check(out, a, b, what):
    want = cpu_gemm(a, b)
    torch.testing.assert_close(out.float().cpu(), want, rtol=RTOL, atol=ATOL, msg=lambda m: f"{what}: {m}")


@pytest.mark.parametrize("M,N,K", [(1, 128, 64), (100, 128, 64), (129, 256, 128), (128, 136, 72),
                                   (257, 384, 1024), (333, 8192, 1024)])
def test_gemm_shapes_and_tails(M, N, K):
    print(f"[case] gemm M={M} N={N} K={K}", flush=True)
    g = wl.make_gemm_inputs(M, N, K, DEV, seed=M * 7 + N)
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16_nt(out, g.a, g.b)
    torch.cuda.synchronize()
    check(out, g.a, g.b, f"{M}x{N}x{K}")


def test_gemm_small_against_c_oracle(oracle):
    g = wl.make_gemm_inputs(70, 96, 160, DEV, seed=5, weight_std=1.0)
    out = torch.empty((70, 96), dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16_nt(out, g.a, g.b)
    torch.cuda.synchronize()
    want = oracle.gemm_bf16_nt(to_bits(g.a), to_bits(g.b))
    got = to_bits(out)
    f = lambda u: (u.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    assert np.all(np.abs(f(got) - f(want)) <= ATOL + RTOL * np.abs(f(want)))


def test_gemm_weave_shape_into_a_staging_slice_with_cu_cap():
    """Config 5's GEMM: [2458, 1024] x [8192, 1024]^T written into rows of a wider
    staging buffer, once uncapped and once on a capped grid; both must agree bitwise."""
    g = wl.make_gemm_inputs(device=DEV)
    M, N = g.a.shape[0], g.b.shape[0]
    stage = torch.zeros((wl.C5_TOTAL_TOKENS, N), dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16_nt(stage[:M], g.a, g.b)
    capped = torch.zeros_like(stage)
    ops.gemm_bf16_nt(capped[:M], g.a, g.b, max_cus=96)
    torch.cuda.synchronize()
    check(stage[:M], g.a, g.b, "weave gemm")
    assert torch.equal(stage, capped)
    assert not stage[M:].any(), "rows of the other split were touched"


def test_gemm_output_with_wide_row_stride():
    g = wl.make_gemm_inputs(65, 128, 64, DEV, seed=9)
    wide = torch.zeros((65, 256), dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16_nt(wide[:, :128], g.a, g.b)
    torch.cuda.synchronize()
    check(wide[:, :128], g.a, g.b, "ldc")
    assert not wide[:, 128:].any()


@pytest.mark.parametrize("M,N,K,ldc,shift", [
    (300, 256, 128, 512, 0),    # 16-byte stores into a slice of a wider buffer
    (300, 388, 128, 388, 0),    # N % 8 != 0: 8-byte stores
    (300, 384, 128, 388, 0),    # row stride % 8 != 0: 8-byte stores
    (300, 384, 128, 384, 4),    # out 8-byte but not 16-byte aligned: 8-byte stores
    (645, 520, 192, 520, 0),    # ragged tile edges in both directions, 16-byte stores
    (2048, 10240, 128, 10240, 0),   # 8 x 27 tiles of 256 x 384 fit one round of 256 compute units
    (2000, 10004, 128, 10004, 0),   # the same tile with ragged edges and 8-byte stores
    (2040, 10000, 192, 10008, 0),   # ... and with 16-byte stores into a wider buffer
])
def test_gemm_large_tile_kernel_store_paths(M, N, K, ldc, shift):
    print(f"[case] gemm stores M={M} N={N} K={K} ldc={ldc} shift={shift}", flush=True)
    g = wl.make_gemm_inputs(M, N, K, DEV, seed=M + N + ldc + shift)
    flat = torch.zeros(M * ldc + 16, dtype=torch.bfloat16, device=DEV)
    out = flat[shift:shift + M * ldc].view(M, ldc)[:, :N]
    ops.gemm_bf16_nt(out, g.a, g.b)
    torch.cuda.synchronize()
    check(out, g.a, g.b, "store path")
    if ldc > N:
        assert not flat[shift:shift + M * ldc].view(M, ldc)[:, N:].any(), "columns past N were written"
    assert not flat[:shift].any() and not flat[shift + M * ldc:].any()


@pytest.mark.parametrize("P,M,N,K,first_row,rows", [
    (8, 300, 512, 128, 0, 300),       # small: every tile kind of the big kernel's edges
    (8, 333, 8192, 1024, 200, 600),   # ragged M, the split starts at a non-zero staging row
    (3, 645, 520, 192, 7, 700),       # odd P, ragged tiles in both directions
    (2, 100, 128, 64, 5, 128),        # too small for the big kernel: one launch per product
])
def test_partials_producer_writes_every_rank_slot(P, M, N, K, first_row, rows):
    """tw_gemm_bf16_nt_partials: the P partial sums of a token split land in rows
    [first_row, first_row + M) of the P staging slots — each against fp32 CPU arithmetic,
    bit-identical to P separate tw_gemm_bf16_nt calls, nothing else touched."""
    print(f"[case] partials P={P} M={M} N={N} K={K} first_row={first_row}", flush=True)
    gs = wl.make_partials_gemm_inputs(P, M, N, K, DEV, seed=P * 1000 + M)
    buf = tw.PartialsBuffer(P, rows, N, rank=0, device=DEV)
    buf.storage.fill_(float("nan"))
    outs = [buf.slot(p)[first_row:first_row + M] for p in range(P)]
    ops.gemm_bf16_nt_partials(outs, [g.a for g in gs], [g.b for g in gs])
    one = tw.PartialsBuffer(P, rows, N, rank=0, device=DEV)
    one.storage.fill_(float("nan"))
    for p in range(P):
        ops.gemm_bf16_nt(one.slot(p)[first_row:first_row + M], gs[p].a, gs[p].b)
    torch.cuda.synchronize()
    for p in range(P):
        check(outs[p], gs[p].a, gs[p].b, f"slot {p}")
    assert torch.equal(buf.storage.view(torch.int16), one.storage.view(torch.int16))
    assert torch.isnan(buf.storage[:, :first_row]).all() and torch.isnan(buf.storage[:, first_row + M:]).all()


def test_partials_producer_feeds_the_fused_norm(oracle):
    """Producer and consumer through one staging buffer: the GEMMs' partial sums are what
    the fused op reads, with no copy in between; checked against the CPU checker fed with
    the GEMM outputs."""
    P, M, N, K = 8, 96, 8192, 256
    gs = wl.make_partials_gemm_inputs(P, M, N, K, DEV, seed=77, weight_std=0.05)
    buf = tw.PartialsBuffer(P, M, N, rank=1, device=DEV)
    ops.gemm_bf16_nt_partials([buf.slot(p) for p in range(P)], [g.a for g in gs], [g.b for g in gs])
    torch.cuda.synchronize()
    parts = [to_bits(buf.slot(p)) for p in range(P)]
    residual = torch.randn(M, N, device=DEV).to(torch.bfloat16)
    r0 = to_bits(residual)
    layer = tw.RMSNorm(N, eps=1e-5, dtype=torch.bfloat16).to(DEV)
    y, r = layer(buf.hidden_states(M), residual, MAX_CTAS=0, fused_ar=True, symm_mem_hdl=buf, rank=1,
                 world_size=P, offset=0)
    torch.cuda.synchronize()
    y_want, r_want = oracle.reduce_add_rms_norm(parts, r0, to_bits(layer.weight.data), 1e-5)
    assert np.array_equal(to_bits(r), r_want)
    from helpers import ulp_distance
    assert ulp_distance(to_bits(y), y_want).max() <= 1


def test_partials_producer_argument_checks():
    gs = wl.make_partials_gemm_inputs(2, 64, 128, 64, DEV, seed=3)
    out = [torch.empty((64, 128), dtype=torch.bfloat16, device=DEV) for _ in range(2)]
    with pytest.raises(RuntimeError, match="one entry per partial"):
        ops.gemm_bf16_nt_partials(out, [gs[0].a], [g.b for g in gs])
    with pytest.raises(RuntimeError, match="partial 1 has"):
        ops.gemm_bf16_nt_partials([out[0], out[1][:32]], [gs[0].a, gs[1].a[:32]], [g.b for g in gs])
    with pytest.raises(RuntimeError, match="not in"):
        ops.gemm_bf16_nt_partials([], [], [])


def test_config5_stage_at_full_size_equals_serial_execution():
    """The weave configuration as it is benchmarked: the producer GEMM of the 2458-row
    split (all eight partials, and the single-partial form) on the current stream while
    the fused norm of the 1638-row split runs on a second stream — same bits as running
    them in turn, and the GEMM against fp32 CPU arithmetic."""
    P, H, K = 8, 8192, wl.C5_GEMM_K
    T, Ta = wl.C5_TOTAL_TOKENS, wl.C5_GEMM_ROWS
    cfg = wl.C5_NORM
    inp = wl.make_norm_inputs(cfg, DEV)
    gs = wl.make_partials_gemm_inputs(P, Ta, H, K, DEV)
    layer = tw.RMSNorm(H, eps=cfg.eps, dtype=torch.bfloat16).to(DEV)
    layer.weight.data.copy_(inp.weight)
    rank = 3

    def setup():
        buf = tw.PartialsBuffer(P, T, H, rank=rank, device=DEV)
        buf.storage.zero_()
        buf.storage[:, Ta:] = inp.staging
        residual = torch.zeros(T, H, dtype=torch.bfloat16, device=DEV)
        residual[Ta:] = inp.residual
        return buf, residual

    def norm(buf, residual):
        layer(buf.local[Ta:], residual[Ta:], MAX_CTAS=0, fused_ar=True, symm_mem_hdl=buf, rank=rank,
              world_size=P, offset=buf.offset_of_row(Ta))

    def gemm8(buf, cus=None):
        ops.gemm_bf16_nt_partials([buf.slot(p)[:Ta] for p in range(P)], [g.a for g in gs], [g.b for g in gs], cus)

    def gemm1(buf, cus=None):
        ops.gemm_bf16_nt(buf.local[:Ta], gs[rank].a, gs[rank].b, cus)

    side = torch.cuda.Stream()
    for name, gemm in (("eight partials", gemm8), ("one partial", gemm1)):
        print(f"[case] config 5 stage, {name}", flush=True)
        buf1, res1 = setup()
        gemm(buf1)
        norm(buf1, res1)
        torch.cuda.synchronize()
        buf2, res2 = setup()
        tw.weave_norm_gemm(lambda: gemm(buf2, 128), lambda: norm(buf2, res2), side, gemm_first=True)
        torch.cuda.synchronize()
        assert torch.equal(buf1.storage.view(torch.int16), buf2.storage.view(torch.int16)), name
        assert torch.equal(res1.view(torch.int16), res2.view(torch.int16)), name
        check(buf2.local[:Ta], gs[rank].a, gs[rank].b, f"config 5 gemm ({name})")
        if gemm is gemm8:
            check(buf2.slot(0)[:Ta], gs[0].a, gs[0].b, "config 5 gemm, slot 0")


def test_weave_step_equals_serial_execution():
    """GEMM of split A on the current stream while split B's fused norm runs on a
    second stream (tokenweave_utils.py:236-260): same bits as running them in turn."""
    ws, H, T = 8, 8192, 512
    Ta = tw.tokenweave_split_size(T)  # 256
    Tb = T - Ta
    cfg = wl.C5_NORM.with_tokens(Tb)
    inp = wl.make_norm_inputs(cfg, DEV)
    g = wl.make_gemm_inputs(Ta, H, 1024, DEV)
    layer = tw.RMSNorm(H, eps=cfg.eps, dtype=torch.bfloat16).to(DEV)
    layer.weight.data.copy_(inp.weight)

    def setup():
        buf = tw.PartialsBuffer(ws, T, H, rank=2, device=DEV)
        buf.storage.zero_()
        buf.storage[:, Ta:] = inp.staging
        residual = torch.zeros(T, H, dtype=torch.bfloat16, device=DEV)
        residual[Ta:] = inp.residual
        return buf, residual

    def norm(buf, residual):
        layer(buf.local[Ta:], residual[Ta:], MAX_CTAS=64, fused_ar=True, symm_mem_hdl=buf, rank=2,
              world_size=ws, offset=buf.offset_of_row(Ta))

    def gemm(buf):
        ops.gemm_bf16_nt(buf.local[:Ta], g.a, g.b, max_cus=192)

    buf1, res1 = setup()
    gemm(buf1)
    norm(buf1, res1)
    torch.cuda.synchronize()
    buf2, res2 = setup()
    side = torch.cuda.Stream()
    for gemm_first in (True, False, True):  # the step is idempotent on split A; split B is reset each time
        buf2.storage[:, Ta:] = inp.staging
        res2[Ta:] = inp.residual
        tw.weave_norm_gemm(lambda: gemm(buf2), lambda: norm(buf2, res2), side, gemm_first=gemm_first)
        torch.cuda.synchronize()
        assert torch.equal(buf1.storage, buf2.storage) and torch.equal(res1, res2)
    check(buf2.local[:Ta], g.a, g.b, "weave gemm split")
