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


# ---------------------------------------------------------------------------
# bias of the in-place linear (vllm/model_executor/layers/linear.py:224-228) and the
# RowParallelLinear call surface (linear.py:1290-1334)
# ---------------------------------------------------------------------------
def reference_linear_inplace(a, b, bias):
    """The reference's two steps on the CPU: the product rounded to bf16
    (torch.matmul(..., out=bf16)), then `output += bias` in bf16 arithmetic (fp32 add, one
    more rounding).  The product is taken from `a @ b.T` in fp32."""
    prod = (a.float().cpu() @ b.float().cpu().t()).to(torch.bfloat16)
    return prod if bias is None else (prod.float() + bias.float().cpu()).to(torch.bfloat16)


@pytest.mark.parametrize("M,N,K,ldc,shift", [
    (100, 128, 64, 128, 0),          # fallback kernel
    (129, 256, 72, 256, 0),          # fallback kernel, K % 64 != 0
    (300, 384, 128, 384, 0),         # big kernel, 16-byte stores
    (300, 388, 128, 388, 0),         # big kernel, 8-byte stores (N % 8 != 0)
    (300, 384, 128, 384, 4),         # big kernel, out not 16-byte aligned
    (2458, 8192, 1024, 8192, 0),     # config 5's shape
    (2048, 10240, 128, 10240, 0),    # 256 x 384 tiles
])
def test_gemm_bias_matches_the_reference_two_step_arithmetic(M, N, K, ldc, shift):
    """out = bf16(bf16(a b^T) + bias): against fp32 CPU arithmetic within the path's
    tolerance, and BIT-identical to adding the bias in bf16 to the library's own
    bias-free product — the reference's `output += bias` on top of its matmul."""
    print(f"[case] gemm bias M={M} N={N} K={K} ldc={ldc} shift={shift}", flush=True)
    g = wl.make_gemm_inputs(M, N, K, DEV, seed=M + N + K + shift)
    gen = torch.Generator(device=DEV)
    gen.manual_seed(M * 31 + N)
    bias = torch.randn(N, generator=gen, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    flat = torch.zeros(M * ldc + 16, dtype=torch.bfloat16, device=DEV)
    out = flat[shift:shift + M * ldc].view(M, ldc)[:, :N]
    plain = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16_nt(out, g.a, g.b, bias=bias)
    ops.gemm_bf16_nt(plain, g.a, g.b)
    torch.cuda.synchronize()
    assert torch.equal(out, plain + bias), "fused bias differs from `output += bias` on the bias-free product"
    want = reference_linear_inplace(g.a, g.b, bias)
    torch.testing.assert_close(out.float().cpu(), want.float(), rtol=RTOL, atol=ATOL)
    assert not flat[:shift].any() and not flat[shift + M * ldc:].any()


def test_gemm_bias_argument_checks():
    g = wl.make_gemm_inputs(64, 128, 64, DEV, seed=3)
    out = torch.empty((64, 128), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="bias has shape"):
        ops.gemm_bf16_nt(out, g.a, g.b, bias=torch.zeros(64, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(RuntimeError, match="dtype"):
        ops.gemm_bf16_nt(out, g.a, g.b, bias=torch.zeros(128, dtype=torch.float32, device=DEV))
    odd = torch.zeros(130, dtype=torch.bfloat16, device=DEV)[1:129]   # 2-byte aligned only
    with pytest.raises(RuntimeError, match="aligned"):
        ops.gemm_bf16_nt(out, g.a, g.b, bias=odd)


def test_partials_producer_adds_only_rank_zero_bias():
    """One GPU standing in for the ranks: biases = [b, None, ...] puts the bias into slot 0
    only, bit-identical to per-rank calls, so the P-way sum holds it once."""
    P, M, N, K = 4, 333, 512, 128
    gs = wl.make_partials_gemm_inputs(P, M, N, K, DEV, seed=77)
    bias = torch.linspace(-2, 2, N, device=DEV).to(torch.bfloat16)
    buf = tw.PartialsBuffer(P, M, N, rank=0, device=DEV)
    ops.gemm_bf16_nt_partials([buf.slot(p)[:M] for p in range(P)], [g.a for g in gs], [g.b for g in gs],
                              biases=[bias] + [None] * (P - 1))
    torch.cuda.synchronize()
    for p in range(P):
        one = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
        ops.gemm_bf16_nt(one, gs[p].a, gs[p].b, bias=bias if p == 0 else None)
        torch.cuda.synchronize()
        assert torch.equal(buf.slot(p)[:M], one), f"slot {p}"


@pytest.mark.parametrize("with_bias", [False, True])
def test_row_parallel_linear_tokenweave_call_site(oracle, with_bias):
    """llama.py:248-249 on one GPU: every rank's o_proj writes its partial sum in place into
    its staging rows (`forward(x_p, output_=rows, is_tokenweave=True)`), the fused norm
    reduces them.  Against fp32 `x @ W.T + b` per rank, and against the CPU checker fed
    with the staged partials."""
    ws, T, H, Kfull = 4, 200, 1024, 1024
    gen = torch.Generator(device=DEV)
    gen.manual_seed(91 + with_bias)
    W = (torch.randn(H, Kfull, generator=gen, device=DEV) * 0.03).to(torch.bfloat16)
    b = torch.randn(H, generator=gen, device=DEV).to(torch.bfloat16)
    x = torch.randn(T, Kfull, generator=gen, device=DEV).to(torch.bfloat16)
    buf = tw.PartialsBuffer(ws, T, H, rank=0, device=DEV)
    layers = []
    for p in range(ws):
        lin = tw.RowParallelLinear(Kfull, H, bias=with_bias, tp_rank=p, tp_size=ws).to(DEV)
        lin.weight_loader(lin.weight, W)
        if with_bias:
            lin.weight_loader(lin.bias, b)
        layers.append(lin)
        shard = Kfull // ws
        xp = x[:, p * shard:(p + 1) * shard].contiguous()
        out, out_bias = lin(xp, buf.slot(p)[:T], is_tokenweave=True)
        assert out.data_ptr() == buf.slot(p).data_ptr() and out_bias is None
        torch.cuda.synchronize()
        want = xp.float().cpu() @ lin.weight.data.float().cpu().t()
        if with_bias and p == 0:
            want = want + b.float().cpu()
        torch.testing.assert_close(out.float().cpu(), want, rtol=RTOL, atol=ATOL)
    # input_is_parallel=False slices the full activation itself
    lin = tw.RowParallelLinear(Kfull, H, bias=False, input_is_parallel=False, tp_rank=2, tp_size=ws).to(DEV)
    lin.weight_loader(lin.weight, W)
    out2 = torch.empty((T, H), dtype=torch.bfloat16, device=DEV)
    lin(x, out2, is_tokenweave=True)
    torch.cuda.synchronize()
    assert torch.equal(out2, buf.slot(2)[:T])
    # the fused op on the staged partials
    parts = [to_bits(buf.slot(p)[:T]) for p in range(ws)]
    res = torch.randn(T, H, generator=gen, device=DEV).to(torch.bfloat16)
    res_bits = to_bits(res)
    norm = tw.RMSNorm(H, eps=1e-5, dtype=torch.bfloat16).to(DEV)
    tw.fused_allreduce_layernorm(norm, buf.hidden_states(T), res, buf, T // ws, 0, ws, 0, row_range=(0, T))
    torch.cuda.synchronize()
    y_w, r_w = oracle.reduce_add_rms_norm(parts, res_bits, to_bits(norm.weight.data), 1e-5)
    assert np.array_equal(to_bits(res), r_w)
    f = lambda u: (u.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    assert np.all(np.abs(f(to_bits(buf.hidden_states(T))) - f(y_w)) <= ATOL + RTOL * np.abs(f(y_w)))


def test_row_parallel_linear_default_mode_and_skip_bias_add():
    T, H, K = 64, 256, 128
    gen = torch.Generator(device=DEV)
    gen.manual_seed(17)
    x = torch.randn(T, K, generator=gen, device=DEV).to(torch.bfloat16)
    lin = tw.RowParallelLinear(K, H, bias=True, skip_bias_add=True).to(DEV)
    lin.weight.data.copy_((torch.randn(H, K, generator=gen, device=DEV) * 0.05).to(torch.bfloat16))
    lin.bias.data.copy_(torch.randn(H, generator=gen, device=DEV).to(torch.bfloat16))
    out, out_bias = lin(x)                      # default mode, tp_size 1: a fresh output, bias handed back
    torch.cuda.synchronize()
    assert out_bias is lin.bias
    torch.testing.assert_close(out.float().cpu(), x.float().cpu() @ lin.weight.data.float().cpu().t(),
                               rtol=RTOL, atol=ATOL)
    with pytest.raises(AssertionError, match="preallocated"):
        lin(x, None, is_tokenweave=True)
    multi = tw.RowParallelLinear(K * 2, H, bias=False, tp_rank=1, tp_size=2).to(DEV)
    with pytest.raises(RuntimeError, match="no collectives"):
        multi(x)


def test_tuner_returns_a_well_formed_table():
    """tune() on one small token count, two offsets, few rounds: the table has the layout
    load_config / weave_plan read, and the budgets come from the measured grid."""
    from tokenweave_amd import tune_weave
    lines = []
    table = tune_weave.tune(2048, 256, 4, [1024], offsets=(0, 128), device=DEV, log=lines.append, k_mlp=512,
                            regions=2, stage_budget_us=300.0)
    assert set(table) == {"1024"}
    e = table["1024"]
    assert set(e) == {"attention_ctas", "mlp_ctas", "split_offset", "gemm_cus", "mlp_gemm_cus", "overlap"}
    cus = ops.num_compute_units(DEV)
    assert e["split_offset"] in (0, 128) and e["overlap"] in (0, 1)
    assert e["attention_ctas"] in (0, cus // 2) and e["mlp_ctas"] in (0, cus // 2)
    assert 0 <= e["gemm_cus"] <= cus and 0 <= e["mlp_gemm_cus"] <= cus
    assert any("split_offset=" in ln for ln in lines)
    plan = tw.weave_plan(1024, {1024: e})
    assert plan is None or plan["split_size"] == tw.tokenweave_split_size(1024, e["split_offset"])


@pytest.mark.parametrize("M,N,K", [(300, 384, 72), (300, 384, 200), (645, 520, 136), (2458, 8192, 3696),
                                   (1024, 8192, 7392), (333, 256, 1000), (2048, 10240, 328)])
def test_gemm_inner_dimension_not_a_multiple_of_the_slab(M, N, K):
    """K % 64 != 0 on the large-tile kernel (Qwen2's row-parallel MLP slices are 3696 and
    7392 wide): the last k-slab's chunks past K are zero-filled.  Against fp32 CPU arithmetic,
    and BIT-identical to the same product with both operands zero-padded to a whole number
    of slabs (the padded columns add exact zeros in the same k-steps)."""
    print(f"[case] gemm K tail M={M} N={N} K={K}", flush=True)
    g = wl.make_gemm_inputs(M, N, K, DEV, seed=M + N + K)
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16_nt(out, g.a, g.b)
    Kp = (K + 63) // 64 * 64
    ap = torch.zeros((M, Kp), dtype=torch.bfloat16, device=DEV)
    bp = torch.zeros((N, Kp), dtype=torch.bfloat16, device=DEV)
    ap[:, :K] = g.a
    bp[:, :K] = g.b
    padded = torch.empty_like(out)
    ops.gemm_bf16_nt(padded, ap, bp)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), padded.view(torch.int16)), "differs from the zero-padded product"
    if M * N * K <= 2458 * 8192 * 3696:
        check(out, g.a, g.b, f"K tail {M}x{N}x{K}")
