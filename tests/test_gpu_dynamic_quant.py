"""Norm + dynamic per-token quantisation (fp8 e4m3fn / int8) on a real GPU.

The reference's own unit test (tests/kernels/test_fused_quant_layernorm.py:107-160)
compares the fused op with `forward_native` followed by the unfused per-token
quantisation: scales at allclose's default tolerance, fp8 codes equal as floats, int8
codes within one step, the residual equal.  The same grid and the same composition
are used here (in torch, on the GPU), and bf16 results are also compared with the CPU
checker's restatement of the reference kernel, P partials included."""
import numpy as np
import pytest
import torch

from helpers import to_bits
from tokenweave_amd import _custom_ops as ops
from tokenweave_amd import workloads as wl

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
FP8 = torch.float8_e4m3fn
EPS = 1e-6

VEC_HIDDEN_SIZES = range(1024, 1030)
NUM_TOKENS_HIDDEN_SIZES = [   # test_fused_quant_layernorm.py:15-21
    *[(1, i) for i in [1, 64, *VEC_HIDDEN_SIZES, 5120, 5137]],
    *[(83, i) for i in [1, 1033, 2048, 5120]],
    *[(2048, i) for i in [1, 64, *VEC_HIDDEN_SIZES, 5137]],
    *[(4096, i) for i in [1, 64, 5137]],
]


def forward_native(x, residual, weight, eps):
    """vllm/model_executor/layers/layernorm.py:173-210."""
    orig = x.dtype
    x32 = x.float()
    if residual is not None:
        x32 = x32 + residual.float()
        residual = x32.to(orig)
    var = x32.pow(2).mean(dim=-1, keepdim=True)
    y = (x32 * torch.rsqrt(var + eps)).to(orig) * weight
    return y, residual


def composed_quant(y, quant_dtype, scale_ub):
    """Unfused per-token quantisation: csrc/quantization/fp8/common.cu:29-90 (fp8),
    the fused kernel's own int8 rule for int8 (scale floor FLT_EPSILON, inverted scale)."""
    n = y.float()
    amax = n.abs().amax(dim=-1, keepdim=True)
    if quant_dtype == FP8:
        s = amax if scale_ub is None else torch.minimum(amax, scale_ub)
        scales = torch.clamp(s / 448.0, min=1.0 / (448.0 * 512.0))
        return (n / scales).clamp(-448.0, 448.0).to(FP8), scales
    scales = torch.clamp(amax / 127.0, min=torch.finfo(torch.float32).eps)
    return torch.round(n * (1.0 / scales)).clamp(-128, 127).to(torch.int8), scales


def code_line(codes: torch.Tensor, quant_dtype) -> np.ndarray:
    """Codes on a monotone integer line (fp8 codes are sign-magnitude)."""
    a = codes.view(torch.int8).cpu().numpy().astype(np.int32)
    return np.where(a < 0, -(a & 0x7F), a) if quant_dtype == FP8 else a


def assert_codes_and_scales(got, got_scales, want, want_scales, quant_dtype, what):
    gs, ws = got_scales.cpu().numpy().reshape(-1), want_scales.cpu().numpy().reshape(-1)
    rel = np.abs(gs - ws) / ws
    # a last-bit difference in the mean of squares can move one rounding of the row
    # maximum: at most one step of the input type, in few rows
    assert rel.max() <= 2.0 ** -7, f"{what}: scale off by {rel.max():.3g}"
    assert (rel > 1e-5).mean() <= 0.02 or (rel > 1e-5).sum() <= 1, f"{what}: {(rel > 1e-5).sum()} rows differ"
    same = rel <= 1e-5
    d = np.abs(code_line(got, quant_dtype) - code_line(want, quant_dtype))[same]
    if d.size:
        assert d.max() <= 1, f"{what}: code off by {d.max()} steps"
        assert (d != 0).mean() <= 5e-3, f"{what}: {(d != 0).mean():.2%} of codes differ"


@pytest.mark.parametrize("num_tokens,hidden_size", NUM_TOKENS_HIDDEN_SIZES)
@pytest.mark.parametrize("add_residual", [False, True])
@pytest.mark.parametrize("use_ub", [True, False])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float, torch.half])
@pytest.mark.parametrize("quant_dtype", [torch.int8, FP8])
def test_reference_grid_against_composition(num_tokens, hidden_size, add_residual, use_ub, dtype, quant_dtype):
    if use_ub and quant_dtype != FP8:
        pytest.skip("scale_ub is fp8-only")
    torch.manual_seed(0)
    weight = torch.empty(hidden_size, dtype=dtype, device=DEV).normal_(mean=1.0, std=0.1)
    scale = 1 / hidden_size
    x = torch.randn(num_tokens, hidden_size, dtype=dtype, device=DEV) * scale
    residual = torch.randn_like(x) * scale if add_residual else None
    y_ref, res_ref = forward_native(x, residual, weight, EPS)
    scale_ub = y_ref.float().abs().mean().reshape(1) if use_ub else None
    want, want_scales = composed_quant(y_ref, quant_dtype, scale_ub)

    x_before = x.clone()
    res = residual.clone() if add_residual else None
    got, got_scales = ops.rms_norm_dynamic_per_token_quant(x, weight, EPS, quant_dtype, scale_ub, res)
    torch.cuda.synchronize()
    assert got.dtype == quant_dtype and got_scales.shape == (num_tokens, 1)
    assert torch.equal(x, x_before), "the op must not modify its input"
    if add_residual:
        assert torch.equal(res, res_ref)
    assert_codes_and_scales(got, got_scales, want, want_scales, quant_dtype,
                            f"T={num_tokens} H={hidden_size} {dtype} {quant_dtype}")


@pytest.mark.parametrize("T,H", [(1, 64), (7, 1024), (83, 5120), (33, 5137), (256, 8192), (40, 8192), (100, 6144),
                                 (5, 16384), (3, 65536)])
@pytest.mark.parametrize("add_residual", [False, True])
@pytest.mark.parametrize("quant_dtype,use_ub", [(torch.int8, False), (FP8, False), (FP8, True)])
def test_bf16_against_checker(oracle, T, H, add_residual, quant_dtype, use_ub):
    torch.manual_seed(T * 31 + H)
    w = torch.empty(H, dtype=torch.bfloat16, device=DEV).normal_(mean=1.0, std=0.1)
    x = torch.randn(T, H, dtype=torch.bfloat16, device=DEV)
    r = torch.randn(T, H, dtype=torch.bfloat16, device=DEV) if add_residual else None
    ub = 1.5 if use_ub else None
    r_np = to_bits(r) if add_residual else None
    kind = oracle.QUANT_FP8 if quant_dtype == FP8 else oracle.QUANT_INT8
    want, want_scales = oracle.rms_norm_dynamic_per_token_quant([to_bits(x)], to_bits(w), 1e-5, kind,
                                                                scale_ub=ub, r=r_np)
    ub_t = torch.tensor([ub], dtype=torch.float32, device=DEV) if use_ub else None
    got, got_scales = ops.rms_norm_dynamic_per_token_quant(x, w, 1e-5, quant_dtype, ub_t, r)
    torch.cuda.synchronize()
    if add_residual:
        assert np.array_equal(to_bits(r), r_np)
    assert_codes_and_scales(got, got_scales, torch.from_numpy(want).view(quant_dtype),
                            torch.from_numpy(want_scales), quant_dtype, f"T={T} H={H}")


@pytest.mark.parametrize("T", [1, 8, 33, 256, 1000])
@pytest.mark.parametrize("add_residual", [False, True])
@pytest.mark.parametrize("quant_dtype,use_ub", [(torch.int8, False), (FP8, False), (FP8, True)])
def test_partials_against_checker_and_grid_cap_invariance(oracle, T, add_residual, quant_dtype, use_ub):
    cfg = wl.C2.with_tokens(T)
    inp = wl.make_norm_inputs(cfg, DEV)
    parts = [to_bits(p) for p in inp.partials]
    r_np = to_bits(inp.residual) if add_residual else None
    ub = 2.0 if use_ub else None
    kind = oracle.QUANT_FP8 if quant_dtype == FP8 else oracle.QUANT_INT8
    want, want_scales = oracle.rms_norm_dynamic_per_token_quant(parts, to_bits(inp.weight), cfg.eps, kind,
                                                                scale_ub=ub, r=r_np)
    ub_t = torch.tensor([ub], dtype=torch.float32, device=DEV) if use_ub else None
    results = []
    for cap in (None, 7, 64):
        out = torch.empty(T, cfg.H, dtype=quant_dtype, device=DEV)
        scales = torch.empty(T, 1, dtype=torch.float32, device=DEV)
        res = inp.residual.clone() if add_residual else None
        before = [p.clone() for p in inp.partials]
        ops.reduce_add_rms_norm_dynamic_per_token_quant(inp.partials, out, scales, res, inp.weight, cfg.eps,
                                                        scale_ub=ub_t, MAX_CTAS=cap)
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(before, inp.partials)), "partials are read-only"
        if add_residual:
            assert np.array_equal(to_bits(res), r_np)
        results.append((out.view(torch.uint8).cpu(), scales.cpu()))
    for o, s in results[1:]:
        assert torch.equal(o, results[0][0]) and torch.equal(s, results[0][1]), "result depends on the grid cap"
    assert_codes_and_scales(results[0][0].view(quant_dtype), results[0][1],
                            torch.from_numpy(want).view(quant_dtype), torch.from_numpy(want_scales),
                            quant_dtype, f"P=8 T={T}")


@pytest.mark.parametrize("quant_dtype", [torch.int8, FP8])
def test_full_size_against_checker_on_sampled_rows_and_properties(oracle, quant_dtype):
    """8192 x 6144, P = 8.  512 rows spread over the launch (the first and last rows, a
    stride through the middle) are compared with the CPU checker code for code; over all
    rows: every row uses the whole code range, dequantised codes reproduce the
    unquantised op's output to the format's precision, the residual equals the
    unquantised op's."""
    cfg = wl.C4
    inp = wl.make_norm_inputs(cfg, DEV)
    out = torch.empty(cfg.T, cfg.H, dtype=quant_dtype, device=DEV)
    scales = torch.empty(cfg.T, 1, dtype=torch.float32, device=DEV)
    res = inp.residual.clone()
    ops.reduce_add_rms_norm_dynamic_per_token_quant(inp.partials, out, scales, res, inp.weight, cfg.eps)
    torch.cuda.synchronize()
    rows = torch.unique(torch.cat([torch.arange(0, 64), torch.arange(cfg.T - 64, cfg.T),
                                   torch.arange(64, cfg.T - 64, (cfg.T - 128) // 384)[:384]])).to(DEV)
    assert rows.numel() >= 500
    kind = oracle.QUANT_FP8 if quant_dtype == FP8 else oracle.QUANT_INT8
    r_np = to_bits(inp.residual[rows])
    want, want_scales = oracle.rms_norm_dynamic_per_token_quant([to_bits(p[rows]) for p in inp.partials],
                                                                to_bits(inp.weight), cfg.eps, kind, r=r_np)
    assert np.array_equal(to_bits(res[rows]), r_np), "residual differs from the checker on the sampled rows"
    assert_codes_and_scales(out[rows], scales[rows], torch.from_numpy(want).view(quant_dtype),
                            torch.from_numpy(want_scales), quant_dtype, "C4 sampled rows")
    y = torch.empty_like(inp.residual)
    res2 = inp.residual.clone()
    ops.reduce_add_rms_norm(inp.partials, y, res2, inp.weight, cfg.eps)
    torch.cuda.synchronize()
    assert torch.equal(res, res2)
    top = 0x7E if quant_dtype == FP8 else 127
    mag = (out.view(torch.uint8) & 0x7F) if quant_dtype == FP8 else out.to(torch.int16).abs()
    assert bool((mag.amax(dim=-1) == top).all())
    deq = out.float() * scales
    n = y.float()
    step = n.abs() * 2.0 ** -4 + scales * 2.0 ** -10 if quant_dtype == FP8 else 0.5 * scales * (1 + 1e-6)
    # the unquantised op rounds once from the rounded residual, this op twice from the
    # unrounded sum: up to two bf16 steps (2^-7 relative each) apart
    assert bool(((deq - n).abs() <= step + n.abs() * 2.0 ** -6).all())
    assert bool((scales > 0).all()) and bool(torch.isfinite(scales).all())


def test_zero_rows_and_upper_bound():
    H = 2048
    w = torch.ones(H, dtype=torch.bfloat16, device=DEV)
    x = torch.zeros(4, H, dtype=torch.bfloat16, device=DEV)
    x[1, 7] = 3.0
    x[2] = -0.5
    out, scales = ops.rms_norm_dynamic_per_token_quant(x, w, EPS, FP8)
    out8, scales8 = ops.rms_norm_dynamic_per_token_quant(x, w, EPS, torch.int8)
    torch.cuda.synchronize()
    codes = out.view(torch.uint8)
    assert bool((codes[0] == 0).all()) and scales[0].item() == np.float32(1.0 / (448.0 * 512.0))
    assert codes[1, 7].item() == 0x7E and int((codes[1] != 0).sum()) == 1
    assert bool((codes[2] == 0xFE).all()) and bool((out8[2] == -127).all())
    assert scales8[0].item() == np.finfo(np.float32).eps and bool((out8[0] == 0).all())
    ub = torch.tensor([0.25], dtype=torch.float32, device=DEV)
    out, scales = ops.rms_norm_dynamic_per_token_quant(x, w, EPS, FP8, ub)
    torch.cuda.synchronize()
    assert scales[2].item() == np.float32(0.25) / np.float32(448.0)
    assert bool((out.view(torch.uint8)[2] == 0xFE).all())      # |n| ~ 1 > ub: saturates


def test_registered_op_and_errors():
    H = 512
    x = torch.randn(3, H, dtype=torch.bfloat16, device=DEV)
    w = torch.ones(H, dtype=torch.bfloat16, device=DEV)
    out = torch.empty(3, H, dtype=FP8, device=DEV)
    scales = torch.empty(3, 1, dtype=torch.float32, device=DEV)
    torch.ops.tokenweave_amd.rms_norm_dynamic_per_token_quant(out, x, w, scales, EPS, None, None)
    want, want_scales = ops.rms_norm_dynamic_per_token_quant(x, w, EPS, FP8)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.uint8), want.view(torch.uint8)) and torch.equal(scales, want_scales)
    ub = torch.ones(1, dtype=torch.float32, device=DEV)
    with pytest.raises(RuntimeError, match="fp8 output only"):
        ops.rms_norm_dynamic_per_token_quant(x, w, EPS, torch.int8, ub)
    with pytest.raises(RuntimeError, match="result must be"):
        ops.rms_norm_dynamic_per_token_quant(x, w, EPS, torch.int16)
    with pytest.raises(RuntimeError, match="scales must"):
        ops.rms_norm_dynamic_per_token_quant_out(out, x, w, scales.double(), EPS)
    with pytest.raises(NotImplementedError):
        ops.rms_norm_dynamic_per_token_quant(x.double(), w.double(), EPS, FP8)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.rms_norm_dynamic_per_token_quant(x.cpu(), w.cpu(), EPS, FP8)
    # empty input: nothing is launched
    e, es = ops.rms_norm_dynamic_per_token_quant(x[:0], w, EPS, FP8)
    assert e.shape == (0, H) and es.shape == (0, 1)
