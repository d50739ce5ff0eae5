"""Norm + static-scale fp8 (e4m3fn) output on a real GPU.

The reference has no CPU twin of these ops; its own unit test
(tests/kernels/test_layernorm.py:67-139) checks the fused op against the
composition `static_scaled_fp8_quant(norm(x))` at atol = rtol = 1e-3.  The same
composition is the definition here, so beyond that tolerance the fused output must
be bit-identical to quantising the unfused op's output, and the checker's
conversion (pinned against torch's cast on every bf16 pattern) must agree."""
import numpy as np
import pytest
import torch

from helpers import to_bits
from tokenweave_amd import _custom_ops as ops
from tokenweave_amd import workloads as wl

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
FP8 = torch.float8_e4m3fn


def torch_quant(y: torch.Tensor, scale: float) -> torch.Tensor:
    inv = torch.tensor(1.0, dtype=torch.float32, device=y.device) / torch.tensor(scale, dtype=torch.float32, device=y.device)
    return (y.float() * inv).clamp(-448.0, 448.0).to(FP8)


@pytest.mark.parametrize("quant_scale", [1.0, 0.01, 10.0])
@pytest.mark.parametrize("dtype", [torch.half, torch.bfloat16, torch.float])
@pytest.mark.parametrize("add_residual", [False, True])
@pytest.mark.parametrize("hidden_size", [8, 768, 769, 771, 5120, 5125, 8192, 8199])
@pytest.mark.parametrize("num_tokens", [7, 83, 4096])
def test_reference_quant_grid(num_tokens, hidden_size, add_residual, dtype, quant_scale):
    torch.manual_seed(0)
    weight = torch.empty(hidden_size, dtype=dtype, device=DEV).normal_(mean=1.0, std=0.1)
    s = 1 / (2 * hidden_size)
    x = torch.randn(num_tokens, hidden_size, dtype=dtype, device=DEV) * s
    scale_t = torch.tensor(quant_scale, dtype=torch.float32, device=DEV)
    fused = torch.empty(num_tokens, hidden_size, dtype=FP8, device=DEV)
    x_before = x.clone()
    if add_residual:
        residual = torch.randn_like(x) * s
        res_fused = residual.clone()
        torch.ops.tokenweave_amd.fused_add_rms_norm_static_fp8_quant(fused, x, res_fused, weight, scale_t, 1e-6)
        x_unfused = x.clone()
        ops.fused_add_rms_norm(x_unfused, residual, weight, 1e-6)
        y = x_unfused
        torch.cuda.synchronize()
        assert torch.equal(res_fused, residual)
    else:
        torch.ops.tokenweave_amd.rms_norm_static_fp8_quant(fused, x, weight, scale_t, 1e-6)
        y = torch.empty_like(x)
        ops.rms_norm(y, x, weight, 1e-6)
        torch.cuda.synchronize()
    assert torch.equal(x, x_before), "the quantising ops must not modify their input"
    want = torch_quant(y, quant_scale)
    torch.testing.assert_close(fused.float(), want.float(), atol=1e-3, rtol=1e-3)
    assert torch.equal(fused.view(torch.uint8), want.view(torch.uint8))


@pytest.mark.parametrize("T", [1, 33, 100, 256, 1000])
@pytest.mark.parametrize("scale", [0.02, 1.0])
def test_reduce_fp8_against_checker(oracle, T, scale):
    cfg = wl.C2.with_tokens(T)
    inp = wl.make_norm_inputs(cfg, DEV)
    parts = [to_bits(p) for p in inp.partials]
    y_want, r_want = oracle.reduce_add_rms_norm(parts, to_bits(inp.residual), to_bits(inp.weight), cfg.eps)
    q_want = oracle.static_fp8_quant(y_want, scale)
    out = torch.empty(T, cfg.H, dtype=FP8, device=DEV)
    res = inp.residual.clone()
    scale_t = torch.tensor(scale, dtype=torch.float32, device=DEV)
    ops.reduce_add_rms_norm_static_fp8_quant(inp.partials, out, res, inp.weight, scale_t, cfg.eps)
    torch.cuda.synchronize()
    assert np.array_equal(to_bits(res), r_want)
    got = out.view(torch.uint8).cpu().numpy()
    # y may differ from the checker by one bf16 ulp on a few elements (summation order of
    # the mean of squares); a bf16 ulp is at most one fp8 step
    diff = got.astype(np.int16) - q_want.astype(np.int16)
    assert np.abs(diff).max() <= 1 and (diff != 0).mean() < 2e-3
    # and bit-identical to quantising this implementation's own bf16 output
    y_hip = torch.empty_like(inp.residual)
    ops.reduce_add_rms_norm(inp.partials, y_hip, inp.residual.clone(), inp.weight, cfg.eps)
    torch.cuda.synchronize()
    assert np.array_equal(got, oracle.static_fp8_quant(to_bits(y_hip), scale))


def test_saturation_and_argument_errors():
    H = 64
    x = torch.full((4, H), 100.0, dtype=torch.bfloat16, device=DEV)
    x[1] = -100.0
    w = torch.full((H,), 2.0, dtype=torch.bfloat16, device=DEV)
    out = torch.empty(4, H, dtype=FP8, device=DEV)
    scale_t = torch.tensor(1e-3, dtype=torch.float32, device=DEV)   # y = +-2 -> +-2000 -> saturates
    ops.rms_norm_static_fp8_quant(out, x, w, scale_t, 1e-6)
    torch.cuda.synchronize()
    got = out.view(torch.uint8).cpu()
    assert (got[0] == 0x7E).all() and (got[1] == 0xFE).all()
    with pytest.raises(NotImplementedError, match="fp8_type"):
        ops.rms_norm_static_fp8_quant(torch.empty(4, H, dtype=torch.uint8, device=DEV), x, w, scale_t, 1e-6)
    with pytest.raises(RuntimeError, match="one float32"):
        ops.rms_norm_static_fp8_quant(out, x, w, torch.ones(2, device=DEV), 1e-6)
    with pytest.raises(RuntimeError, match="16-byte aligned"):
        ops.reduce_add_rms_norm_static_fp8_quant([x[:, :8].contiguous()], torch.empty(4, 8, dtype=FP8, device=DEV),
                                                 x[:, :8].contiguous(), w[:8].contiguous(), scale_t, 1e-6)
