"""Host-side mirror of the reference's Python interface for the path: schema
strings, argument validation, row sharding, split arithmetic.  CPU only."""
import pytest
import torch

import tokenweave_amd as tw
from tokenweave_amd import _custom_ops as ops
from tokenweave_amd import workloads as wl


def test_schema_strings_are_the_reference_ones():
    # csrc/torch_bindings.cpp:135-171
    assert ops.SCHEMAS["fused_add_rms_norm"] == (
        "fused_add_rms_norm(Tensor! input, Tensor! residual, Tensor weight, float epsilon) -> ()")
    assert ops.SCHEMAS["rms_norm"] == "rms_norm(Tensor! result, Tensor input, Tensor weight, float epsilon) -> ()"
    assert ops.SCHEMAS["fused_rs_ln_ag_cta"] == (
        "fused_rs_ln_ag_cta(Tensor! input, Tensor! residual, Tensor weight, int mcptr, int signal_pads, "
        "int rank, int world_size, int MAX_CTAS, float epsilon) -> ()")
    for name in ops.SCHEMAS:
        op = getattr(torch.ops.tokenweave_amd, name)
        schema = op.default._schema
        assert schema.name == f"tokenweave_amd::{name}"
        assert len(schema.returns) == 0
        assert schema.arguments[0].alias_info is not None and schema.arguments[0].alias_info.is_write


def test_ops_refuse_cpu_tensors_loudly():
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    w = torch.ones(64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        ops.fused_add_rms_norm(x, x.clone(), w, 1e-5)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        torch.ops.tokenweave_amd.rms_norm(x.clone(), x, w, 1e-5)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.reduce_add_rms_norm([x], x.clone(), x.clone(), w, 1e-5)
    with pytest.raises(RuntimeError, match="GPU only"):
        tw.RMSNorm(64, dtype=torch.bfloat16)(x, x.clone())


def test_dtype_errors_use_dispatch_wording():
    x = torch.zeros(4, 64, dtype=torch.float64)
    with pytest.raises(NotImplementedError, match="not implemented for"):
        ops.fused_add_rms_norm(x, x.clone(), torch.ones(64, dtype=torch.float64), 1e-5)
    h = torch.zeros(4, 64, dtype=torch.float16)
    with pytest.raises(NotImplementedError, match="fused_add_rms_norm_cta_kernel"):
        ops.fused_add_rms_norm_cta(h, h.clone(), torch.ones(64, dtype=torch.float16), 8, 1e-5)


def test_shard_bounds():
    assert tw.shard_bounds(2048, 3, 8) == (768, 1024)
    with pytest.raises(AssertionError, match="Mismatch in token count"):
        tw.shard_bounds(3001, 0, 8)
    with pytest.raises(AssertionError, match="Invalid rank"):
        tw.shard_bounds(2048, 8, 8)
    floor = [tw.shard_bounds(3001, r, 8, "floor") for r in range(8)]
    ceil = [tw.shard_bounds(3001, r, 8, "ceil") for r in range(8)]
    for parts in (floor, ceil):
        assert parts[0][0] == 0 and parts[-1][1] == 3001
        assert all(parts[i][1] == parts[i + 1][0] for i in range(7))
    assert floor[-1][1] - floor[-1][0] == 376 and ceil[-1][1] - ceil[-1][0] == 369
    assert tw.shard_bounds(5, 7, 8, "ceil") == (5, 5)


def test_split_size_formula():
    # ((N + 255) & ~255) // 2 + split_offset, vllm/model_executor/models/llama.py:521
    assert tw.tokenweave_split_size(4096) == 2048
    assert tw.tokenweave_split_size(4097) == 2176
    assert tw.tokenweave_split_size(1024, 256) == 768
    assert tw.tokenweave_split_size(1) == 128


class _Recorder(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.calls = []

    def forward(self, x, residual, **kw):
        self.calls.append((x, residual, kw))


def test_fused_allreduce_layernorm_slices_and_offsets_like_the_reference():
    # tokenweave_utils.py:59-91
    H, T, ws = 64, 32, 8
    hs = torch.zeros(T, H, dtype=torch.bfloat16)
    res = torch.zeros(T, H, dtype=torch.bfloat16)
    rec = _Recorder()
    tw.fused_allreduce_layernorm(rec, hs, res, "hdl", T // ws, 3, ws, 16, offset_symm_mem=4096)
    x, r, kw = rec.calls[0]
    assert x.data_ptr() == hs[12:16].data_ptr() and x.shape == (4, H)
    assert r.data_ptr() == res[12:16].data_ptr()
    assert kw == dict(MAX_CTAS=4, fused_ar=True, symm_mem_hdl="hdl", rank=3, world_size=ws,
                      offset=4096 + 12 * H * 2)
    with pytest.raises(AssertionError, match="same shape"):
        tw.fused_allreduce_layernorm(rec, hs, res[:8], "hdl", 4, 0, ws, 16)
    with pytest.raises(AssertionError, match="Mismatch in token count: expected 40, got 32"):
        tw.fused_allreduce_layernorm(rec, hs, res, "hdl", 5, 0, ws, 16)
    with pytest.raises(AssertionError, match="Invalid rank 8"):
        tw.fused_allreduce_layernorm(rec, hs, res, "hdl", 4, 8, ws, 16)
    # ragged extension
    tw.fused_allreduce_layernorm(rec, hs, res, "hdl", 0, 7, ws, 16, row_range=(28, 32))
    assert rec.calls[-1][2]["offset"] == 28 * H * 2 and rec.calls[-1][0].shape == (4, H)


def test_rmsnorm_module_surface_and_native_path():
    layer = tw.RMSNorm(64, eps=1e-5)
    assert layer.weight.shape == (64,) and layer.variance_epsilon == 1e-5
    x = torch.randn(3, 64)
    r = torch.randn(3, 64)
    y, r2 = layer.forward_native(x, r)
    s = x + r
    torch.testing.assert_close(r2, s)
    torch.testing.assert_close(y, s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + 1e-5))
    with pytest.raises(ValueError, match="Expected hidden_size to be 64"):
        layer.forward_native(torch.randn(3, 32))
    import inspect
    params = list(inspect.signature(layer.forward).parameters)
    assert params == ["x", "residual", "out", "MAX_CTAS", "fused_ar", "fused_rs", "symm_mem_hdl",
                      "rank", "world_size", "offset"]


def test_partials_region_lookup():
    class Owner:
        pass
    o, o2 = Owner(), Owner()
    ops.register_partials_region(0x10000, 0x1000, 8, o, usable_bytes=0xC00)
    ops.register_partials_region(0x40000, 0x2000, 4, o2)
    assert ops._peer_stride(0x10000 + 0x800, 8, 0x400) == 0x1000
    assert ops._peer_stride(0x40000, 4, 0x2000) == 0x2000          # the other region, then back
    assert ops._peer_stride(0x10000, 8, 0xC00) == 0x1000
    with pytest.raises(RuntimeError, match="not inside slot 0"):
        ops._peer_stride(0x10000 + 0x1000, 8, 16)
    with pytest.raises(RuntimeError, match="exceeds the 8 slots"):
        ops._peer_stride(0x10000, 9, 16)
    # the rows a call reads must stay inside the usable part of a slot (a too large
    # hidden_states or offset would read past the staging buffer of the last rank)
    with pytest.raises(RuntimeError, match="reach past the 3072 usable bytes"):
        ops._peer_stride(0x10000 + 0x800, 8, 0x401)
    with pytest.raises(RuntimeError, match="reach past"):
        ops._peer_stride(0x40000 + 0x1000, 4, 0x1010)
    assert ops._peer_stride(0xdead0, 1, 1 << 40) == 16
    del o
    with pytest.raises(RuntimeError, match="not inside slot 0"):
        ops._peer_stride(0x10000, 8, 16)
    assert ops._peer_stride(0x40000, 4, 16) == 0x2000


def test_algorithmic_bytes_table():
    assert wl.algorithmic_bytes(1, 512, 8192) == 33570816
    assert wl.algorithmic_bytes(8, 256, 8192) == 46153728
    assert wl.algorithmic_bytes(8, 1, 8192) == 196608
    assert wl.algorithmic_bytes(8, 3001, 8192) == 540868608
    assert wl.algorithmic_bytes(8, 8192, 6144) == 1107308544
    assert wl.algorithmic_bytes(8, 1638, 8192) == 295223296
    cfgs = wl.norm_configs()
    assert cfgs["c2_llama70b_tp8_shard@T256"].bytes == 46153728
    assert {"c1_add_rmsnorm", "c3_qwen72b_ragged", "c4_mixtral_8x22b_chunk", "c5_weave_norm_split"} <= set(cfgs)


def test_workload_generation_is_seeded_and_shaped():
    cfg = wl.C3.with_tokens(5)
    a, b = wl.make_norm_inputs(cfg, "cpu"), wl.make_norm_inputs(cfg, "cpu")
    assert torch.equal(a.staging, b.staging) and torch.equal(a.weight, b.weight)
    assert a.staging.shape == (8, 5, 8192) and a.residual.dtype == torch.bfloat16
    assert 0.5 <= a.weight.float().min() and a.weight.float().max() <= 1.5
    c = wl.make_norm_inputs(cfg, "cpu", seed_offset=1)
    assert not torch.equal(a.staging, c.staging)
    g = wl.make_gemm_inputs(16, 32, 64, "cpu")
    assert g.a.shape == (16, 64) and g.b.shape == (32, 64) and abs(g.b.float().std() - 0.02) < 0.005


def test_weave_config_table_and_plan():
    cfg = tw.load_config()          # packaged llama_config_8.json, same layout as the reference's tables
    assert cfg is tw.load_config()  # cached per path (tokenweave_utils.py:10)
    assert all(isinstance(k, int) for k in cfg) and 1024 in cfg
    for entry in cfg.values():
        assert {"attention_ctas", "mlp_ctas", "split_offset", "gemm_cus"} <= set(entry)
    assert tw.select_config(cfg, 1500) is cfg[1024]      # closest length, llama.py:516
    assert tw.select_config(cfg, 1537) is cfg[2048]
    assert tw.weave_plan(1023, cfg) is None              # below the weave threshold: fuse only
    plan = tw.weave_plan(4096, cfg)
    off = cfg[4096]["split_offset"]
    assert plan["split_size"] == 2048 + off and plan["rest_size"] == 4096 - plan["split_size"]
    assert plan["gemm_cus"] == cfg[4096]["gemm_cus"]
    table = {1024: {"attention_ctas": 8, "mlp_ctas": 4, "split_offset": 256}}
    assert tw.weave_plan(1100, table) == {"split_size": 896, "rest_size": 204, "attention_ctas": 8,
                                          "mlp_ctas": 4, "gemm_cus": 0}


@pytest.mark.parametrize("name", ["llama_config_4", "llama_config_8", "mixtral_config_8", "qwen2_config_4",
                                  "qwen2_config_8"])
def test_every_reference_model_has_a_tuned_table(name):
    """The reference ships five tables (vllm/tokenweave_configs/*.json); each has a
    counterpart measured on MI355X with the same token counts, the reference's three
    keys, the GEMM budgets and the measured overlap flag, and plans from it."""
    cfg = tw.load_config(f"tokenweave_configs/{name}.json")
    assert sorted(cfg) == [1024, 2048, 4096, 8192, 16384, 32768, 65536]
    cus = 256
    for n, e in cfg.items():
        assert {"attention_ctas", "mlp_ctas", "split_offset", "gemm_cus", "mlp_gemm_cus", "overlap"} <= set(e)
        assert e["overlap"] in (0, 1) and e["split_offset"] in (0, 64, 128, 192, 256)
        assert all(0 <= e[k] <= cus for k in ("attention_ctas", "mlp_ctas", "gemm_cus", "mlp_gemm_cus"))
        plan = tw.weave_plan(n, cfg)
        if e["overlap"]:
            assert plan["split_size"] == n // 2 + e["split_offset"] and plan["rest_size"] == n - plan["split_size"]
            assert plan["gemm_cus"] == e["gemm_cus"] and plan["mlp_gemm_cus"] == e["mlp_gemm_cus"]
        else:
            assert plan is None
    assert cfg[65536]["overlap"] == 1, "long prefill chunks overlap on MI355X"


def test_bind_checks_arguments_at_bind_time():
    import tokenweave_amd._custom_ops as ops
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    w = torch.ones(64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.bind_reduce_add_rms_norm([x], x, x.clone(), w, 1e-5)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.bind_gemm_bf16_nt(torch.zeros(4, 4, dtype=torch.bfloat16), x, x)


def test_fuse_only_schedule_calls_in_reference_order():
    """tokenweave_with_fuse_only (reference tokenweave_utils.py:95-172): layer-0 norm with
    out=residual, attention on the actual tokens, post-attention fused norm, MLP, fused
    norm of the next layer — with the shard arithmetic of fused_allreduce_layernorm."""
    log = []

    class Norm:
        def __init__(self, name):
            self.name = name

        def __call__(self, x, residual=None, out=None, **kw):
            log.append((self.name, tuple(x.shape), "out" if out is not None else "res", kw.get("offset"),
                        kw.get("MAX_CTAS"), kw.get("fused_ar", False)))

    class Layer:
        input_layernorm = Norm("input")
        post_attention_layernorm = Norm("post")

        def self_attn(self, positions, hidden_states):
            log.append(("attn", tuple(hidden_states.shape)))

    hs = torch.zeros(16, 8, dtype=torch.bfloat16)
    res = torch.zeros_like(hs)
    tw.tokenweave_with_fuse_only(Layer(), torch.arange(13), hs, res, object(), 0, rank=2, world_size=4,
                                 next_layer_norm=Norm("next"), actual_tokens=13,
                                 nearest_multiple_of_world_size=16, MAX_CTAS_ATTN=3, MAX_CTAS_MLP=32,
                                 mlp_fn=lambda x: log.append(("mlp", tuple(x.shape))))
    row_bytes = 8 * 2
    assert log == [
        ("input", (16, 8), "out", None, None, False),
        ("attn", (13, 8)),
        ("post", (4, 8), "res", 2 * 4 * row_bytes, 3, True),
        ("mlp", (13, 8)),
        ("next", (4, 8), "res", 2 * 4 * row_bytes, 4, True),   # MAX_CTAS is capped by the shard's rows
    ]
    with pytest.raises(AssertionError, match="mlp_fn"):
        tw.tokenweave_with_fuse_only(Layer(), None, hs, res, object(), 1, nearest_multiple_of_world_size=16)


def test_weave_plan_honours_measured_no_overlap_entries():
    table = {1024: {"attention_ctas": 0, "mlp_ctas": 0, "split_offset": 256, "gemm_cus": 128, "overlap": 0},
             8192: {"attention_ctas": 0, "mlp_ctas": 0, "split_offset": 256, "gemm_cus": 128, "overlap": 1}}
    assert tw.weave_plan(1500, table) is None
    assert tw.weave_plan(8000, table)["gemm_cus"] == 128
    shipped = tw.load_config()
    assert all("overlap" in e for e in shipped.values())
    assert tw.weave_plan(16384, shipped) is not None


def test_row_parallel_linear_constructor_contract():
    """Constructor checks of RowParallelLinear (vllm/model_executor/layers/linear.py:1185-1240):
    shapes per rank, the reduce_results / bias guard, rank bounds."""
    import tokenweave_amd as tw
    lin = tw.RowParallelLinear(8192, 8192, bias=True, tp_rank=3, tp_size=8)
    assert tuple(lin.weight.shape) == (8192, 1024) and tuple(lin.bias.shape) == (8192,)
    assert lin.weight.dtype == torch.bfloat16 and lin.input_size_per_partition == 1024
    assert "tp_size=8" in lin.extra_repr() and "input_features=1024" in lin.extra_repr()
    assert tw.RowParallelLinear(64, 64, bias=False).bias is None
    with pytest.raises(ValueError, match="When not reduce the results"):
        tw.RowParallelLinear(64, 64, bias=True, reduce_results=False)
    with pytest.raises(ValueError, match="Invalid rank"):
        tw.RowParallelLinear(64, 64, tp_rank=2, tp_size=2)
    with pytest.raises(ValueError, match="not divisible"):
        tw.RowParallelLinear(100, 64, tp_size=8)
    full = torch.arange(64 * 64, dtype=torch.float32).view(64, 64).to(torch.bfloat16)
    lin = tw.RowParallelLinear(64, 64, bias=False, tp_rank=1, tp_size=4)
    lin.weight_loader(lin.weight, full)
    assert torch.equal(lin.weight.data, full[:, 16:32])
