"""The two layer-level schedules of the reference's tokenweave_utils.py
(`tokenweave_with_fuse_only` :95-172, `tokenweave_overlap` :175-340) on a toy
decoder stack: one GPU plays all the ranks (`all_ranks=True`), attention and MLP are
stand-ins that leave P different partial sums in the P staging slots.  Rows are
independent, so the split, two-stream schedule must reproduce the unsplit one bit for
bit; both are checked against plain fp32 torch arithmetic."""
import pytest
import torch

import tokenweave_amd as tw
from helpers import ATOL, RTOL

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
H, WS, RANK, LAYERS, EPS = 512, 4, 1, 3, 1e-5


class ToyLayer:
    """`self_attn` / `mlp` read this rank's staging rows (the normalised input) and
    write partial p = bf16(x * a[p] + b[p]) into slot p: what P ranks' row-parallel
    projections would leave behind."""

    def __init__(self, buf, seed):
        g = torch.Generator(device=DEV).manual_seed(seed)
        self.buf = buf
        self.input_layernorm = tw.RMSNorm(H, eps=EPS, dtype=torch.bfloat16).to(DEV)
        self.post_attention_layernorm = tw.RMSNorm(H, eps=EPS, dtype=torch.bfloat16).to(DEV)
        for ln in (self.input_layernorm, self.post_attention_layernorm):
            ln.weight.data.copy_(1 + 0.1 * torch.randn(H, generator=g, device=DEV))
        self.coef = {k: (torch.randn(WS, generator=g, device=DEV) * 0.5,
                         torch.randn(WS, H, generator=g, device=DEV) * 0.1) for k in ("attn", "mlp")}
        self.calls = []
        self.budgets = []   # the compute-unit budget each projection was given

    def _project(self, kind, hidden_states):
        row_bytes = H * 2
        first = (hidden_states.data_ptr() - self.buf.local.data_ptr()) // row_bytes
        n = hidden_states.shape[0]
        x = hidden_states.float()
        a, b = self.coef[kind]
        for p in range(WS):
            self.buf.slot(p)[first:first + n].copy_((x * a[p] + b[p]).to(torch.bfloat16))
        self.calls.append((kind, int(first), int(n)))

    def self_attn(self, positions, hidden_states, gemm_cus=None, **kwargs):
        assert positions.shape[0] == hidden_states.shape[0]
        self._project("attn", hidden_states)
        self.budgets.append(gemm_cus)
        return hidden_states

    def mlp(self, hidden_states, gemm_cus=None):
        self._project("mlp", hidden_states)
        self.budgets.append(gemm_cus)
        return hidden_states


def torch_stack(emb, layers, final_norm):
    """fp32 statement of the same stack (single rounding points as in the ops)."""
    def norm(s, w):
        r = s.to(torch.bfloat16)
        inv = torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + EPS)
        return (r.float() * inv * w.float()).to(torch.bfloat16), r
    x, res = norm(emb.float(), layers[0].input_layernorm.weight)
    for i, layer in enumerate(layers):
        nxt = layers[i + 1].input_layernorm if i + 1 < len(layers) else final_norm
        for kind, ln in (("attn", layer.post_attention_layernorm), ("mlp", nxt)):
            a, b = layer.coef[kind]
            s = res.float()
            part = [(x.float() * a[p] + b[p]).to(torch.bfloat16).float() for p in range(WS)]
            acc = part[0]
            for p in range(1, WS):
                acc = acc + part[p]
            x, res = norm(acc + s, ln.weight)
    return x, res


def run_stack(T, schedule, gemm_cus=0, mlp_gemm_cus=None):
    torch.manual_seed(7)
    buf = tw.PartialsBuffer(WS, T, H, rank=RANK, device=DEV)
    layers = [ToyLayer(buf, 100 + i) for i in range(LAYERS)]
    final_norm = tw.RMSNorm(H, eps=EPS, dtype=torch.bfloat16).to(DEV)
    emb = torch.randn(T, H, device=DEV).to(torch.bfloat16)
    buf.storage.zero_()
    hidden_states = buf.hidden_states(T)
    hidden_states.copy_(emb)             # the other ranks' slots hold zeros: the sum is emb
    residual = torch.empty_like(hidden_states)
    positions = torch.arange(T, device=DEV)
    cur, side = torch.cuda.current_stream(), torch.cuda.Stream()
    split = tw.tokenweave_split_size(T)
    for i, layer in enumerate(layers):
        nxt = layers[i + 1].input_layernorm if i + 1 < LAYERS else final_norm
        if schedule == "fuse_only":
            tw.tokenweave_with_fuse_only(
                layer, positions, hidden_states, residual, buf, i, rank=RANK, world_size=WS,
                next_layer_norm=nxt, actual_tokens=T, nearest_multiple_of_world_size=T,
                MAX_CTAS_ATTN=16, MAX_CTAS_MLP=16, mlp_fn=layer.mlp, all_ranks=True)
        else:
            tw.tokenweave_overlap(
                layer, positions, hidden_states, residual, buf, i, end_layer=LAYERS, rank=RANK,
                world_size=WS, current_stream=cur, copy_stream=side, next_layer_norm=nxt,
                split_size=split, actual_tokens=T, num_tokens_padded=T, MAX_CTAS_ATTN=16,
                MAX_CTAS_MLP=16, mlp_fn=layer.mlp, all_ranks=True, gemm_cus=gemm_cus,
                mlp_gemm_cus=mlp_gemm_cus)
    torch.cuda.synchronize()
    return hidden_states.clone(), residual.clone(), emb, layers, final_norm, split


@pytest.mark.parametrize("T", [640, 1000])
def test_overlap_schedule_equals_fuse_only_schedule(T):
    y0, r0, emb, layers, final_norm, _ = run_stack(T, "fuse_only")
    y1, r1, _, layers1, _, split = run_stack(T, "overlap")
    assert torch.equal(y0, y1) and torch.equal(r0, r1)
    # the overlap schedule really worked on the two splits
    assert ("attn", 0, split) in layers1[1].calls and ("attn", split, T - split) in layers1[1].calls
    y_ref, r_ref = torch_stack(emb, layers, final_norm)
    torch.testing.assert_close(r0.float(), r_ref.float(), rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(y0.float(), y_ref.float(), rtol=RTOL, atol=ATOL)


def test_overlap_schedule_hands_the_gemm_budget_of_the_plan_to_the_projections():
    """weave_plan's gemm_cus reaches every projection that runs beside a norm; without a
    budget the layer's callables are called with the reference's keywords only."""
    plan = tw.weave_plan(16384, tw.load_config("tokenweave_configs/llama_config_8.json"))
    assert plan is not None and plan["gemm_cus"] > 0 and plan["mlp_gemm_cus"] > 0
    y0, r0, _, layers, _, _ = run_stack(1000, "overlap", gemm_cus=plan["gemm_cus"],
                                        mlp_gemm_cus=plan["mlp_gemm_cus"])
    for layer in layers:   # attention of both splits, then the MLP of both splits
        assert layer.budgets == [plan["gemm_cus"]] * 2 + [plan["mlp_gemm_cus"]] * 2
    y1, r1, _, layers, _, _ = run_stack(1000, "overlap")
    assert all(layer.budgets == [None] * 4 for layer in layers)
    assert torch.equal(y0, y1) and torch.equal(r0, r1)


def test_fuse_only_touches_only_this_ranks_shard_without_all_ranks():
    T = 64
    buf = tw.PartialsBuffer(WS, T, H, rank=RANK, device=DEV)
    layer = ToyLayer(buf, 5)
    nxt = tw.RMSNorm(H, eps=EPS, dtype=torch.bfloat16).to(DEV)
    buf.storage.zero_()
    hidden_states = buf.hidden_states(T)
    hidden_states.copy_(torch.randn(T, H, device=DEV))
    residual = torch.zeros_like(hidden_states)
    positions = torch.arange(T, device=DEV)
    # the attention stand-in marks residual so that the rows the norms rewrite can be told apart
    orig = layer.self_attn
    layer.self_attn = lambda positions, hidden_states, **kw: (orig(positions, hidden_states), residual.fill_(7.0))[0]
    tw.tokenweave_with_fuse_only(layer, positions, hidden_states, residual, buf, 1, rank=RANK, world_size=WS,
                                 next_layer_norm=nxt, actual_tokens=T, nearest_multiple_of_world_size=T,
                                 mlp_fn=layer.mlp)
    torch.cuda.synchronize()
    per = T // WS
    mine = slice(RANK * per, (RANK + 1) * per)
    changed = (residual != 7.0).any(dim=-1)
    assert bool(changed[mine].all()) and int(changed.sum()) == per
