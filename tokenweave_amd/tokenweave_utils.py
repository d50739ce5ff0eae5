"""Host-side orchestration of the fused op: row sharding, the staging buffers
that stand in for symmetric memory on one GPU, and the two-stream weave step.

Mirror of ``vllm/model_executor/models/tokenweave_utils.py``:
``fused_allreduce_layernorm`` (:24-92) keeps its argument list, assertions and
slice/offset arithmetic; ``tokenweave_with_fuse_only`` (:95-172) and
``tokenweave_overlap`` (:175-340) keep theirs and the order of their stream
hand-offs; ``weave_norm_gemm`` is one stage of the overlap — the norm of one
token split on a second stream while the other split's row-parallel GEMM runs
on the current stream.
"""
from __future__ import annotations

import json
import os
from functools import lru_cache
from typing import Any, Callable, Dict, Optional, Tuple

import torch

from . import _custom_ops as ops
from .layernorm import RMSNorm


@lru_cache(maxsize=None)
def load_config(config_path: str = "tokenweave_configs/llama_config_8.json") -> Dict[int, Dict[str, int]]:
    """Per-model weave table: token count -> {"attention_ctas", "mlp_ctas", "split_offset",
    "gemm_cus", "mlp_gemm_cus", "overlap"}.  Same file layout and loader contract as the reference
    (tokenweave_utils.py:10-21, vllm/tokenweave_configs/*.json): JSON object with
    string token-count keys, returned with integer keys and cached per path.
    `*_ctas` is the MAX_CTAS given to the fused norm of the attention / MLP stage (0 =
    one workgroup per row), `gemm_cus` / `mlp_gemm_cus` the compute-unit budget of the GEMM it overlaps
    with — the knob that matters on MI355X, where a GEMM workgroup and a norm workgroup
    cannot share a compute unit.  Relative paths resolve against this package."""
    base_dir = os.path.dirname(os.path.abspath(__file__))
    full_path = config_path if os.path.isabs(config_path) else os.path.normpath(
        os.path.join(base_dir, config_path))
    with open(full_path, "r") as f:
        data = json.load(f)
    return {int(k): v for k, v in data.items()}


def select_config(config: Dict[int, Dict[str, int]], num_tokens: int) -> Dict[str, int]:
    """The entry whose token count is closest to num_tokens
    (vllm/model_executor/models/llama.py:516-517); ties go to the smaller count."""
    closest = min(sorted(config), key=lambda k: abs(k - num_tokens))
    return config[closest]


def weave_plan(num_tokens: int, config: Dict[int, Dict[str, int]],
               threshold: int = 1024) -> Optional[Dict[str, int]]:
    """What the model forward decides per batch (llama.py:509-521): below `threshold`
    tokens no weave (fuse only) -> None; otherwise the split point and the budgets of
    the closest table entry.  An entry may carry `"overlap": 0` — measured on the
    target GPU, the two-stream stage was no faster than running its kernels on one
    stream at that size — which also means fuse only."""
    if num_tokens < threshold:
        return None
    entry = select_config(config, num_tokens)
    if not entry.get("overlap", 1):
        return None
    split = min(tokenweave_split_size(num_tokens, entry.get("split_offset", 0)), num_tokens)
    gemm_cus = entry.get("gemm_cus", 0)
    plan = {"split_size": split, "rest_size": num_tokens - split,
            "attention_ctas": entry.get("attention_ctas", 0), "mlp_ctas": entry.get("mlp_ctas", 0),
            "gemm_cus": gemm_cus}
    if "mlp_gemm_cus" in entry:
        plan["mlp_gemm_cus"] = entry["mlp_gemm_cus"]
    return plan


class PartialsBuffer:
    """The P ranks' staging buffers as P equally spaced slots of one allocation.

    In the reference every rank owns one symmetric-memory staging buffer and
    ``symm_mem_hdl.multicast_ptr`` names all of them at once
    (vllm/model_executor/models/llama.py:437-441).  Here slot p holds what rank
    p's buffer would hold — its partial sum — and the object exposes the two
    attributes the layer reads from the handle (layernorm.py:79-80):
    ``multicast_ptr`` (address of slot 0) and ``signal_pad_ptrs_dev`` (0: there
    are no peers to signal).  Rows are [max_tokens, hidden_size] bf16.
    """

    def __init__(self, world_size: int, max_tokens: int, hidden_size: int, rank: int = 0,
                 device: Any = "cuda", dtype: torch.dtype = torch.bfloat16,
                 slot_pad_bytes: int = 0) -> None:
        assert 0 <= rank < world_size, f"Invalid rank {rank}, must be in [0, {world_size - 1}]"
        if dtype != torch.bfloat16:
            raise NotImplementedError("staging buffers are bf16, like the reference's")
        if hidden_size % 8 != 0:
            raise RuntimeError(ops.ALIGNMENT_MESSAGE)
        if slot_pad_bytes < 0 or slot_pad_bytes % 16 != 0:
            raise ValueError("slot_pad_bytes must be a non-negative multiple of 16")
        self.world_size = world_size
        self.rank = rank
        self.max_tokens = max_tokens
        self.hidden_size = hidden_size
        # slot_pad_bytes spaces the slots apart, for callers that want the P streams of
        # one row to fall on different memory channels
        slot_elems = max_tokens * hidden_size + slot_pad_bytes // 2
        self._backing = torch.empty(world_size * slot_elems, dtype=dtype, device=device)
        self.storage = self._backing.as_strided((world_size, max_tokens, hidden_size),
                                                (slot_elems, hidden_size, 1))
        self.peer_stride_bytes = slot_elems * 2
        self.multicast_ptr = self._backing.data_ptr()
        self.signal_pad_ptrs_dev = 0
        ops.register_partials_region(self.multicast_ptr, self.peer_stride_bytes, world_size,
                                     self._backing, usable_bytes=max_tokens * hidden_size * 2)

    def slot(self, p: int) -> torch.Tensor:
        """Rank p's staging buffer, [max_tokens, hidden_size]."""
        return self.storage[p]

    @property
    def local(self) -> torch.Tensor:
        """This rank's staging buffer: where its GEMM writes and where y lands."""
        return self.storage[self.rank]

    def hidden_states(self, num_tokens: int, first_row: int = 0) -> torch.Tensor:
        return self.local[first_row:first_row + num_tokens]

    def offset_of_row(self, row: int) -> int:
        """Byte offset of a row inside every slot (`offset_symm_mem` of the reference)."""
        return row * self.hidden_size * self.storage.element_size()


def shard_bounds(total_tokens: int, rank: int, world_size: int,
                 mode: str = "even") -> Tuple[int, int]:
    """Rows [start, end) that `rank` owns.

    "even"  — the reference's contract: total_tokens == per_rank * world_size
              (tokenweave_utils.py:63-77);
    "floor" — per_rank = total // world_size, the last rank takes the remainder;
    "ceil"  — per_rank = ceil(total / world_size), the last ranks take what is left.
    """
    assert 0 <= rank < world_size, f"Invalid rank {rank}, must be in [0, {world_size - 1}]"
    if mode == "even":
        per = total_tokens // world_size
        assert per * world_size == total_tokens, (
            f"Mismatch in token count: expected {per * world_size}, got {total_tokens}")
        return rank * per, (rank + 1) * per
    if mode == "floor":
        per = total_tokens // world_size
        start = rank * per
        return start, (total_tokens if rank == world_size - 1 else start + per)
    if mode == "ceil":
        per = -(-total_tokens // world_size)
        start = min(rank * per, total_tokens)
        return start, min(start + per, total_tokens)
    raise ValueError(f"unknown shard mode {mode!r}")


def fused_allreduce_layernorm(
    layernorm: RMSNorm,
    hidden_states: torch.Tensor,
    residual: torch.Tensor,
    symm_mem_hdl: Any,
    num_tokens_per_rank: int,
    rank: int,
    world_size: int,
    MAX_CTAS: int,
    offset_symm_mem: int = 0,
    row_range: Optional[Tuple[int, int]] = None,
) -> None:
    """Fused reduce + residual add + RMSNorm on this rank's rows, in place.

    hidden_states / residual: [total_tokens, hidden] — this rank's staging rows
    and the residual stream.  Same contract as the reference
    (tokenweave_utils.py:24-92).  `row_range=(start, end)` overrides the even
    split for ragged token counts (the reference pads instead, llama.py:536).
    """
    assert hidden_states.shape == residual.shape, \
        "hidden_states and residual must have the same shape"
    assert 0 <= rank < world_size, f"Invalid rank {rank}, must be in [0, {world_size - 1}]"
    total_tokens = hidden_states.shape[0]
    if row_range is None:
        expected_tokens = num_tokens_per_rank * world_size
        assert total_tokens == expected_tokens, (
            f"Mismatch in token count: expected {expected_tokens}, got {total_tokens}")
        start_idx = rank * num_tokens_per_rank
        end_idx = (rank + 1) * num_tokens_per_rank
    else:
        start_idx, end_idx = row_range
        assert 0 <= start_idx <= end_idx <= total_tokens, \
            f"row_range {row_range} outside [0, {total_tokens}]"
    rows = end_idx - start_idx
    if rows == 0:
        return
    row_bytes = hidden_states.shape[1] * hidden_states.element_size()
    layernorm(
        hidden_states[start_idx:end_idx],
        residual[start_idx:end_idx],
        MAX_CTAS=min(MAX_CTAS, rows),
        fused_ar=True,
        symm_mem_hdl=symm_mem_hdl,
        rank=rank,
        world_size=world_size,
        offset=offset_symm_mem + start_idx * row_bytes,
    )


def tokenweave_split_size(num_tokens: int, split_offset: int = 0) -> int:
    """Rows of the first token split (vllm/model_executor/models/llama.py:521):
    half of the token count rounded up to a multiple of 256, plus an offset."""
    return ((num_tokens + 255) & ~255) // 2 + split_offset


def weave_norm_gemm(gemm: Callable[[], None], norm: Callable[[], None],
                    norm_stream: torch.cuda.Stream, gemm_first: bool = True) -> None:
    """One weave stage: `norm` (the fused reduce+norm of one token split) runs on
    `norm_stream` while `gemm` (the other split's row-parallel GEMM) runs on the
    current stream, with the reference's hand-offs on both sides
    (tokenweave_utils.py:238-260): the norm waits for everything queued on the
    current stream before the stage, and the current stream afterwards waits for
    the norm.  Both streams keep the default priority.

    The reference enqueues the communication kernel first.  Here the GEMM goes
    first by default: capped to its compute-unit budget it leaves the other units
    idle, and the norm's one-workgroup-per-row grid then fills exactly those; the
    other order lets the norm occupy every unit and the GEMM's workgroups queue
    behind it (measured on MI355X: 82 us against 112 us for the 2458/1638-row
    split)."""
    current = torch.cuda.current_stream()
    if not gemm_first:
        norm_stream.wait_stream(current)
        with torch.cuda.stream(norm_stream):
            norm()
        gemm()
    else:
        before = torch.cuda.Event()
        before.record(current)
        gemm()
        norm_stream.wait_event(before)
        with torch.cuda.stream(norm_stream):
            norm()
    current.wait_stream(norm_stream)


def _shard_rows(total_tokens: int, rank: int, world_size: int, all_ranks: bool):
    """row_range for fused_allreduce_layernorm: None = the reference's even split
    for `rank`; every row when one process plays all the ranks."""
    return (0, total_tokens) if all_ranks else None


def tokenweave_with_fuse_only(
    self,
    positions: torch.Tensor,
    hidden_states: torch.Tensor,
    residual: Optional[torch.Tensor],
    symm_mem_hdl: Any,
    layer_id: int,
    rank: int = 0,
    world_size: int = 1,
    next_layer_norm: Optional[RMSNorm] = None,
    actual_tokens: Optional[int] = None,
    nearest_multiple_of_world_size: Optional[int] = None,
    MAX_CTAS_ATTN: int = 16,
    MAX_CTAS_MLP: int = 16,
    mlp_fn: Optional[Callable] = None,
    all_ranks: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """One decoder layer with the fused reduce + add + norm after attention and
    after the MLP, no overlap (reference tokenweave_utils.py:95-172, same
    arguments).  `self` is the layer: it provides `input_layernorm`,
    `post_attention_layernorm` and `self_attn(positions=, hidden_states=)`, whose
    row-parallel output projection leaves this rank's partial sum in
    `hidden_states` (this rank's staging rows); `mlp_fn` does the same for the MLP.

    `all_ranks=True` (no counterpart in the reference) normalises every row instead
    of this rank's shard: one GPU standing in for all the ranks, whose shards the
    all-gather would have delivered."""
    assert mlp_fn is not None, "mlp_fn must be provided"
    num_tokens_per_rank = nearest_multiple_of_world_size // world_size
    rows = _shard_rows(hidden_states.shape[0], rank, world_size, all_ranks)
    if residual is None:
        residual = torch.empty_like(hidden_states)
    if layer_id == 0:
        self.input_layernorm(hidden_states, out=residual)

    self.self_attn(positions=positions, hidden_states=hidden_states[:actual_tokens])
    fused_allreduce_layernorm(
        layernorm=self.post_attention_layernorm, hidden_states=hidden_states, residual=residual,
        symm_mem_hdl=symm_mem_hdl, num_tokens_per_rank=num_tokens_per_rank, rank=rank,
        world_size=world_size, MAX_CTAS=MAX_CTAS_ATTN, row_range=rows)
    mlp_fn(hidden_states[:actual_tokens])
    fused_allreduce_layernorm(
        layernorm=next_layer_norm, hidden_states=hidden_states, residual=residual,
        symm_mem_hdl=symm_mem_hdl, num_tokens_per_rank=num_tokens_per_rank, rank=rank,
        world_size=world_size, MAX_CTAS=MAX_CTAS_MLP, row_range=rows)
    return hidden_states, residual


def tokenweave_overlap(
    self,
    positions: torch.Tensor,
    hidden_states: torch.Tensor,
    residual: Optional[torch.Tensor],
    symm_mem_hdl: Any,
    layer_id: int,
    end_layer: Optional[int] = None,
    rank: int = 0,
    world_size: int = 1,
    current_stream: Optional[torch.cuda.Stream] = None,
    copy_stream: Optional[torch.cuda.Stream] = None,
    next_layer_norm: Optional[RMSNorm] = None,
    split_size: Optional[int] = None,
    actual_tokens: Optional[int] = None,
    num_tokens_padded: Optional[int] = None,
    MAX_CTAS_ATTN: int = 16,
    MAX_CTAS_MLP: int = 16,
    mlp_fn: Optional[Callable] = None,
    all_ranks: bool = False,
    gemm_cus: int = 0,
    mlp_gemm_cus: Optional[int] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """One decoder layer under the TokenWeave schedule (reference
    tokenweave_utils.py:175-340, same arguments and the same order of hand-offs):
    the tokens are cut at `split_size`; while one split computes (attention, MLP) on
    `current_stream`, the fused reduce + add + norm of the other runs on
    `copy_stream`.  Every compute step ends with `current_stream.wait_stream(copy_stream)`
    and every norm starts with `copy_stream.wait_stream(current_stream)`, exactly as
    in the reference, so the result equals the unsplit schedule's.

    Layer 0 (reference :203-226): split 0 has nothing to reduce and takes
    `input_layernorm(x, out=residual)`; for split 1 the reference reduce-scatters,
    normalises its shard and all-gathers — on one GPU that is the fused op on a
    zeroed residual (residual <- sum of the partials, x <- norm of it).
    The last layer normalises split 1 after its MLP on the current stream (:327-339).

    `gemm_cus` / `mlp_gemm_cus` (no counterpart in the reference; `weave_plan(...)`) are the
    compute-unit budgets of the GEMMs that run beside a norm (`mlp_gemm_cus` defaults to
    `gemm_cus`): when non-zero they are handed to
    `self.self_attn(..., gemm_cus=)` and `mlp_fn(hidden_states, gemm_cus=)`, which pass it as
    `max_cus` to their row-parallel output projection (`ops.gemm_bf16_nt` /
    `ops.gemm_bf16_nt_partials`) so that the norm's workgroups find free compute units.  On
    MI355X that, not the norm's grid cap, is the knob of the overlap.

    The two norms that the reference launches with hard-coded grids (8 CTAs in layer
    0, 16 or 32 after the last layer) have nothing to share the GPU with and are
    launched uncapped here: on MI355X a compute unit streams at most ~45 GB/s, so a
    grid of N workgroups is limited to N times that."""
    assert mlp_fn is not None, "mlp_fn must be provided"
    hidden = hidden_states.shape[1]
    offset_second = split_size * hidden * hidden_states.element_size()
    if residual is None:
        residual = torch.empty_like(hidden_states)
    hidden_states_1, hidden_states_2 = hidden_states[:split_size], hidden_states[split_size:]
    residual_1, residual_2 = residual[:split_size], residual[split_size:]
    blpr_1 = split_size // world_size
    blpr_2 = hidden_states_2.shape[0] // world_size
    rows_1 = _shard_rows(split_size, rank, world_size, all_ranks)
    rows_2 = _shard_rows(hidden_states_2.shape[0], rank, world_size, all_ranks)

    budget = {"gemm_cus": gemm_cus} if gemm_cus else {}
    mlp_cus = gemm_cus if mlp_gemm_cus is None else mlp_gemm_cus
    mlp_budget = {"gemm_cus": mlp_cus} if mlp_cus else {}

    def norm(layernorm, split, max_ctas):
        hs, res, blpr, off, rows = ((hidden_states_1, residual_1, blpr_1, 0, rows_1) if split == 0 else
                                    (hidden_states_2, residual_2, blpr_2, offset_second, rows_2))
        fused_allreduce_layernorm(
            layernorm=layernorm, hidden_states=hs, residual=res, symm_mem_hdl=symm_mem_hdl,
            num_tokens_per_rank=blpr, rank=rank, world_size=world_size, MAX_CTAS=max_ctas,
            offset_symm_mem=off, row_range=rows)

    if layer_id == 0:
        self.input_layernorm(hidden_states_1, out=residual_1)
        residual_2.zero_()
        norm(self.input_layernorm, 1, 0)
    else:
        with torch.cuda.stream(copy_stream):
            copy_stream.wait_stream(current_stream)
            norm(self.input_layernorm, 1, MAX_CTAS_ATTN)

    with torch.cuda.stream(current_stream):
        self.self_attn(positions=positions[:split_size], hidden_states=hidden_states_1, split_id=0,
                       split_size=split_size, num_actual_tokens=split_size, **budget)
        current_stream.wait_stream(copy_stream)
    with torch.cuda.stream(copy_stream):
        copy_stream.wait_stream(current_stream)
        norm(self.post_attention_layernorm, 0, MAX_CTAS_ATTN)

    with torch.cuda.stream(current_stream):
        self.self_attn(positions=positions[split_size:], hidden_states=hidden_states_2, split_id=1,
                       split_size=split_size, num_actual_tokens=actual_tokens - split_size, **budget)
        current_stream.wait_stream(copy_stream)
    with torch.cuda.stream(copy_stream):
        copy_stream.wait_stream(current_stream)
        norm(self.post_attention_layernorm, 1, MAX_CTAS_MLP)

    with torch.cuda.stream(current_stream):
        mlp_fn(hidden_states_1, **mlp_budget)
        current_stream.wait_stream(copy_stream)
    with torch.cuda.stream(copy_stream):
        copy_stream.wait_stream(current_stream)
        norm(next_layer_norm, 0, MAX_CTAS_MLP)

    with torch.cuda.stream(current_stream):
        mlp_fn(hidden_states_2, **mlp_budget)
        current_stream.wait_stream(copy_stream)

    if layer_id == end_layer - 1:
        with torch.cuda.stream(current_stream):
            norm(next_layer_norm, 1, 0)
    return hidden_states, residual
