"""RMSNorm layer with the reference's call surface.

Mirror of ``vllm/model_executor/layers/layernorm.py``: the module-level helpers
(:21-104) and ``RMSNorm`` with ``forward_native`` (:173-210) and the keyword
surface of ``forward_cuda`` (:212-281), so the call sites in the reference's
model files (``layer(x, residual, MAX_CTAS=..., fused_ar=True, symm_mem_hdl=...,
rank=..., world_size=..., offset=...)``) work unchanged.
"""
from __future__ import annotations

from typing import Any, Optional, Tuple, Union

import torch
import torch.nn as nn

from . import _custom_ops as ops


def rms_norm(x: torch.Tensor, weight: torch.Tensor, variance_epsilon: float) -> torch.Tensor:
    out = torch.empty_like(x)
    ops.rms_norm(out, x, weight, variance_epsilon)
    return out


def rms_norm_inplace(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor,
                     variance_epsilon: float) -> torch.Tensor:
    ops.rms_norm_inplace(out, x, weight, variance_epsilon)
    return x


def fused_add_rms_norm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                       variance_epsilon: float) -> Tuple[torch.Tensor, torch.Tensor]:
    ops.fused_add_rms_norm(x, residual, weight, variance_epsilon)
    return x, residual


def fused_add_rms_norm_cta(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                           MAX_CTAS: int,
                           variance_epsilon: float) -> Tuple[torch.Tensor, torch.Tensor]:
    ops.fused_add_rms_norm_cta(x, residual, weight, MAX_CTAS, variance_epsilon)
    return x, residual


def fused_rs_ln_ag_cta(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                       symm_mem_hdl, rank: int, world_size: int, MAX_CTAS: int, offset: int,
                       variance_epsilon: float) -> Tuple[torch.Tensor, torch.Tensor]:
    ops.fused_rs_ln_ag_cta(x, residual, weight, symm_mem_hdl.multicast_ptr + offset,
                           symm_mem_hdl.signal_pad_ptrs_dev, rank, world_size, MAX_CTAS,
                           variance_epsilon)
    return x, residual


def fused_rs_ln_cta(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                    symm_mem_hdl, rank: int, world_size: int, MAX_CTAS: int, offset: int,
                    variance_epsilon: float) -> Tuple[torch.Tensor, torch.Tensor]:
    ops.fused_rs_ln_cta(x, residual, weight, symm_mem_hdl.multicast_ptr + offset,
                        symm_mem_hdl.signal_pad_ptrs_dev, rank, world_size, MAX_CTAS,
                        variance_epsilon)
    return x, residual


class RMSNorm(nn.Module):
    """Root mean square normalization: x -> w * x / sqrt(E[x^2] + eps).

    ``forward`` is the reference's ``forward_cuda`` (its CustomOp dispatch sends
    CUDA, ROCm and CPU there, vllm/model_executor/custom_op.py:38-49,72-101).
    """

    def __init__(self, hidden_size: int, eps: float = 1e-6,
                 var_hidden_size: Optional[int] = None, has_weight: bool = True,
                 dtype: Optional[torch.dtype] = None) -> None:
        super().__init__()
        self.hidden_size = hidden_size
        self.variance_epsilon = eps
        self.variance_size_override = (None if var_hidden_size == hidden_size
                                       else var_hidden_size)
        self.has_weight = has_weight
        if dtype is not None:
            self.weight = torch.ones(hidden_size, dtype=dtype)
        else:
            self.weight = torch.ones(hidden_size)
        if self.has_weight:
            self.weight = nn.Parameter(self.weight)

    def forward_native(
        self, x: torch.Tensor, residual: Optional[torch.Tensor] = None,
        out: Optional[torch.Tensor] = None,
    ) -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
        """The op in plain torch, not in place: fp32 sum and mean of squares, one
        rounding to the input dtype, then the weight multiply in that dtype
        (semantics of layernorm.py:173-210, the reference's unit-test oracle)."""
        if x.shape[-1] != self.hidden_size:
            raise ValueError("Expected hidden_size to be "
                             f"{self.hidden_size}, but found: {x.shape[-1]}")
        n_var = self.variance_size_override
        if n_var is not None and self.hidden_size < n_var:
            raise ValueError("Expected hidden_size to be at least "
                             f"{n_var}, but found: {self.hidden_size}")
        acc = x.float()
        new_residual = None
        if residual is not None:
            acc = acc + residual.float()
            new_residual = acc.to(x.dtype)
        squares = (acc if n_var is None else acc[..., :n_var]).square()
        inv = torch.rsqrt(squares.mean(dim=-1, keepdim=True) + self.variance_epsilon)
        y = (acc * inv).to(x.dtype)
        if self.has_weight:
            y = y * self.weight
        return y if new_residual is None else (y, new_residual)

    def forward_cuda(
        self, x: torch.Tensor, residual: Optional[torch.Tensor] = None,
        out: Optional[torch.Tensor] = None, MAX_CTAS: Optional[int] = None,
        fused_ar: Optional[bool] = False, fused_rs: Optional[bool] = False,
        symm_mem_hdl: Optional[Any] = None, rank: Optional[int] = 0,
        world_size: Optional[int] = 1, offset: Optional[int] = 0,
    ) -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
        if self.variance_size_override is not None:
            return self.forward_native(x, residual)
        w = self.weight.data
        eps = self.variance_epsilon
        if fused_ar:
            return fused_rs_ln_ag_cta(x, residual, w, symm_mem_hdl, rank, world_size, MAX_CTAS,
                                      offset, eps)
        if fused_rs:
            return fused_rs_ln_cta(x, residual, w, symm_mem_hdl, rank, world_size, MAX_CTAS,
                                   offset, eps)
        if residual is not None:
            if MAX_CTAS is None:
                return fused_add_rms_norm(x, residual, w, eps)
            return fused_add_rms_norm_cta(x, residual, w, MAX_CTAS, eps)
        if out is None:
            return rms_norm(x, w, eps)
        return rms_norm_inplace(out, x, w, eps)

    forward = forward_cuda

    def extra_repr(self) -> str:
        s = f"hidden_size={self.weight.data.size(0)}"
        s += f", eps={self.variance_epsilon}"
        return s
