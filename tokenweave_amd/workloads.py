"""Seeded synthetic inputs for the benchmark configurations of the fused
reduce + residual-add + RMSNorm path, and the byte count used for bandwidth.

Tensors are generated on the requested device with a ``torch.Generator`` seeded
per configuration, so the GPU path and a CPU checker can be fed identical bits
(copy the tensors; do not regenerate on another device).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch


def algorithmic_bytes(P: int, T: int, H: int) -> int:
    """bf16 bytes one call must move: P partial reads, residual read + write,
    y write, weight read once."""
    return P * T * H * 2 + 2 * T * H * 2 + T * H * 2 + H * 2


@dataclass(frozen=True)
class NormConfig:
    name: str
    P: int
    T: int
    H: int
    eps: float
    seed: int
    partial_dist: str = "normal"   # "normal": N(0, partial_std^2); "student_t3": t(3) * partial_scale
    partial_std: float = 1.0
    partial_scale: float = 1.0
    residual_std: float = 1.0
    weight_dist: str = "normal"    # "normal": N(1, 0.1^2); "uniform": U(0.5, 1.5)

    @property
    def bytes(self) -> int:
        return algorithmic_bytes(self.P, self.T, self.H)

    def with_tokens(self, T: int, name: Optional[str] = None) -> "NormConfig":
        d = dict(self.__dict__)
        d["T"] = T
        d["name"] = name or f"{self.name.split('@')[0]}@T{T}"
        return NormConfig(**d)


_INV_SQRT8 = 8.0 ** -0.5  # "N(0, 1/8)" is read as variance 1/8: the 8-way sum is ~N(0, 1)

C1 = NormConfig("c1_add_rmsnorm", P=1, T=512, H=8192, eps=1e-5, seed=1001)
C2 = NormConfig("c2_llama70b_tp8_shard", P=8, T=256, H=8192, eps=1e-5, seed=1002,
                partial_std=_INV_SQRT8)
C2_TOKENS = (1, 8, 32, 256, 1024)
C3 = NormConfig("c3_qwen72b_ragged", P=8, T=3001, H=8192, eps=1e-6, seed=1003,
                partial_dist="student_t3", partial_scale=1.0 / 8.0, residual_std=2.0,
                weight_dist="uniform")
C4 = NormConfig("c4_mixtral_8x22b_chunk", P=8, T=8192, H=6144, eps=1e-5, seed=1004,
                partial_std=_INV_SQRT8)
C5_NORM = NormConfig("c5_weave_norm_split", P=8, T=1638, H=8192, eps=1e-5, seed=1005,
                     partial_std=_INV_SQRT8)
C5_TOTAL_TOKENS = 4096
C5_GEMM_ROWS = 2458          # 60 % split: o_proj runs on these rows
C5_GEMM_K = 1024             # 8192 / 8: this rank's slice of the attention output
C5_WEIGHT_STD = 0.02


def norm_configs() -> Dict[str, NormConfig]:
    out = {C1.name: C1}
    for t in C2_TOKENS:
        c = C2.with_tokens(t)
        out[c.name] = c
    out[C3.name] = C3
    out["c3_shard_floor@T376"] = C3.with_tokens(376, "c3_shard_floor@T376")
    out["c3_shard_ceil@T369"] = C3.with_tokens(369, "c3_shard_ceil@T369")
    out[C4.name] = C4
    out[C5_NORM.name] = C5_NORM
    return out


@dataclass
class NormInputs:
    cfg: NormConfig
    partials: List[torch.Tensor]   # P x [T, H] bf16 (views of `staging` when it exists)
    residual: torch.Tensor         # [T, H] bf16
    weight: torch.Tensor           # [H] bf16
    staging: Optional[torch.Tensor] = None  # [P, T, H] when the partials are contiguous slots


def _generator(device, seed: int) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def make_norm_inputs(cfg: NormConfig, device="cuda", seed_offset: int = 0) -> NormInputs:
    """Draw one input set.  `seed_offset` gives independent sets for buffer rotation."""
    dev = torch.device(device)
    g = _generator(dev, cfg.seed + 7919 * seed_offset)
    shape = (cfg.P, cfg.T, cfg.H)
    if cfg.partial_dist == "normal":
        stage = torch.randn(shape, generator=g, device=dev, dtype=torch.float32) * cfg.partial_std
    elif cfg.partial_dist == "student_t3":
        z = torch.randn(shape, generator=g, device=dev, dtype=torch.float32)
        chi2 = torch.zeros(shape, device=dev, dtype=torch.float32)
        for _ in range(3):
            chi2 += torch.randn(shape, generator=g, device=dev, dtype=torch.float32).square_()
        stage = z / torch.sqrt(chi2 / 3.0) * cfg.partial_scale
        del z, chi2
    else:
        raise ValueError(cfg.partial_dist)
    stage = stage.to(torch.bfloat16)
    residual = (torch.randn((cfg.T, cfg.H), generator=g, device=dev, dtype=torch.float32)
                * cfg.residual_std).to(torch.bfloat16)
    if cfg.weight_dist == "normal":
        weight = 1.0 + 0.1 * torch.randn((cfg.H,), generator=g, device=dev, dtype=torch.float32)
    elif cfg.weight_dist == "uniform":
        weight = 0.5 + torch.rand((cfg.H,), generator=g, device=dev, dtype=torch.float32)
    else:
        raise ValueError(cfg.weight_dist)
    weight = weight.to(torch.bfloat16)
    return NormInputs(cfg, [stage[p] for p in range(cfg.P)], residual, weight, stage)


@dataclass
class GemmInputs:
    a: torch.Tensor   # [M, K] bf16 activations of the GEMM split
    b: torch.Tensor   # [N, K] bf16 weight (row-parallel slice of o_proj)


def make_partials_gemm_inputs(P: int = 8, M: int = C5_GEMM_ROWS, N: int = 8192, K: int = C5_GEMM_K,
                              device="cuda", seed: int = C5_NORM.seed + 2,
                              weight_std: float = C5_WEIGHT_STD) -> List["GemmInputs"]:
    """The row-parallel GEMMs of P simulated ranks on one token split: rank p holds its own
    K-slice of the activations and of the weight."""
    return [make_gemm_inputs(M, N, K, device, seed + 101 * p, weight_std) for p in range(P)]


def make_gemm_inputs(M: int = C5_GEMM_ROWS, N: int = 8192, K: int = C5_GEMM_K, device="cuda",
                     seed: int = C5_NORM.seed + 1, weight_std: float = C5_WEIGHT_STD) -> GemmInputs:
    dev = torch.device(device)
    g = _generator(dev, seed)
    a = torch.randn((M, K), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    b = (torch.randn((N, K), generator=g, device=dev, dtype=torch.float32) * weight_std).to(torch.bfloat16)
    return GemmInputs(a, b)
