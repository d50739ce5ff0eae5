"""tokenweave_amd: MI355X-native fused P-partial reduce + residual-add + RMSNorm.

Python host side over the C ABI in ``include/tokenweave_amd.h``; mirrors the
reference's op shims (``vllm/_custom_ops.py:176-221``), its ``RMSNorm`` layer
(``vllm/model_executor/layers/layernorm.py``) and
``fused_allreduce_layernorm`` (``vllm/model_executor/models/tokenweave_utils.py:24-92``).
"""
from . import _custom_ops as ops  # noqa: F401
from .layernorm import RMSNorm  # noqa: F401
from .linear import RowParallelLinear, UnquantizedLinearMethod  # noqa: F401
from .tokenweave_utils import (PartialsBuffer, fused_allreduce_layernorm,  # noqa: F401
                               load_config, select_config, shard_bounds, tokenweave_split_size,
                               tokenweave_overlap, tokenweave_with_fuse_only,
                               weave_norm_gemm, weave_plan)

__all__ = ["ops", "RMSNorm", "RowParallelLinear", "UnquantizedLinearMethod", "PartialsBuffer", "fused_allreduce_layernorm", "shard_bounds",
           "tokenweave_split_size", "tokenweave_with_fuse_only", "tokenweave_overlap", "weave_norm_gemm", "load_config", "select_config", "weave_plan"]
__version__ = "0.1.0"
