"""Row-parallel linear layer with the reference's TokenWeave call surface.

Mirror of ``RowParallelLinear.forward(input_, output_, is_tokenweave=True)``
(``vllm/model_executor/layers/linear.py:1290-1334``) over
``UnquantizedLinearMethod.apply_inplace`` (``:203-228``): the layer's GEMM writes
this rank's partial sum straight into a preallocated output — the rank's staging
rows — and leaves the reduction to the fused norm that follows
(``vllm/model_executor/models/llama.py:99-103, 248-249``).  The weight is this
rank's slice ``[output_size, input_size / tp_size]``; only rank 0 adds the bias, so
the sum over the ranks holds it once (``linear.py:1306-1308``).

There is no process group on one GPU: ``tp_rank`` and ``tp_size`` are constructor
arguments, and the default (non-TokenWeave) mode, which all-reduces its result in
the reference, is available only where that all-reduce is the identity.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn as nn
from torch.nn.parameter import Parameter

from . import _custom_ops as ops


class UnquantizedLinearMethod:
    """``apply`` / ``apply_inplace`` of the reference's unquantised method
    (linear.py:195-228) on the library's bf16 MFMA GEMM.  ``max_cus`` (no counterpart in
    the reference) is the GEMM's compute-unit budget under the weave schedule."""

    def apply(self, layer: nn.Module, x: torch.Tensor, bias: Optional[torch.Tensor] = None,
              max_cus: Optional[int] = None) -> torch.Tensor:
        output = torch.empty(x.shape[:-1] + (layer.weight.shape[0],), dtype=x.dtype, device=x.device)
        return self.apply_inplace(layer, x, output, bias, max_cus)

    def apply_inplace(self, layer: nn.Module, x: torch.Tensor, output: torch.Tensor,
                      bias: Optional[torch.Tensor] = None, max_cus: Optional[int] = None) -> torch.Tensor:
        """output <- x @ layer.weight.T, then output += bias (if given), both in place."""
        w = layer.weight.data
        x2 = x.reshape(-1, x.shape[-1])
        out2 = output if output.dim() == 2 else output.view(-1, output.shape[-1])
        ops.gemm_bf16_nt(out2, x2, w, max_cus, None if bias is None else bias.data)
        return output


class RowParallelLinear(nn.Module):
    """Y = X A + b with A split along its first dimension (X along its last) over
    ``tp_size`` ranks; this module is rank ``tp_rank``'s share.  Constructor and
    ``forward`` follow linear.py:1185-1334."""

    def __init__(self, input_size: int, output_size: int, bias: bool = True, input_is_parallel: bool = True,
                 skip_bias_add: bool = False, params_dtype: Optional[torch.dtype] = None,
                 reduce_results: bool = True, *, tp_rank: int = 0, tp_size: int = 1,
                 return_bias: bool = True) -> None:
        super().__init__()
        if not 0 <= tp_rank < tp_size:
            raise ValueError(f"Invalid rank {tp_rank}, must be in [0, {tp_size - 1}]")
        if input_size % tp_size != 0:
            raise ValueError(f"{input_size} is not divisible by {tp_size}")
        if not reduce_results and (bias and not skip_bias_add):
            raise ValueError("When not reduce the results, adding bias to the "
                             "results can lead to incorrect results")
        self.tp_rank, self.tp_size = tp_rank, tp_size
        self.input_size, self.output_size = input_size, output_size
        self.input_size_per_partition = input_size // tp_size
        self.output_size_per_partition = output_size
        self.input_is_parallel = input_is_parallel
        self.skip_bias_add = skip_bias_add
        self.reduce_results = reduce_results
        self.return_bias = return_bias
        self.params_dtype = params_dtype or torch.bfloat16
        self.quant_method = UnquantizedLinearMethod()
        self.weight = Parameter(torch.empty(output_size, self.input_size_per_partition, dtype=self.params_dtype),
                                requires_grad=False)
        if bias:
            self.bias = Parameter(torch.empty(output_size, dtype=self.params_dtype), requires_grad=False)
        else:
            self.register_parameter("bias", None)

    def weight_loader(self, param: Parameter, loaded_weight: torch.Tensor) -> None:
        """This rank's slice of a full weight along the input dimension; biases whole
        (linear.py:1243-1277)."""
        if param is self.weight and loaded_weight.shape[1] != self.input_size_per_partition:
            shard = self.input_size_per_partition
            loaded_weight = loaded_weight.narrow(1, self.tp_rank * shard, shard)
        assert param.data.shape == loaded_weight.shape
        param.data.copy_(loaded_weight)

    def forward(self, input_: torch.Tensor, output_: Optional[torch.Tensor] = None,
                is_tokenweave: Optional[bool] = False, gemm_cus: Optional[int] = None
                ) -> Tuple[torch.Tensor, Optional[Parameter]]:
        if self.input_is_parallel:
            input_parallel = input_
        else:
            shard = self.input_size_per_partition
            input_parallel = input_[..., self.tp_rank * shard:(self.tp_rank + 1) * shard].contiguous()
        # Only rank 0 adds the bias, so that the sum over the ranks holds it once.
        bias_ = None if (self.tp_rank > 0 or self.skip_bias_add) else self.bias
        output_bias = self.bias if self.skip_bias_add else None
        if is_tokenweave:
            assert output_ is not None, "TokenWeave requires a preallocated output tensor"
            output = self.quant_method.apply_inplace(self, input_parallel, output=output_, bias=bias_,
                                                     max_cus=gemm_cus)
        else:
            if self.reduce_results and self.tp_size > 1:
                raise RuntimeError(
                    "RowParallelLinear without is_tokenweave=True all-reduces its result over the "
                    "tensor-parallel group; there are no collectives on one GPU — write the partial "
                    "sum into the staging rows (is_tokenweave=True) and let the fused norm reduce it")
            output = self.quant_method.apply(self, input_parallel, bias=bias_, max_cus=gemm_cus)
        if not self.return_bias:
            return output
        return output, output_bias

    def extra_repr(self) -> str:
        s = f"input_features={self.input_size_per_partition}"
        s += f", output_features={self.output_size}"
        s += f", bias={self.bias is not None}"
        s += f", tp_size={self.tp_size}"
        s += f", reduce_results={self.reduce_results}"
        return s
