"""``GroupedLinear``: ``group_num`` expert weights ``[group_num, out_features, in_features]`` applied
to the packed token rows of their groups through the low-precision grouped GEMMs.

Constructor, parameter layout, initialisation, ``forward(x, group_lens, group_offs=None)`` and
``extra_repr`` are those of the reference's module (primus_turbo/pytorch/modules/grouped_linear.py:
17-52). The reference's module multiplies in bf16 (its ``grouped_gemm`` op); the bf16 grouped GEMM is
not part of the low-precision path, so this module takes the quantization ``config`` that the
reference's callers pass to ``grouped_gemm_fp8`` / ``grouped_gemm_fp4`` themselves: as a keyword of
the constructor, or assigned to ``module.config`` afterwards. Constructing without one works, as
with the reference (existing call sites keep constructing); ``forward`` then raises rather than
changing a caller's numerics behind its back."""

from __future__ import annotations

import math
from typing import Optional, Union

import torch
from torch import nn

from primus_turbo.pytorch.core.low_precision import Float4QuantConfig, Float8QuantConfig
from primus_turbo.pytorch.ops.grouped_gemm_fp4 import grouped_gemm_fp4
from primus_turbo.pytorch.ops.grouped_gemm_fp8 import grouped_gemm_fp8

__all__ = ["GroupedLinear"]


class GroupedLinear(nn.Module):
    def __init__(self, group_num: int, in_features: int, out_features: int, device=None, dtype=None, *,
                 config: Optional[Union[Float8QuantConfig, Float4QuantConfig]] = None):
        super().__init__()
        assert config is None or isinstance(config, (Float8QuantConfig, Float4QuantConfig)), f"unsupported config {type(config)}"
        self.in_features, self.out_features, self.group_num = in_features, out_features, group_num
        self.dtype, self.config = dtype, config
        self.weight = nn.Parameter(torch.empty((group_num, out_features, in_features), device=device, dtype=dtype))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        if not self.weight.is_meta:
            nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))

    def forward(self, x: torch.Tensor, group_lens: torch.Tensor, group_offs: Optional[torch.Tensor] = None) -> torch.Tensor:
        if self.config is None:
            raise NotImplementedError(
                "GroupedLinear.forward needs a Float8QuantConfig or Float4QuantConfig (constructor keyword `config`, or "
                "assign `module.config`): the unquantized (bf16) grouped GEMM is not part of this library"
            )
        op = grouped_gemm_fp4 if isinstance(self.config, Float4QuantConfig) else grouped_gemm_fp8
        return op(x, self.weight, group_lens, group_offs, trans_b=True, config=self.config)

    def extra_repr(self) -> str:
        return (f"group_num={self.group_num},in_features={self.in_features}, out_features={self.out_features}, "
                f"config={self.config}")
