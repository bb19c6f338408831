"""Modules on top of the low-precision ops (the callers of the hot path that the reference ships
in ``primus_turbo/pytorch/modules``: the FP8 linear layer and the grouped linear layer of an MoE
expert bank)."""

from .grouped_linear import GroupedLinear
from .linear_fp8 import Float8Linear

__all__ = ["Float8Linear", "GroupedLinear"]
