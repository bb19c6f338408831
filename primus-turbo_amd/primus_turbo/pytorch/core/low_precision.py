"""Quantization configs and enums of the low-precision path.

Same names, fields and validation rules as the reference
(primus_turbo/pytorch/core/low_precision.py:105-213). This build targets gfx950
only, so the FP8 storage dtypes are always the OCP ones (``float8_e4m3fn`` /
``float8_e5m2``) and FP4 is ``float4_e2m1fn_x2``; importing never touches a GPU.
"""

from __future__ import annotations

from dataclasses import dataclass
from enum import Enum, auto
from typing import NamedTuple, Optional, Tuple

import torch

from primus_turbo.pytorch.core.utils import get_device_compute_capability

__all__ = ["float8_e4m3", "float8_e5m2"]

float8_e4m3 = torch.float8_e4m3fn
float8_e5m2 = torch.float8_e5m2
float4_e2m1fn_x2 = getattr(torch, "float4_e2m1fn_x2", None)

MXFP4_BLOCK_SIZE = 32
MXFP4_PADDING_ALIGN_SIZE = 128
MXFP8_BLOCK_SIZE = 32
MXFP8_PADDING_ALIGN_SIZE = 128
DEFAULT_BLOCK_SIZE = 128

_FP8_DTYPES = (torch.float8_e4m3fn, torch.float8_e4m3fnuz, torch.float8_e5m2, torch.float8_e5m2fnuz)


def is_fp8_dtype(dtype) -> bool:
    return dtype in _FP8_DTYPES


def is_fp4_dtype(dtype) -> bool:
    return float4_e2m1fn_x2 is not None and dtype == float4_e2m1fn_x2


def _needs(capability: Tuple[int, int], what: str) -> Tuple[bool, str]:
    if torch.cuda.is_available() and get_device_compute_capability() >= capability:
        return True, ""
    arch = "gfx942" if capability == (9, 4) else "gfx950"
    return False, f"Device compute capability {arch} or higher required for {what}."


def check_fp8_support() -> Tuple[bool, str]:
    return _needs((9, 4), "FP8 execution")


def check_fp8_ocp_support() -> Tuple[bool, str]:
    return _needs((9, 5), "FP8 OCP format")


def check_mxfp8_support() -> Tuple[bool, str]:
    return _needs((9, 5), "MXFP8 execution")


def check_mxfp4_support() -> Tuple[bool, str]:
    return _needs((9, 5), "FP4 execution")


class Format(Enum):
    """Element format of the quantized operands (HYBRID = E4M3 forward, E5M2 gradients)."""

    E4M3 = auto()
    E5M2 = auto()
    E2M1_X2 = auto()
    HYBRID = auto()


class ScaleDtype(Enum):
    FP32 = auto()
    E8M0 = auto()


class ScalingGranularity(Enum):
    TENSORWISE = auto()
    ROWWISE = auto()
    BLOCKWISE = auto()
    MX_BLOCKWISE = auto()


class ScalingStrategy(Enum):
    DYNAMIC = auto()


class ScalingRecipe(NamedTuple):
    """Per-operand quantization recipe.

    use_2d_block  one scale per square tile (128x128 FP8 blockwise, 32x32 MX) instead of 1-D blocks
    use_sr        stochastic rounding (MXFP4 only)
    use_rht       the recipe's fixed 16-point Hadamard transform before quantization (MXFP4 only)
    shuffle_scale / shuffle_out  pre-shuffled memory layouts (MXFP4 only)
    """

    use_2d_block: bool = False
    use_sr: bool = False
    use_rht: bool = False
    shuffle_scale: bool = False
    shuffle_out: bool = False


@dataclass
class Float8QuantConfig:
    format: Format = Format.E4M3
    granularity: ScalingGranularity = ScalingGranularity.TENSORWISE
    strategy: ScalingStrategy = ScalingStrategy.DYNAMIC
    scale_dtype: ScaleDtype = ScaleDtype.FP32
    block_size: Optional[int] = None

    def __post_init__(self):
        g = self.granularity
        if g == ScalingGranularity.BLOCKWISE:
            assert self.block_size is not None, "block_size must be set when granularity is BLOCKWISE"
        elif g == ScalingGranularity.MX_BLOCKWISE:
            allowed = [MXFP8_BLOCK_SIZE]
            assert self.block_size in allowed, f"block_size should be {allowed} when granularity is MX_BLOCKWISE"
            assert self.scale_dtype == ScaleDtype.E8M0, (
                f"scale_dtype should be {ScaleDtype.E8M0} when granularity is MX_BLOCKWISE"
            )


@dataclass
class Float4QuantConfig:
    format: Format = Format.E2M1_X2
    granularity: ScalingGranularity = ScalingGranularity.MX_BLOCKWISE
    strategy: ScalingStrategy = ScalingStrategy.DYNAMIC
    scale_dtype: ScaleDtype = ScaleDtype.E8M0
    block_size: int = 32
    use_gradient_sr: bool = False
    use_preshuffle: bool = False

    def __post_init__(self):
        assert self.granularity == ScalingGranularity.MX_BLOCKWISE, (
            "Float4QuantConfig currently only supports MX_BLOCKWISE granularity"
        )
        allowed = [MXFP4_BLOCK_SIZE]
        assert self.block_size in allowed, f"block_size should be {allowed} when granularity is MX_BLOCKWISE"
        assert self.format == Format.E2M1_X2, "Format must be E2M1_X2 for Float4QuantConfig"
        assert self.scale_dtype == ScaleDtype.E8M0, (
            f"scale_dtype should be {ScaleDtype.E8M0} when granularity is MX_BLOCKWISE"
        )
