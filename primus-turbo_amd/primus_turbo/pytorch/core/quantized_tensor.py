"""``QuantizedTensor``: low-precision payload + inverse scales + the recipe that made them.

The reference implements this as a ``torch.Tensor`` wrapper subclass with view / reshape /
FSDP flatten support (primus_turbo/pytorch/core/quantized_tensor.py:148-894). The ops of
this build only need the slice used by the GEMM wrappers — construct by quantizing,
carry ``qdata`` / ``scale_inv`` and the metadata ``check_quantized_tensor`` validates,
de-quantize, and transpose a tensorwise tensor — so it is a plain container here.
"""

from __future__ import annotations

from typing import NamedTuple, Optional

import torch

from primus_turbo import _native as N
from primus_turbo.pytorch.core.low_precision import (
    Float8QuantConfig,
    ScalingGranularity,
    ScalingRecipe,
    float4_e2m1fn_x2,
    float8_e4m3,
    float8_e5m2,
)

_SUPPORTED = tuple(d for d in (float8_e4m3, float8_e5m2, float4_e2m1fn_x2) if d is not None)


def _norm_axis(axis: Optional[int], ndim: int) -> Optional[int]:
    if axis is None:
        return None
    return axis if axis >= 0 else axis + ndim


class QuantizedTensor:
    """Container for a quantized tensor. ``shape`` / ``dtype`` describe the logical
    high-precision tensor, ``real_dtype`` the storage format."""

    def __init__(self, data: torch.Tensor, scale_inv: torch.Tensor, *, shape, orig_dtype: torch.dtype,
                 dest_dtype: torch.dtype, granularity: ScalingGranularity, block_size: Optional[int] = None,
                 scaling_recipe: Optional[ScalingRecipe] = None, quantized_axis: Optional[int] = None):
        assert dest_dtype in _SUPPORTED, "Unsupported quantized dtype"
        assert data.is_contiguous(), "data must be contiguous"
        assert scale_inv.is_contiguous(), "scale_inv must be contiguous"
        self._data, self._scale_inv = data, scale_inv
        self.shape = torch.Size(shape)
        self._orig_dtype, self._dest_dtype = orig_dtype, dest_dtype
        self._granularity, self._block_size = granularity, block_size
        self._scaling_recipe = scaling_recipe if scaling_recipe is not None else ScalingRecipe()
        self._quantized_axis = quantized_axis

    # -- construction ------------------------------------------------------------------
    @classmethod
    def quantize(cls, hp_tensor: torch.Tensor, dest_dtype: torch.dtype, granularity: ScalingGranularity, *,
                 axis: Optional[int] = None, block_size: Optional[int] = None,
                 scaling_recipe: Optional[ScalingRecipe] = None) -> "QuantizedTensor":
        from primus_turbo.pytorch.ops.quantization import quantize_fp4, quantize_fp8

        assert hp_tensor.ndim in (2, 3), f"data must be a 2D or 3D tensor, got {hp_tensor.ndim}D"
        x = hp_tensor.detach()
        if granularity in (ScalingGranularity.TENSORWISE, ScalingGranularity.ROWWISE):
            x = x.contiguous()
        if dest_dtype == float4_e2m1fn_x2 and float4_e2m1fn_x2 is not None:
            q, s = quantize_fp4(x, dest_dtype, granularity, block_size=block_size, axis=axis, scaling_recipe=scaling_recipe)
        else:
            q, s = quantize_fp8(x, dest_dtype, granularity, block_size=block_size, axis=axis, scaling_recipe=scaling_recipe)
        return cls(q, s, shape=hp_tensor.shape, orig_dtype=hp_tensor.dtype, dest_dtype=dest_dtype,
                   granularity=granularity, block_size=block_size, scaling_recipe=scaling_recipe,
                   quantized_axis=_norm_axis(axis, hp_tensor.ndim))

    # -- accessors ---------------------------------------------------------------------
    @property
    def qdata(self) -> torch.Tensor:
        return self._data

    @property
    def scale_inv(self) -> torch.Tensor:
        return self._scale_inv

    @property
    def dtype(self) -> torch.dtype:
        return self._orig_dtype

    @property
    def real_dtype(self) -> torch.dtype:
        return self._dest_dtype

    @property
    def granularity(self) -> ScalingGranularity:
        return self._granularity

    @property
    def block_size(self) -> Optional[int]:
        return self._block_size

    @property
    def scaling_recipe(self) -> ScalingRecipe:
        return self._scaling_recipe

    @property
    def quantized_axis(self) -> Optional[int]:
        return self._quantized_axis

    @property
    def device(self):
        return self._data.device

    @property
    def ndim(self) -> int:
        return len(self.shape)

    def dim(self) -> int:
        return len(self.shape)

    def is_contiguous(self) -> bool:
        return True

    def contiguous(self) -> "QuantizedTensor":
        return self

    def size(self, d=None):
        return self.shape if d is None else self.shape[d]

    # -- ops ---------------------------------------------------------------------------
    def dequantize(self) -> torch.Tensor:
        from primus_turbo.pytorch.ops.quantization import dequantize_fp4, dequantize_fp8

        fn = dequantize_fp4 if (float4_e2m1fn_x2 is not None and self._dest_dtype == float4_e2m1fn_x2) else dequantize_fp8
        return fn(self._data, self._orig_dtype, self._granularity, block_size=self._block_size,
                  axis=self._quantized_axis, scale_inv=self._scale_inv, scaling_recipe=self._scaling_recipe)

    def t(self) -> "QuantizedTensor":
        """Transpose of a 2-D tensorwise tensor (the payload is physically transposed; the
        single scale is shared)."""
        assert self._granularity == ScalingGranularity.TENSORWISE, "t() is provided for TENSORWISE tensors"
        assert self._data.dim() == 2
        R, C = self._data.shape
        out = torch.empty((C, R), dtype=self._data.dtype, device=self._data.device)
        N.check(N.lib().pt_transpose_u8(N.ptr(self._data), N.ptr(out), 1, R, C, N.stream_of(self._data)))
        return QuantizedTensor(out, self._scale_inv, shape=(self.shape[1], self.shape[0]), orig_dtype=self._orig_dtype,
                               dest_dtype=self._dest_dtype, granularity=self._granularity,
                               block_size=self._block_size, scaling_recipe=self._scaling_recipe,
                               quantized_axis=self._quantized_axis)

    def __repr__(self) -> str:
        return (f"QuantizedTensor(shape={tuple(self.shape)}, dtype={self._orig_dtype}, real_dtype={self._dest_dtype}, "
                f"granularity={self._granularity.name}, axis={self._quantized_axis}, block_size={self._block_size})")


class QuantizedTensorPair(NamedTuple):
    """A tensor quantized for the forward layout plus its counterpart for the backward layout."""

    data: QuantizedTensor
    data_t: Optional[QuantizedTensor] = None


def check_quantized_tensor(t: QuantizedTensor, config, axis: Optional[int] = None,
                           scaling_recipe: Optional[ScalingRecipe] = None) -> None:
    """Validate that a pre-quantized operand matches what the op would have produced."""
    assert isinstance(t, QuantizedTensor)
    assert t.granularity == config.granularity, (
        f"QuantizedTensor granularity {t.granularity} does not match config {config.granularity}"
    )
    if config.granularity in (ScalingGranularity.BLOCKWISE, ScalingGranularity.MX_BLOCKWISE):
        assert t.block_size == config.block_size, "QuantizedTensor block_size does not match the config"
    if axis is not None and t.quantized_axis is not None:
        assert t.quantized_axis == _norm_axis(axis, t.ndim), (
            f"QuantizedTensor was quantized along axis {t.quantized_axis}, expected {_norm_axis(axis, t.ndim)}"
        )
    if scaling_recipe is not None:
        assert t.scaling_recipe.use_2d_block == scaling_recipe.use_2d_block, "scaling recipe (2-D block) mismatch"
