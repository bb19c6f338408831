"""Public quantize / dequantize entry points (reference: primus_turbo/pytorch/ops/quantization.py).

Same names, argument meaning and error behaviour as the reference ops; each call lands in
one gfx950 HIP kernel family through the impl layer.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from primus_turbo.pytorch.core.low_precision import (
    MXFP4_BLOCK_SIZE,
    MXFP8_BLOCK_SIZE,
    ScalingGranularity,
    ScalingRecipe,
)
from primus_turbo.pytorch.kernels.quantization import quantization_impl as _impl

__all__ = [
    "quantize_fp8",
    "quantize_fp8_with_trans",
    "dequantize_fp8",
    "quantize_fp4",
    "quantize_fp4_with_trans",
    "dequantize_fp4",
    "grouped_quantize_fp8",
    "grouped_quantize_fp8_with_trans",
    "grouped_dequantize_fp8",
    "grouped_quantize_fp4",
    "grouped_quantize_fp4_with_trans",
    "grouped_dequantize_fp4",
]

_G = ScalingGranularity


def _unknown(granularity):
    return NotImplementedError(f"Unknown granularity {granularity}")


def _need_mx_block(block_size, expect, what):
    assert block_size == expect, f"The block size must be {expect} for {what} quantization"


def quantize_fp8(
    x: torch.Tensor,
    out_dtype: torch.dtype,
    granularity: ScalingGranularity,
    *,
    block_size: Optional[int] = None,
    axis: Optional[int] = None,
    scaling_recipe: Optional[ScalingRecipe] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Quantize ``x`` to FP8; returns ``(x_fp8, scale_inv)``.

    ROWWISE needs ``axis``; BLOCKWISE needs ``block_size`` and either ``axis`` (1-D blocks)
    or ``scaling_recipe.use_2d_block`` (one scale per square tile, for weights);
    MX_BLOCKWISE needs a 2-D/3-D ``x``, ``block_size == 32`` and ``axis`` as the direction.
    """
    if granularity == _G.TENSORWISE:
        return _impl.quantize_fp8_tensorwise_impl(x, out_dtype)
    if granularity == _G.ROWWISE:
        return _impl.quantize_fp8_rowwise_impl(x, out_dtype, axis)
    if granularity == _G.BLOCKWISE:
        assert block_size is not None, "block_size must be specified for BLOCKWISE quantization"
        if scaling_recipe is not None and scaling_recipe.use_2d_block:
            return _impl.quant_fp8_blockwise_for_weight_impl(x, out_dtype, block_size=block_size)
        assert axis is not None, "axis must be specified for 1D BLOCKWISE quantization"
        return _impl.quant_fp8_blockwise_impl(x, out_dtype, axis=axis, block_size=block_size)
    if granularity == _G.MX_BLOCKWISE:
        _need_mx_block(block_size, MXFP8_BLOCK_SIZE, "MXFP8")
        return _impl.quantize_mxfp8_impl(x, out_dtype, axis, block_size, False, scaling_recipe)
    raise _unknown(granularity)


def quantize_fp8_with_trans(
    x: torch.Tensor,
    out_dtype: torch.dtype,
    granularity: ScalingGranularity,
    *,
    block_size: Optional[int] = None,
    scaling_recipe: Optional[ScalingRecipe] = None,
    scaling_recipe_for_trans: Optional[ScalingRecipe] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Quantize along both directions from one read of ``x``.

    Returns ``(x_rowwise, scale_inv_rowwise, x_colwise, scale_inv_colwise)``.
    """
    if granularity == _G.MX_BLOCKWISE:
        _need_mx_block(block_size, MXFP8_BLOCK_SIZE, "MXFP8")
        return _impl.quantize_mxfp8_impl(
            x, out_dtype, None, block_size, True, scaling_recipe, scaling_recipe_for_trans
        )
    if granularity == _G.BLOCKWISE:
        return _impl.quant_fp8_blockwise_dual_impl(x, out_dtype, block_size=block_size)
    raise _unknown(granularity)


def dequantize_fp8(
    x: torch.Tensor,
    out_dtype: torch.dtype,
    granularity: ScalingGranularity,
    *,
    block_size: Optional[int] = None,
    axis: Optional[int] = None,
    scale_inv: torch.Tensor,
    scaling_recipe: Optional[ScalingRecipe] = None,
):
    """Inverse of :func:`quantize_fp8` for the same granularity / axis / recipe."""
    if granularity == _G.TENSORWISE:
        return _impl.dequantize_fp8_tensorwise_impl(x, out_dtype, scale_inv)
    if granularity == _G.ROWWISE:
        if axis is None:
            raise ValueError("axis must be specified for rowwise FP8 de-quantization")
        return _impl.dequantize_fp8_rowwise_impl(x, out_dtype, axis, scale_inv)
    if granularity == _G.BLOCKWISE:
        assert block_size is not None, "block_size must be specified for BLOCKWISE de-quantization"
        if scaling_recipe is not None and scaling_recipe.use_2d_block:
            return _impl.dequant_fp8_blockwise_for_weight_impl(x, scale_inv, out_dtype, block_size)
        assert axis is not None, "axis must be specified for 1D BLOCKWISE de-quantization"
        return _impl.dequant_fp8_blockwise_impl(x, scale_inv, out_dtype, axis, block_size)
    if granularity == _G.MX_BLOCKWISE:
        _need_mx_block(block_size, MXFP8_BLOCK_SIZE, "MXFP8")
        if scaling_recipe is not None and (scaling_recipe.shuffle_out or scaling_recipe.shuffle_scale):
            assert x.dim() == 2, "shuffled layouts are de-quantized as 2-D tensors"
            x, scale_inv = _impl.mx_plain_layout(x, scale_inv, scaling_recipe.shuffle_out, scaling_recipe.shuffle_scale)
        return _impl.dequantize_mxfp8_impl(x, out_dtype, axis, block_size, scale_inv)
    raise _unknown(granularity)


def quantize_fp4(
    x: torch.Tensor,
    out_dtype: torch.dtype,
    granularity: ScalingGranularity,
    *,
    block_size: Optional[int] = None,
    axis: Optional[int] = None,
    scaling_recipe: Optional[ScalingRecipe] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """MXFP4 quantize in one direction (2-D: axis 1 = along rows, axis 0 = transposed output)."""
    if granularity == _G.MX_BLOCKWISE:
        _need_mx_block(block_size, MXFP4_BLOCK_SIZE, "MXFP4")
        assert axis is not None, "axis must be specified for MXFP4 quantization"
        return _impl.quantize_mxfp4_impl(
            x, out_dtype, axis, block_size, with_trans=False, scaling_recipe=scaling_recipe
        )
    raise _unknown(granularity)


def quantize_fp4_with_trans(
    x: torch.Tensor,
    out_dtype: torch.dtype,
    granularity: ScalingGranularity,
    *,
    block_size: Optional[int] = None,
    axis: Optional[int] = None,
    scaling_recipe: Optional[ScalingRecipe] = None,
    scaling_recipe_for_trans: Optional[ScalingRecipe] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """MXFP4 quantize in both directions from one read of ``x``."""
    if granularity == _G.MX_BLOCKWISE:
        _need_mx_block(block_size, MXFP4_BLOCK_SIZE, "MXFP4")
        return _impl.quantize_mxfp4_impl(
            x,
            out_dtype,
            axis,
            block_size,
            with_trans=True,
            scaling_recipe=scaling_recipe,
            scaling_recipe_for_trans=scaling_recipe_for_trans,
        )
    raise _unknown(granularity)


def dequantize_fp4(
    x: torch.Tensor,
    out_dtype: torch.dtype,
    granularity: ScalingGranularity,
    *,
    block_size: Optional[int] = None,
    axis: Optional[int] = None,
    scale_inv: torch.Tensor,
    scaling_recipe: Optional[ScalingRecipe] = None,
) -> torch.Tensor:
    if granularity == _G.MX_BLOCKWISE:
        _need_mx_block(block_size, MXFP4_BLOCK_SIZE, "MXFP4")
        if scaling_recipe is not None and (scaling_recipe.shuffle_out or scaling_recipe.shuffle_scale):
            assert x.dim() == 2, "shuffled layouts are de-quantized as 2-D tensors"
            x, scale_inv = _impl.mx_plain_layout(x, scale_inv, scaling_recipe.shuffle_out, scaling_recipe.shuffle_scale)
        return _impl.dequantize_mxfp4_impl(x, out_dtype, axis, block_size, scale_inv)
    raise _unknown(granularity)


# --- grouped MX quantizers (MoE experts): per-group padded layouts ------------------------------
def grouped_quantize_fp8(x, out_dtype, granularity, group_lens, group_offs, *, block_size=None, axis=None,
                         scaling_recipe=None):
    """Quantize the packed rows of G groups (MX_BLOCKWISE): ``axis`` 1 (or -1) -> rows, every group
    padded to 32 rows; ``axis`` 0 -> the transposed column direction, padded to 128.
    Returns ``(x_fp8, scale_inv, group_lens_padded, group_offs_padded)``."""
    if granularity == _G.MX_BLOCKWISE:
        _need_mx_block(block_size, MXFP8_BLOCK_SIZE, "MXFP8")
        assert axis is not None, "axis must be specified for grouped MXFP8 quantization"
        return _impl.grouped_quantize_mxfp8_impl(x, out_dtype, axis % x.dim(), block_size, group_lens, group_offs,
                                                 False, scaling_recipe)
    raise _unknown(granularity)


def grouped_quantize_fp8_with_trans(x, out_dtype, granularity, group_lens, group_offs, *, block_size=None,
                                    scaling_recipe=None, scaling_recipe_for_trans=None):
    """Both directions from one read of ``x``: ``(x_fp8_row, scale_row, x_fp8_col, scale_col,
    lens_padded_row, offs_padded_row, lens_padded_col, offs_padded_col)``."""
    if granularity == _G.MX_BLOCKWISE:
        _need_mx_block(block_size, MXFP8_BLOCK_SIZE, "MXFP8")
        return _impl.grouped_quantize_mxfp8_impl(x, out_dtype, None, block_size, group_lens, group_offs, True,
                                                 scaling_recipe, scaling_recipe_for_trans)
    raise _unknown(granularity)


def grouped_dequantize_fp8(x, out_dtype, granularity, group_offs, group_offs_padded, *, block_size=None, axis=None,
                           scale_inv=None, scaling_recipe=None, total_M=None):
    """Inverse of ``grouped_quantize_fp8``: the packed ``[total_M, N_pad]`` rows."""
    if granularity == _G.MX_BLOCKWISE:
        _need_mx_block(block_size, MXFP8_BLOCK_SIZE, "MXFP8")
        assert axis is not None and scale_inv is not None
        return _impl.grouped_dequantize_mxfp8_impl(x, out_dtype, axis % 2, block_size, scale_inv, group_offs,
                                                   group_offs_padded, total_M)
    raise _unknown(granularity)


def grouped_quantize_fp4(x, out_dtype, granularity, group_lens, group_offs, *, block_size=None, axis=None,
                         scaling_recipe=None):
    """MXFP4 quantization of the packed rows ``[total_m, N]`` of G groups in one direction
    (reference: ops/quantization.py:340-385): ``axis`` 1 -> rows, in place (row i = input row i, the
    returned padded lens / offs are the originals); ``axis`` 0 -> the transposed column direction
    ``[N, M_pad_col/2]`` with every group padded to 256 rows (the variable-K wgrad operand).
    Returns ``(data, scale_inv, group_lens_padded, group_offs_padded)``."""
    if granularity == _G.MX_BLOCKWISE:
        _need_mx_block(block_size, MXFP4_BLOCK_SIZE, "MXFP4")
        assert x.ndim == 2, "grouped MXFP4 quantize expects a 2D packed-M tensor"
        assert axis in (0, 1), "axis must be 0 (colwise) or 1 (rowwise) for grouped MXFP4"
        return _impl.grouped_quantize_mxfp4_impl(x, out_dtype, axis, block_size, group_lens, group_offs, False,
                                                 scaling_recipe)
    raise _unknown(granularity)


def grouped_quantize_fp4_with_trans(x, out_dtype, granularity, group_lens, group_offs, *, block_size=None,
                                    scaling_recipe=None, scaling_recipe_for_trans=None):
    """Both directions from one read of ``x`` (reference: ops/quantization.py:388-443):
    ``(row_q [total_m, N_pad/2], row_scale [total_m, N_pad/32], col_q [N, M_pad_col/2], col_scale
    [N, M_pad_col/32], group_lens, group_offs, lens_padded_col, offs_padded_col)``."""
    if granularity == _G.MX_BLOCKWISE:
        _need_mx_block(block_size, MXFP4_BLOCK_SIZE, "MXFP4")
        assert x.ndim == 2, "grouped MXFP4 quantize expects a 2D packed-M tensor"
        return _impl.grouped_quantize_mxfp4_impl(x, out_dtype, None, block_size, group_lens, group_offs, True,
                                                 scaling_recipe, scaling_recipe_for_trans)
    raise _unknown(granularity)


def grouped_dequantize_fp4(x, out_dtype, granularity, *, block_size=None, axis=None, scale_inv=None,
                           scaling_recipe=None):
    """Row-direction grouped MXFP4 data are plain rows: the dense de-quantizer
    (reference: ops/quantization.py:519-537)."""
    if granularity == _G.MX_BLOCKWISE:
        _need_mx_block(block_size, MXFP4_BLOCK_SIZE, "MXFP4")
        if scaling_recipe is not None and (scaling_recipe.shuffle_out or scaling_recipe.shuffle_scale):
            assert x.dim() == 2, "shuffled layouts are de-quantized as 2-D tensors"
            x, scale_inv = _impl.mx_plain_layout(x, scale_inv, scaling_recipe.shuffle_out, scaling_recipe.shuffle_scale)
        return _impl.dequantize_mxfp4_impl(x, out_dtype, axis, block_size, scale_inv)
    raise _unknown(granularity)
