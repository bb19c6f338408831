"""``gemm_fp4``: MXFP4 (E2M1, E8M0 scale per 32 elements) GEMM with autograd
(reference: primus_turbo/pytorch/ops/gemm_fp4.py:76-290).

Forward, dgrad and wgrad are all NT products of MX-quantized operands: activations and
gradients use 1 x 32 blocks, the weight 32 x 32 blocks; each tensor is quantized in both
directions from one read. As in the reference's recipe (its lines 108-160, 220-240) the two wgrad
operands -- the column-direction quantizations of ``a`` and of ``grad_out`` -- carry the fixed
16-point Hadamard transform along the token axis, which cancels in their product and spreads
outliers over 16 values before they are quantized; ``use_gradient_sr`` rounds both quantizations of
``grad_out`` stochastically. ``use_preshuffle`` selects, in the reference, the shuffled operand
layouts of AITER's kernel; the kernel here reads plain layouts, so the flag only decides which
layout pre-quantized operands are expected in (they are brought back to the plain one on entry)
and leaves the result unchanged.
"""

from __future__ import annotations

from typing import Optional, Union

import torch

from primus_turbo.pytorch.core.backend import BackendType
from primus_turbo.pytorch.core.low_precision import (
    Float4QuantConfig,
    Format,
    ScalingRecipe,
    check_mxfp4_support,
)
from primus_turbo.pytorch.core.quantized_tensor import (
    QuantizedTensor,
    QuantizedTensorPair,
    check_quantized_tensor,
)
from primus_turbo.pytorch.kernels.gemm.gemm_fp4_impl import gemm_fp4_accum_impl, gemm_fp4_impl
from primus_turbo.pytorch.kernels.quantization.quantization_impl import mx_plain_layout, quantize_mxfp4_impl
from primus_turbo.pytorch.ops.quantization import quantize_fp4_with_trans
from primus_turbo.pytorch.ops.utils import _get_dummy_wgrad, _setup_fused_grad_accum

__all__ = ["gemm_fp4"]

_NATIVE = BackendType.HIPBLASLT.value  # placeholder id: a single backend exists here


def _bgrad_gemm_fp4_impl_wrapper(a, a_s, trans_a, b, b_s, trans_b, out_dtype, trans_c, granularity,
                                 inplace_add_to_out=False, out=None):
    if not inplace_add_to_out:
        return gemm_fp4_impl(a, a_s, trans_a, b, b_s, trans_b, out_dtype, trans_c, granularity, _NATIVE)
    assert out is not None, "out should not be None when inplace_add_to_out is True"
    gemm_fp4_accum_impl(a, a_s, trans_a, b, b_s, trans_b, out.dtype, trans_c, granularity, out, _NATIVE)
    return _get_dummy_wgrad(out.shape, out_dtype)


class FP4GemmMXFunction(torch.autograd.Function):
    @staticmethod
    def get_fp4_dtype(format: Format):
        if format == Format.E2M1_X2:
            return torch.float4_e2m1fn_x2
        raise ValueError(f"Unsupported FP4 format: {format}")

    @staticmethod
    def forward(ctx, a, b, a_t, b_t, trans_a, trans_b, out_dtype, config, fuse_bgrad_accum_pattern=None):
        ok, why = check_mxfp4_support()
        assert ok, why
        pre = config.use_preshuffle
        fuse, main_grad = _setup_fused_grad_accum(b, fuse_bgrad_accum_pattern)
        dt = FP4GemmMXFunction.get_fp4_dtype(config.format)
        gran, bs = config.granularity, config.block_size

        need_bwd = any(ctx.needs_input_grad[:2])

        def both_ways(x, x_t, recipe, recipe_t):
            """Row- and column-direction quantizations in the plain layout. ``recipe`` / ``recipe_t`` are
            what a pre-quantized operand must carry (the reference's recipes, shuffle flags included)."""
            if isinstance(x, QuantizedTensor):
                check_quantized_tensor(x, config, scaling_recipe=recipe)
                if x_t is None:
                    x_t = QuantizedTensor.quantize(x.dequantize(), x.real_dtype, gran, axis=-2, block_size=bs,
                                                   scaling_recipe=recipe_t)
                else:
                    check_quantized_tensor(x_t, config, scaling_recipe=recipe_t)
                q, sc = mx_plain_layout(x.qdata, x.scale_inv, recipe.shuffle_out, recipe.shuffle_scale)
                q_t, sc_t = mx_plain_layout(x_t.qdata, x_t.scale_inv, recipe_t.shuffle_out, recipe_t.shuffle_scale)
                return q, sc, q_t, sc_t
            recipe = recipe._replace(shuffle_out=False, shuffle_scale=False)
            recipe_t = recipe_t._replace(shuffle_out=False, shuffle_scale=False)
            if not need_bwd:
                # the transposed copies only feed backward: skip them when nothing asks for a gradient
                q, sc = quantize_mxfp4_impl(x, dt, x.dim() - 1, bs, scaling_recipe=recipe)
                return q, sc, q, sc
            return quantize_fp4_with_trans(x, dt, gran, block_size=bs, scaling_recipe=recipe,
                                           scaling_recipe_for_trans=recipe_t)

        # reference lines 112-160: the second operand of each product is the one held pre-shuffled
        w_recipe = ScalingRecipe(use_2d_block=True, shuffle_scale=pre, shuffle_out=pre)
        a_row, a_row_s, a_col, a_col_s = both_ways(a, a_t, ScalingRecipe(shuffle_scale=pre),
                                                   ScalingRecipe(use_rht=True, shuffle_scale=pre, shuffle_out=pre))
        b_row, b_row_s, b_col, b_col_s = both_ways(b, b_t, w_recipe, w_recipe)
        out = gemm_fp4_impl(a_row, a_row_s, False, b_row, b_row_s, True, out_dtype, False, gran.value, _NATIVE)
        ctx.save_for_backward(a_col, a_col_s, b_col, b_col_s)
        ctx.meta = (out_dtype, config, fuse, main_grad)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        out_dtype, config, fuse, main_grad = ctx.meta
        a_col, a_col_s, b_col, b_col_s = ctx.saved_tensors
        dt = FP4GemmMXFunction.get_fp4_dtype(config.format)
        gran = config.granularity
        g = grad_out.reshape(grad_out.shape[0], -1).contiguous()
        g_row, g_row_s, g_col, g_col_s = quantize_fp4_with_trans(
            g, dt, gran, block_size=config.block_size, scaling_recipe=ScalingRecipe(use_sr=config.use_gradient_sr),
            scaling_recipe_for_trans=ScalingRecipe(use_sr=config.use_gradient_sr, use_rht=True),  # pairs with a_col
        )
        # both directions are stored transposed, so dgrad and wgrad are NT products as well
        grad_a = gemm_fp4_impl(g_row, g_row_s, False, b_col, b_col_s, True, out_dtype, False, gran.value, _NATIVE)
        grad_b = _bgrad_gemm_fp4_impl_wrapper(g_col, g_col_s, False, a_col, a_col_s, True, out_dtype, False, gran.value,
                                              inplace_add_to_out=fuse, out=main_grad)
        return grad_a, grad_b, None, None, None, None, None, None, None


def gemm_fp4(
    a: Union[torch.Tensor, QuantizedTensor, QuantizedTensorPair],
    b: Union[torch.Tensor, QuantizedTensor, QuantizedTensorPair],
    trans_a: bool = False,
    trans_b: bool = False,
    out_dtype: Optional[torch.dtype] = None,
    config: Optional[Float4QuantConfig] = None,
    fuse_bgrad_accum_pattern: Optional[str] = None,
) -> torch.Tensor:
    """MXFP4 GEMM with autograd: ``a`` is ``(M, K)`` (activation), ``b`` is ``(N, K)`` (weight,
    ``trans_b=True`` is required, as is ``trans_a=False``); ``M``, ``N``, ``K`` multiples of 32.
    Operands may be pre-quantized ``QuantizedTensor`` / ``QuantizedTensorPair``."""
    if config is None:
        config = Float4QuantConfig()
    a_data, a_t = (a.data, a.data_t) if isinstance(a, QuantizedTensorPair) else (a, None)
    b_data, b_t = (b.data, b.data_t) if isinstance(b, QuantizedTensorPair) else (b, None)
    assert a_data.ndim == 2 and b_data.ndim == 2, "Only 2D tensors are supported"
    assert trans_a == False and trans_b == True, "Only NT layout is supported (trans_a=False, trans_b=True)"  # noqa: E712
    if out_dtype is None:
        out_dtype = torch.promote_types(a_data.dtype, b_data.dtype)
    return FP4GemmMXFunction.apply(a_data, b_data, a_t, b_t, trans_a, trans_b, out_dtype, config,
                                   fuse_bgrad_accum_pattern)
