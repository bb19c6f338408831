"""``grouped_gemm_fp4``: MoE grouped GEMM on MXFP4 (E2M1, E8M0 scale per 32 elements) operands with
autograd (reference: primus_turbo/pytorch/ops/grouped_gemm_fp4.py:101-400).

    fwd   : out    = a_row            @ b_row^T           (contract K)
    dgrad : grad_a = grad_out_row     @ b_col^T           (contract N)
    wgrad : grad_b = grad_out_col[g]  @ a_col[g]^T        (contract the group's tokens)

Activations and gradients use 1 x 32 blocks and are quantized in both directions from one read
(rows in place, transposed columns padded to 256 tokens per group); the weight uses 32 x 32
blocks. As in the reference the two wgrad operands (the column-direction quantizations of ``a`` and
``grad_out``) carry the recipe's fixed 16-point Hadamard transform along the token axis, which
cancels in their product; ``use_gradient_sr`` rounds both quantizations of ``grad_out``
stochastically. ``use_preshuffle`` must be off, as in the reference.
"""

from __future__ import annotations

from typing import Optional, Union

import torch

from primus_turbo.pytorch.core.backend import BackendType
from primus_turbo.pytorch.core.low_precision import (
    MXFP4_BLOCK_SIZE,
    Float4QuantConfig,
    ScalingGranularity,
    ScalingRecipe,
    check_mxfp4_support,
    float4_e2m1fn_x2,
)
from primus_turbo.pytorch.core.quantized_tensor import (
    QuantizedTensor,
    QuantizedTensorPair,
    check_quantized_tensor,
)
from primus_turbo.pytorch.kernels.grouped_gemm.grouped_gemm_fp4_impl import (
    grouped_gemm_fp4_impl,
    grouped_gemm_fp4_variable_k_accum_impl,
    grouped_gemm_fp4_variable_k_impl,
)
from primus_turbo.pytorch.kernels.grouped_gemm.grouped_gemm_utils import group_offs_from_lens
from primus_turbo.pytorch.kernels.quantization.quantization_impl import (
    glu_grouped_quantize_mx_impl,
    quantize_mxfp4_impl,
)
from primus_turbo.pytorch.ops.quantization import (
    grouped_quantize_fp4,
    grouped_quantize_fp4_with_trans,
    quantize_fp4_with_trans,
)
from primus_turbo.pytorch.ops.utils import (
    _ensure_contiguous_grad_out,
    _get_dummy_wgrad,
    _setup_fused_grad_accum,
)

__all__ = ["grouped_gemm_fp4", "glu_grouped_gemm_fp4"]

_NATIVE = BackendType.HIPBLASLT.value  # placeholder id: a single backend exists here


def _bgrad_grouped_gemm_fp4_impl_wrapper(a, b, a_scales, b_scales, group_lens, group_offs, trans_a, trans_b, trans_c,
                                         out_dtype, granularity, num_cu, default_backend, inplace_add_to_out=False,
                                         out=None):
    """Variable-K wgrad; with ``inplace_add_to_out`` it accumulates into ``out`` (``main_grad``) and
    hands autograd a dummy of the weight's dtype instead."""
    args = (a, b, a_scales, b_scales, group_lens, group_offs, trans_a, trans_b, trans_c, out_dtype, granularity, num_cu,
            default_backend)
    if not inplace_add_to_out:
        return grouped_gemm_fp4_variable_k_impl(*args)
    assert out is not None, "out should not be None when inplace_add_to_out is True"
    grouped_gemm_fp4_variable_k_accum_impl(*args, out)
    return _get_dummy_wgrad(out.shape, out_dtype)


def _fp4_weight_operands(b, b_t, config, need_bwd):
    """The expert weights ``[G, N, K]`` as MXFP4 operands with 32 x 32 blocks: ``(row codes, row scales,
    column codes, column scales)``, the column pair (the transposed quantization dgrad reads) only
    when a backward pass will follow."""
    gran, bs = config.granularity, config.block_size
    w_recipe = ScalingRecipe(use_2d_block=True)
    b_col = b_col_s = None
    if isinstance(b, QuantizedTensor):
        check_quantized_tensor(b, config, axis=-1, scaling_recipe=w_recipe)
        b_row, b_row_s = b.qdata, b.scale_inv
        if need_bwd:
            if b_t is None:
                b_t = QuantizedTensor.quantize(b.dequantize(), b.real_dtype, gran, axis=-2, block_size=bs,
                                               scaling_recipe=w_recipe)
            assert isinstance(b_t, QuantizedTensor)
            b_col, b_col_s = b_t.qdata, b_t.scale_inv
    elif need_bwd:
        b_row, b_row_s, b_col, b_col_s = quantize_fp4_with_trans(
            b.contiguous(), float4_e2m1fn_x2, gran, block_size=bs, scaling_recipe=w_recipe,
            scaling_recipe_for_trans=w_recipe)
    else:
        b_row, b_row_s = quantize_mxfp4_impl(b.contiguous(), float4_e2m1fn_x2, 2, bs, scaling_recipe=w_recipe)
    return b_row, b_row_s, b_col, b_col_s


def _fp4_backward_products(grad_out, a_col, a_col_s, b_col, b_col_s, group_lens, group_offs, config, dgrad_dtype,
                           wgrad_dtype, num_cu, total_m, fuse_bgrad_accum, main_grad):
    """dgrad and wgrad of the MXFP4 grouped product from the saved column-direction operands."""
    gran = config.granularity
    g_row, g_row_s, g_col, g_col_s, _, offs_row, lens_col, offs_col = grouped_quantize_fp4_with_trans(
        grad_out, float4_e2m1fn_x2, gran, group_lens, group_offs, block_size=config.block_size,
        scaling_recipe=ScalingRecipe(use_sr=config.use_gradient_sr),
        scaling_recipe_for_trans=ScalingRecipe(use_sr=config.use_gradient_sr, use_rht=True))
    # dgrad: grad_a = grad_out @ b as an NT product with the transposed weight quantization [G, K, N]
    grad_a = grouped_gemm_fp4_impl(g_row, b_col, g_row_s, b_col_s, group_lens, offs_row, False, True, dgrad_dtype,
                                   gran.value, num_cu, _NATIVE, False, group_offs)[:total_m]
    # wgrad: grad_b[g] = grad_out_g^T @ a_g over the 256-padded token ranges -> [G, N, K]
    grad_b = _bgrad_grouped_gemm_fp4_impl_wrapper(
        g_col, a_col, g_col_s, a_col_s, lens_col, offs_col, False, False, False, wgrad_dtype, gran.value, num_cu,
        _NATIVE, inplace_add_to_out=fuse_bgrad_accum, out=main_grad)
    return grad_a, grad_b


class FP4GroupedGemmMXFunc(torch.autograd.Function):
    """MXFP4 grouped GEMM autograd (MX_BLOCKWISE, NT only)."""

    @staticmethod
    def forward(ctx, a, b, a_t, b_t, group_lens, group_offs, trans_b, out_dtype, config, num_cu,
                fuse_bgrad_accum_pattern=None):
        fuse_bgrad_accum, main_grad = _setup_fused_grad_accum(b, fuse_bgrad_accum_pattern)
        assert config.granularity == ScalingGranularity.MX_BLOCKWISE
        assert a.ndim == 2 and b.ndim == 3
        assert out_dtype in (torch.float16, torch.bfloat16)
        assert trans_b, "MXFP4 grouped GEMM only supports trans_b=True (NT layout)."
        # as the reference (its line 126): the grouped product has no pre-shuffled form
        assert not config.use_preshuffle, "MXFP4 grouped GEMM does not use preshuffle."
        supported, reason = check_mxfp4_support()
        assert supported, reason
        N, K = int(b.shape[-2]), int(b.shape[-1])
        assert K % MXFP4_BLOCK_SIZE == 0, f"K must be a multiple of {MXFP4_BLOCK_SIZE} (got {K})."
        assert N % MXFP4_BLOCK_SIZE == 0, f"N must be a multiple of {MXFP4_BLOCK_SIZE} (got {N})."
        assert group_lens.size(0) == b.size(0), "group_lens size must match b size(0)."
        total_m = int(a.size(0))
        gran, bs = config.granularity, config.block_size
        need_bwd = any(ctx.needs_input_grad[:2])
        a_recipe, a_t_recipe = ScalingRecipe(), ScalingRecipe(use_rht=True)
        if isinstance(a, QuantizedTensor):
            # a grouped (packed rows) quantization made by the caller
            check_quantized_tensor(a, config, axis=-1, scaling_recipe=a_recipe)
            a_row, a_row_s, offs_row = a.qdata, a.scale_inv, a.group_offs
            a_col = a_col_s = None
            if need_bwd:
                if a_t is None:
                    a_t = QuantizedTensor.quantize(a.dequantize(), a.real_dtype, gran, axis=-2, block_size=bs,
                                                   scaling_recipe=a_t_recipe, group_lens=group_lens)
                assert isinstance(a_t, QuantizedTensor)
                check_quantized_tensor(a_t, config, scaling_recipe=a_t_recipe)
                a_col, a_col_s = a_t.qdata, a_t.scale_inv
        elif need_bwd:
            a_row, a_row_s, a_col, a_col_s, _, offs_row, _, _ = grouped_quantize_fp4_with_trans(
                a.contiguous(), float4_e2m1fn_x2, gran, group_lens, group_offs, block_size=bs,
                scaling_recipe=a_recipe, scaling_recipe_for_trans=a_t_recipe)
        else:
            a_row, a_row_s, _, offs_row = grouped_quantize_fp4(
                a.contiguous(), float4_e2m1fn_x2, gran, group_lens, group_offs, block_size=bs, axis=1)
            a_col = a_col_s = None

        b_row, b_row_s, b_col, b_col_s = _fp4_weight_operands(b, b_t, config, need_bwd)

        out = grouped_gemm_fp4_impl(a_row, b_row, a_row_s, b_row_s, group_lens, offs_row, False, True, out_dtype,
                                    gran.value, num_cu, _NATIVE, False, group_offs)[:total_m]
        if need_bwd:
            ctx.save_for_backward(a_col, a_col_s, b_col, b_col_s, group_lens, group_offs)
        ctx.meta = (config, out_dtype, num_cu, total_m, fuse_bgrad_accum, main_grad)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        grad_out = _ensure_contiguous_grad_out(grad_out)
        a_col, a_col_s, b_col, b_col_s, group_lens, group_offs = ctx.saved_tensors
        config, out_dtype, num_cu, total_m, fuse_bgrad_accum, main_grad = ctx.meta
        grad_a, grad_b = _fp4_backward_products(grad_out, a_col, a_col_s, b_col, b_col_s, group_lens, group_offs, config,
                                                out_dtype, out_dtype, num_cu, total_m, fuse_bgrad_accum, main_grad)
        return grad_a, grad_b, None, None, None, None, None, None, None, None, None


class FP4GluGroupedGemmMXFunc(torch.autograd.Function):
    """Gated activation -> MXFP4 grouped GEMM (fc2 of an MoE expert MLP) with the activation fused
    into the grouped quantizer of the GEMM's activation operand (rows as they are, transposed
    columns Hadamard-transformed for wgrad): the bf16 activation is neither written nor re-read."""

    @staticmethod
    def forward(ctx, x, probs, row_mask, act_type, b, group_lens, group_offs, trans_b, out_dtype, config, num_cu,
                fuse_bgrad_accum_pattern=None):
        fuse_bgrad_accum, main_grad = _setup_fused_grad_accum(b, fuse_bgrad_accum_pattern)
        assert config.granularity == ScalingGranularity.MX_BLOCKWISE and config.block_size == MXFP4_BLOCK_SIZE
        assert x.ndim == 2 and x.size(1) % 2 == 0, "x must be [tokens, 2 * hidden]"
        assert b.ndim == 3 and out_dtype in (torch.float16, torch.bfloat16)
        assert trans_b, "MXFP4 grouped GEMM only supports trans_b=True (NT layout)."
        assert not config.use_preshuffle, "MXFP4 grouped GEMM does not use preshuffle."
        supported, reason = check_mxfp4_support()
        assert supported, reason
        N, K = int(b.shape[-2]), int(b.shape[-1])
        assert K % MXFP4_BLOCK_SIZE == 0 and N % MXFP4_BLOCK_SIZE == 0, "N and K must be multiples of 32"
        assert K == x.size(1) // 2, "x must hold 2 * K columns"
        assert group_lens.size(0) == b.size(0), "group_lens size must match b size(0)."
        assert probs.dtype == torch.float32 and probs.numel() == x.size(0), "probs must be float32, one per token"
        total_m = int(x.size(0))
        need_bwd = any(ctx.needs_input_grad[i] for i in (0, 1, 4))
        x2, p1 = x.contiguous(), probs.reshape(-1).contiguous()
        a_row, a_row_s, a_col, a_col_s, _, _, _, _ = glu_grouped_quantize_mx_impl(
            x2, p1, row_mask, act_type, float4_e2m1fn_x2, group_lens, group_offs, need_bwd, 2)
        b_row, b_row_s, b_col, b_col_s = _fp4_weight_operands(b, None, config, need_bwd)
        out = grouped_gemm_fp4_impl(a_row, b_row, a_row_s, b_row_s, group_lens, group_offs, False, True, out_dtype,
                                    config.granularity.value, num_cu, _NATIVE, False, group_offs)[:total_m]
        if need_bwd:
            ctx.save_for_backward(x2, p1, row_mask, a_col, a_col_s, b_col, b_col_s, group_lens, group_offs)
        ctx.meta = (config, out_dtype, num_cu, total_m, fuse_bgrad_accum, main_grad, act_type, probs.shape)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        from primus_turbo.pytorch.kernels.activation.glu_impl import ACT_GELU, ACT_SILU, glu_bwd_with_probs

        grad_out = _ensure_contiguous_grad_out(grad_out)
        x2, p1, row_mask, a_col, a_col_s, b_col, b_col_s, group_lens, group_offs = ctx.saved_tensors
        config, out_dtype, num_cu, total_m, fuse_bgrad_accum, main_grad, act_type, probs_shape = ctx.meta
        grad_act, grad_b = _fp4_backward_products(grad_out, a_col, a_col_s, b_col, b_col_s, group_lens, group_offs, config,
                                                  x2.dtype, out_dtype, num_cu, total_m, fuse_bgrad_accum, main_grad)
        grad_x, grad_probs = glu_bwd_with_probs(grad_act.contiguous(), x2, p1, row_mask,
                                                ACT_SILU if act_type == "silu" else ACT_GELU)
        return grad_x, grad_probs.view(probs_shape), None, None, grad_b, None, None, None, None, None, None, None


def grouped_gemm_fp4(
    a: Union[torch.Tensor, QuantizedTensor, QuantizedTensorPair],
    b: Union[torch.Tensor, QuantizedTensor, QuantizedTensorPair],
    group_lens: torch.Tensor,
    group_offs: Optional[torch.Tensor] = None,
    trans_b: bool = True,
    out_dtype: Optional[torch.dtype] = None,
    config: Optional[Float4QuantConfig] = None,
    num_cu: Optional[int] = None,
    fuse_bgrad_accum_pattern: Optional[str] = None,
) -> torch.Tensor:
    """Grouped GEMM with MXFP4 quantization: ``out[rows of group g] = a[rows of group g] @ b[g]^T``.

    ``a``: ``[sum(group_lens), K]`` (fp16 / bf16), or a grouped ``QuantizedTensor`` / pair (``data_t`` =
    the column-direction quantization that wgrad reads); ``b``: ``[G, N, K]`` (``trans_b`` must be
    True), or a pre-quantized 32 x 32-block ``QuantizedTensor`` / ``QuantizedTensorPair`` (``data_t`` =
    the transposed quantization that dgrad reads); ``group_lens``: int64 ``[G]`` on the device
    (groups may be empty); N and K multiples of 32. ``fuse_bgrad_accum_pattern="megatron"``
    accumulates the weight gradient into ``b.main_grad`` (any of fp32 / bf16 / fp16)."""
    if config is None:
        config = Float4QuantConfig()
    if group_offs is None:
        group_offs = group_offs_from_lens(group_lens)
    a_data, a_data_t = (a.data, a.data_t) if isinstance(a, QuantizedTensorPair) else (a, None)
    b_data, b_data_t = (b.data, b.data_t) if isinstance(b, QuantizedTensorPair) else (b, None)
    if out_dtype is None:
        out_dtype = torch.promote_types(a_data.dtype, b_data.dtype)
    assert a_data.ndim == 2, "a must be 2D [total_m, K]"
    assert b_data.ndim == 3, "b must be 3D [G, N, K]"
    if config.granularity == ScalingGranularity.MX_BLOCKWISE:
        return FP4GroupedGemmMXFunc.apply(a_data, b_data, a_data_t, b_data_t, group_lens, group_offs, trans_b,
                                          out_dtype, config, num_cu, fuse_bgrad_accum_pattern)
    raise ValueError(f"Unsupported FP4 ScalingGranularity: {config.granularity}")


def glu_grouped_gemm_fp4(
    x: torch.Tensor,
    probs: torch.Tensor,
    b: Union[torch.Tensor, QuantizedTensor],
    group_lens: torch.Tensor,
    group_offs: Optional[torch.Tensor] = None,
    trans_b: bool = True,
    out_dtype: Optional[torch.dtype] = None,
    config: Optional[Float4QuantConfig] = None,
    num_cu: Optional[int] = None,
    row_mask: Optional[torch.Tensor] = None,
    act_type: str = "silu",
    fuse_bgrad_accum_pattern: Optional[str] = None,
) -> torch.Tensor:
    """``grouped_gemm_fp4(swiglu_with_probs(x, probs, row_mask), b, group_lens, ...)`` (``act_type="gelu"``:
    ``geglu_with_probs``) as one operation: fc1's output ``x [tokens, 2 K]`` is read once by a grouped
    MXFP4 quantizer that applies the gated activation on load, so the bf16 activation never goes
    through HBM; results and gradients are bit-identical with the two-step form. (The reference has
    the two steps only: ops/activation.py:21-83, ops/grouped_gemm_fp4.py:101-400.)"""
    if config is None:
        config = Float4QuantConfig()
    if config.granularity != ScalingGranularity.MX_BLOCKWISE:
        raise ValueError(f"Unsupported FP4 ScalingGranularity: {config.granularity}")
    assert act_type in ("silu", "gelu"), f"Unsupported act_type: {act_type}"
    if group_offs is None:
        group_offs = group_offs_from_lens(group_lens)
    if out_dtype is None:
        out_dtype = torch.promote_types(x.dtype, b.dtype)
    return FP4GluGroupedGemmMXFunc.apply(x, probs, row_mask, act_type, b, group_lens, group_offs, trans_b, out_dtype, config,
                                         num_cu, fuse_bgrad_accum_pattern)
